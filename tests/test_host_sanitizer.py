"""The host side of the C-ABI library under UndefinedBehaviorSanitizer (host code only; the device code is compiled as usual).

The library is rebuilt with ``-Xarch_host -fsanitize=undefined -Xarch_host -fsanitize-trap=undefined`` into a temporary
directory and a child process drives every host path that needs no GPU -- workspace queries, the chunk-width model and
the argument checks of all entry points -- over a sweep that includes sizes at and beyond the 32-bit limits.  Undefined
behaviour (a signed overflow in a size computation, a bad shift) traps and kills the child.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
import textwrap

import pytest

from skyrl_amd.csrc import build as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.skipif(
    not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")), reason="hipcc not available"
)

DRIVER = textwrap.dedent("""
    import ctypes, itertools, sys
    sys.path.insert(0, sys.argv[2])
    from skyrl_amd import _lib
    lib = ctypes.CDLL(sys.argv[1])
    for name, (res, args) in _lib.SIGNATURES.items():
        f = getattr(lib, name); f.restype = res; f.argtypes = args
    assert lib.skyrl_lmhead_version() == _lib.ABI_VERSION
    big = (1, 63, 300, 16384, 1 << 20, (1 << 31) - 1, 1 << 31, 1 << 40)
    for T, H, V, vc in itertools.product(big, (64, 896, 3584, 1 << 20), (5, 1000, 152064, 1 << 31, 1 << 40), (0, 256, 49152, 1 << 40)):
        lib.skyrl_lmhead_fwd_workspace_bytes(T, H, V); lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, vc)
        lib.skyrl_softce_fwd_workspace_bytes(T, H, V); lib.skyrl_softce_bwd_workspace_bytes(T, H, V, vc)
        lib.skyrl_lmhead_bwd_active_rows_workspace_bytes(T, H, V, vc)
        for terms in (1, 2, 3, 1 << 40): lib.skyrl_lmhead_bwd_split_workspace_bytes(T, H, terms, V, vc, 1)
        for k in (1, 32, 1024, 1025, 1 << 40): lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, k)
    p = 0x10000
    for T, H, V in itertools.product(big, (64, 3584, 1 << 20), (5, 152064, 1 << 31, 1 << 40)):
        ld = H
        assert lib.skyrl_lmhead_fwd(p, ld, p, ld, p, T, H, V, 1.0, p, None, None, None, p, 16, None) < 0
        assert lib.skyrl_lmhead_bwd(p, ld, p, ld, p, p, None, p, None, T, H, V, 1.0, p, p, 0, 0, p, 16, None) < 0
        assert lib.skyrl_lmhead_bwd_active_rows(p, ld, p, ld, p, p, None, p, None, T, H, V, 1.0, p, p, 0, 0, p, 16, None) < 0
        assert lib.skyrl_lmhead_bwd_split(p, 3 * ld, p, 3 * ld, p, p, None, p, None, T, H, 3, V, 1.0, p, p, 0, 0, 1, p, 16, None) < 0
        assert lib.skyrl_lmhead_fwd_static_scratch(p, ld, p, ld, p, T, H, V, float("nan"), p, None, None, None, None) < 0
        assert lib.skyrl_lmhead_split_operand(p, 1, ld, T, H, 3, p, 2 * ld, None) < 0
        assert lib.skyrl_softce_fwd(p, ld, p, ld, p, ld, T, T, 1, H, V, 1.0, p, p, p, p, 16, None) < 0
        assert lib.skyrl_softce_bwd(p, ld, p, ld, p, ld, p, p, p, T, T, 1, H, V, 1.0, p, 0, p, 16, None) < 0
        for k in (1, 5, 1 << 40):
            assert lib.skyrl_lmhead_topk_logits(p, ld, p, ld, T, H, V, k, 1.0, p, p, p, 16, None) < 0
            assert lib.skyrl_softce_topk_fwd(p, ld, p, ld, p, p, T, 0, 1, H, V, k, 1.0, p, p, p, None) < 0
            assert lib.skyrl_softce_topk_bwd(p, ld, p, p, p, T, H, V, k, 1.0, p, 0, None) < 0
    for T, V, ld in itertools.product(big, (1, 152064, (1 << 31) - 1, 1 << 31, 1 << 40), (0, 152064, 1 << 40, 1 << 62)):
        assert lib.skyrl_logits_fwd(p, 7, ld, p, T, V, 1.0, p, None, None, None, None) < 0
        assert lib.skyrl_logits_fwd(p + 1, 0, ld, p, T, V, 1.0, p, None, None, None, None) < 0
        assert lib.skyrl_logits_bwd(p, 1, ld, p, p, None, p, None, T, V, 1.0, p + 2, ld, None) < 0
    assert lib.skyrl_ppo_policy_loss(p, p, p, None, None, 0, 0.2, 0.2, 3.0, 0, p, None, None, None) < 0
    for rows, cols in itertools.product((0, 1 << 31, 1 << 40), (0, 5, 1 << 41)):
        assert lib.skyrl_off_policy_correction(p, p, None, rows, cols, 1, 2.0, 0, 0.0, 0.0, None, None, None, None, p, p, p, p, p, None) < 0
    assert lib.skyrl_off_policy_correction(p, p, None, 4, 4, 3, 2.0, 0, 0.0, 0.0, None, None, None, None, p, p, p, p, p, None) < 0
    assert lib.skyrl_off_policy_correction(p, p, None, 4, 4, 1, float("inf"), 0, 0.0, 0.0, None, None, None, None, p, p, p, p, p, None) < 0
    assert lib.skyrl_off_policy_correction(p, p, None, 4, 4, 0, 0.0, 0, 0.0, 0.0, None, None, None, None, p, p, p, None, p, None) < 0
    assert lib.skyrl_actor_loss(p, p, p, None, None, None, None, 1 << 40, 1 << 40, 0, 0.2, 0.2, 3.0, 3, 1.0, 1.0, 0.0, 0.0, p, p,
                                None, None, None) < 0
    assert lib.skyrl_approx_kl(p, p, None, 1 << 40, 4, 3, None, p, p, 0, None, None) < 0
    for n, out, part in ((0, p, p), (-1, p, p), (16, None, p), (16, p, None)):
        assert lib.skyrl_logprob_diff_metrics(p, p, None, n, out, part, None) < 0
    assert lib.skyrl_masked_mean(p, None, 1 << 40, 4, p, None, None) < 0
    assert lib.skyrl_actor_loss(p, p, p, None, None, None, p, 1 << 30, 1 << 40, 0, 0.2, 0.2, 3.0, 3, 1.0, 1.0, 0.0, 0.0, p, p,
                                None, p, None) < 0
    assert lib.skyrl_packed_next_token_labels(p, p, 3, 1 << 62, p, None) < 0
    assert lib.skyrl_packed_scatter_logprobs(p, p, 3, 1 << 62, None, None, None, None, 3, 5, p, None) < 0
    assert lib.skyrl_packed_gather_grad(p, p, 3, 8, None, None, None, None, 1 << 40, 1 << 40, p, None) < 0
    print("host paths clean")
""")


def test_host_code_has_no_undefined_behaviour(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    lib = tmp_path / "libskyrl_lmhead_ubsan.so"
    flags = [f for f in B.HIPCC_FLAGS if f != "-O3"] + ["-O1", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
                                                         "-fsanitize-trap=undefined"]
    cmd = [hipcc, *flags, "-o", str(lib), *[os.path.join(B.HERE, s) for s in B.SOURCES]]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    run = subprocess.run([sys.executable, "-c", DRIVER, str(lib), ROOT], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and "host paths clean" in run.stdout, (run.returncode, run.stdout[-500:], run.stderr[-2000:])

"""Checks on the generated gfx950 code of the MFMA kernels (no GPU needed: hipcc cross-compiles to assembly).

The mainloop issues its MFMAs as inline assembly (``gemm_core.hpp: mfma_16x16x32``), so the compiler neither pads the
MFMA -> accumulator-read hazard nor knows that the accumulators must stay where they are.  These tests read the assembly of
every kernel that contains MFMAs and check the properties the source relies on:

* every ``v_accvgpr_read`` comes after the explicit wait states that follow the last MFMA before it, and no
  ``v_accvgpr_write`` sits right in front of an MFMA;
* every MFMA accumulates in place, in AGPRs (no rotation of accumulators through the loop);
* the steady-state loop (the block with MFMAs and global->LDS copies) has no scratch (spill) traffic and no accumulator moves.
"""

from __future__ import annotations

import os
import re
import shutil
import subprocess

import pytest

from skyrl_amd.csrc import build as B

pytestmark = pytest.mark.skipif(
    not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")), reason="hipcc not available"
)


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = tmp_path_factory.mktemp("isa") / "lmhead.s"
    flags = [f for f in B.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [hipcc, *flags, "-S", "--cuda-device-only", "-o", str(out), os.path.join(B.HERE, B.SOURCES[0])]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    text = out.read_text()
    found = {}
    for m in re.finditer(r"^(_Z\w+):", text, re.M):
        name = m.group(1)
        end = text.find(".end_amdhsa_kernel", m.end())
        nxt = text.find("\n_Z", m.end())
        body = text[m.end(): end if end != -1 else None]
        if nxt != -1 and nxt < end:
            continue  # a device function label, not a kernel body
        lines = [ln.strip() for ln in body.split("\n") if ln.strip() and not ln.strip().startswith(";")]
        if any(ln.startswith("v_mfma") for ln in lines):
            found[name] = lines
    return found


def test_mfma_kernels_found(kernels):
    names = " ".join(kernels)
    for expect in ("lmhead_fwd_tiles", "lmhead_bwd_dz", "lmhead_bwd_gemm", "mfma_probe"):
        assert expect in names, f"no MFMA kernel named *{expect}* in the assembly: {list(kernels)}"


def test_accumulator_reads_follow_the_wait_states(kernels):
    for name, lines in kernels.items():
        waited = False
        for ln in lines:
            if ln.startswith("v_mfma"):
                waited = False
            elif ln.startswith("s_nop 15"):
                waited = True
            elif ln.startswith("v_accvgpr_read"):
                assert waited, f"{name}: '{ln}' is not behind the wait states that follow the last MFMA"


def test_no_accumulator_write_right_before_an_mfma(kernels):
    for name, lines in kernels.items():
        for k, ln in enumerate(lines):
            if ln.startswith("v_mfma"):
                near = [p for p in lines[max(0, k - 3):k] if p.startswith("v_accvgpr_write")]
                assert not near, f"{name}: {near[0]} within three instructions of '{ln}'"


def test_every_lds_copy_sets_m0_first(kernels):
    """global_load_lds takes its LDS destination from M0: each one must be preceded, within a few instructions and with no
    other copy in between, by a write of M0."""
    for name, lines in kernels.items():
        for k, ln in enumerate(lines):
            if ln.startswith("global_load_lds"):
                window = lines[max(0, k - 4):k]
                writes = [i for i, p in enumerate(window) if re.match(r"s_(mov_b32|add_i32|add_u32) m0,", p)]
                assert writes, f"{name}: no M0 write right before '{ln}': {window}"
                assert not any(p.startswith("global_load_lds") for p in window[writes[-1]:]), f"{name}: stale M0 before '{ln}'"


def test_no_packed_fp32_arithmetic(kernels):
    """The build switches the packed fp32 instructions off (``-packed-fp32-ops``); none may appear in the MFMA kernels."""
    for name, lines in kernels.items():
        bad = [ln for ln in lines if ln.startswith(("v_pk_add_f32", "v_pk_mul_f32", "v_pk_fma_f32"))]
        assert not bad, f"{name}: {bad[:3]}"


def test_mfma_accumulates_in_place_in_agprs(kernels):
    pat = re.compile(r"v_mfma_f32_16x16x32_bf16 (a\[\d+:\d+\]), v\[\d+:\d+\], v\[\d+:\d+\], (a\[\d+:\d+\])$")
    for name, lines in kernels.items():
        for ln in lines:
            if ln.startswith("v_mfma"):
                m = pat.match(ln)
                assert m and m.group(1) == m.group(2), f"{name}: unexpected MFMA form '{ln}'"


def test_steady_state_loop_is_clean(kernels):
    for name, lines in kernels.items():
        # split into basic blocks at labels
        blocks, cur = [], []
        for ln in lines:
            if re.match(r"^\.LBB\w+:", ln):
                blocks.append(cur)
                cur = []
            cur.append(ln)
        blocks.append(cur)
        matched = 0
        for b in blocks:
            n_mfma = sum(ln.startswith("v_mfma") for ln in b)
            n_copy = sum(ln.startswith("global_load_lds") for ln in b)
            if n_mfma and n_mfma % 128 == 0 and n_copy * 8 == n_mfma:  # steady-state k-tile steps: 16 copies per 128 MFMAs
                matched += 1
                bad = [ln for ln in b if ln.startswith(("scratch_", "v_accvgpr_"))]
                assert not bad, f"{name}: steady-state loop has spill / accumulator traffic: {bad[:4]}"
        if any(ln.startswith("global_load_lds") for ln in lines):
            assert matched >= 1, f"{name}: no steady-state loop block recognised"


def test_even_kernels_issue_both_k_steps_of_an_accumulator_back_to_back(kernels):
    """The accumulator-stationary mainloop (gemm_core.hpp: mainloop_pairs) is what the EVEN instantiations and the gradient
    GEMMs run: in their steady-state loop every MFMA shares its accumulator with the MFMA before or after it.  The k-step
    mainloop of the other instantiations never repeats an accumulator within a step."""
    acc = re.compile(r"v_mfma_f32_16x16x32_bf16 (a\[\d+:\d+\])")
    seen_pairs = seen_ksteps = 0
    for name, lines in kernels.items():
        blocks, cur = [], []
        for ln in lines:
            if re.match(r"^\.LBB\w+:", ln):
                blocks.append(cur)
                cur = []
            cur.append(ln)
        blocks.append(cur)
        for b in blocks:
            regs = [acc.match(ln).group(1) for ln in b if ln.startswith("v_mfma")]
            n_copy = sum(ln.startswith("global_load_lds") for ln in b)
            if not regs or len(regs) % 128 or n_copy * 8 != len(regs):
                continue  # not a steady-state loop body
            paired = sum(1 for k in range(0, len(regs) - 1, 2) if regs[k] == regs[k + 1])
            if len(regs) == 256:      # two k-tiles per body: the pairs loop
                assert paired == 128, f"{name}: {paired} of 128 accumulator pairs in the steady-state loop"
                seen_pairs += 1
            else:                     # one k-tile per body: the k-step loop
                assert paired == 0, f"{name}: the k-step loop repeats an accumulator"
                seen_ksteps += 1
    assert seen_pairs >= 3 and seen_ksteps >= 2, (seen_pairs, seen_ksteps)


def test_nothing_waits_on_memory_before_the_first_copy(kernels):
    """A tile's first global -> LDS copies must leave before anything waits for a vector-memory load: per-token inputs of
    the epilogues are issued in front of them as unconditional loads and first used behind the mainloop.  (Loaded under a
    `t < T` condition they become branches with a wait each -- several memory round trips at the head of every tile.)"""
    checked = 0
    for name, lines in kernels.items():
        if not any(k in name for k in ("fwd_tiles", "bwd_dz", "bwd_gemm", "dz_tiles", "filter_tiles")):
            continue
        first = next(i for i, ln in enumerate(lines) if ln.startswith("global_load_lds_dwordx4"))
        head = lines[:first]
        waits = [ln for ln in head if ln.startswith("s_waitcnt") and "vmcnt" in ln]
        assert not waits, f"{name}: {waits[:3]} before the first copy"
        if "bwd_dz" in name or "dz_tiles" in name or "filter_tiles" in name:
            assert any(ln.startswith("global_load_dword") for ln in head), f"{name}: per-token loads not in front of the copies"
        checked += 1
    assert checked >= 8

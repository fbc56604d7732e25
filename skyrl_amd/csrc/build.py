"""Build the C-ABI shared library of the fused LM-head path for gfx950 with hipcc.

Usage: ``python -m skyrl_amd.csrc.build`` (or ``build()`` from Python).  The library is written next to the sources as
``libskyrl_lmhead.so``; nothing is installed outside the source tree.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libskyrl_lmhead.so"
SOURCES = ["lmhead_kernels.hip", "packed_kernels.hip", "loss_kernels.hip", "logits_kernels.hip"]
# -packed-fp32-ops off: the compiler must not form v_pk_{add,mul,fma}_f32 from the scalar fp32 epilogue code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",  # the copy instruction names M0 as clobbered; clang warns that M0 is a reserved register
]


def lib_path() -> str:
    return os.path.join(HERE, LIB_NAME)


def build(verbose: bool = False, extra_flags=(), out: str | None = None) -> str:
    """Compile the library.  ``extra_flags`` / ``out``: a variant build (the timing-only ablations of
    ``skyrl_amd/bench_ablations.py``) written somewhere else than the product library."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found: the fused LM-head library can only be built with the ROCm toolchain")
    out = out or lib_path()
    # Compile into a temporary name and rename, so a failed build never leaves a half-written library behind.
    fd, tmp = tempfile.mkstemp(suffix=".so", dir=os.path.dirname(out) or ".")
    os.close(fd)
    cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-o", tmp, *[os.path.join(HERE, s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        os.unlink(tmp)
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, out)
    os.chmod(out, 0o755)
    return out


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))

"""Where the time of a step goes, and what bounds it: timing-only ablations of the MFMA kernels on one MI355X.

    python -m skyrl_amd.bench_ablations --build          # on any machine with hipcc: compile the variant libraries
    python -m skyrl_amd.bench_ablations [--config NAME] [--rounds R] [--steps K]      # on the GPU box: time them

Every variant is the product source compiled with one ``-DLMHEAD_ABLATE=<bit>`` (``skyrl_amd/csrc/lmhead_kernels.hip``): a
piece of a kernel is left out, the results of that kernel are wrong, and what is read off is only how long the kernel takes
without the piece.  The forward and the dz launches of a variant are always fed row statistics from the unmodified library,
so that the data every other kernel sees stay what they are in the product.  Variants alternate inside every round (same
box, same thermal state).  Around the table the script also prints what else is needed to judge it: the board power while
the product steps run against the board's cap, the matrix pipe's own rate on random and on zero operands, the vendor
library's GEMM on the same operands, the product step with the backward's tiny-probability flush, the board power by kind of
work (idle, matrix pipe alone, HBM copy alone, forward launches, backward launches), and the duration of the fp32 atomic adds
alone that a fully fused backward would issue.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

from . import _lib
from .csrc import build as B

VARIANT_DIR = os.path.join(B.HERE, "ablations")
_ALL = ("lmhead_fwd_tiles", "lmhead_bwd_dz", "lmhead_bwd_gemm")
VARIANTS = [
    # name, LMHEAD_ABLATE, the kernels whose time the variant changes, what is left out
    ("product", 0, (), "nothing"),
    ("fwd_no_epilogue", 1, ("lmhead_fwd_tiles",), "the forward's statistics epilogue (max, exp, sums, partial stores)"),
    ("dz_no_epilogue", 2, ("lmhead_bwd_dz",), "the dz arithmetic, its staging through LDS and the panel stores"),
    ("dz_no_stores", 4, ("lmhead_bwd_dz",), "the global stores of the dz panel (arithmetic and staging stay)"),
    ("l2_only_fwd_dz", 8, ("lmhead_fwd_tiles", "lmhead_bwd_dz"), "operand traffic beyond L2: every tile reads one 4 x 8 patch of tiles"),
    ("l2_only_gemm", 16, ("lmhead_bwd_gemm",), "the same for the gradient-GEMM tiles"),
    # what the mainloop's energy goes into (the launches are power-limited: time is energy)
    ("no_epilogues", 1 | 2, ("lmhead_fwd_tiles", "lmhead_bwd_dz"), "both epilogues: the three mainloops alone"),
    ("mainloops_no_lds_reads", 1 | 2 | 32, _ALL, "epilogues, and every fragment read from LDS inside the k loop"),
    ("mainloops_no_copies", 1 | 2 | 64, _ALL, "epilogues, and every global -> LDS copy behind the first two k-tiles"),
    ("mainloops_mfma_only", 1 | 2 | 32 | 64, _ALL, "epilogues, fragment reads and copies: the MFMAs of the k loop alone"),
]


def variant_path(name: str) -> str:
    return os.path.join(VARIANT_DIR, f"libskyrl_lmhead_{name}.so")


def build_variants(verbose: bool = True) -> None:
    os.makedirs(VARIANT_DIR, exist_ok=True)
    for name, bits, _, _ in VARIANTS:
        out = variant_path(name)
        B.build(verbose=verbose, extra_flags=[f"-DLMHEAD_ABLATE={bits}"], out=out)
        print(f"built {out}", flush=True)


def load_variant(path: str):
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in _lib.SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, argtypes
    return lib


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--build", action="store_true", help="compile the variant libraries and exit")
    ap.add_argument("--config", default="qwen2.5-7b-fwdbwd")
    ap.add_argument("--rounds", type=int, default=5)
    ap.add_argument("--steps", type=int, default=3)
    args = ap.parse_args()
    if args.build:
        build_variants()
        return 0

    import torch

    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if repo not in sys.path:
        sys.path.insert(0, repo)
    import bench as bench_py  # the extra legs of the benchmark line: power, vendor GEMM, matrix-pipe probe
    from .bench_inputs import CONFIGS, make_inputs
    from . import ops

    missing = [n for n, _, _, _ in VARIANTS if not os.path.exists(variant_path(n))]
    if missing:
        print(f"variant libraries missing: {missing}; run `python -m skyrl_amd.bench_ablations --build` first", file=sys.stderr)
        return 2
    cfg = CONFIGS[args.config]
    if not cfg.backward:
        print("the ablations are of a forward + backward step", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    d = make_inputs(cfg)
    T, H, V = cfg.T, cfg.H, cfg.V
    rt = 1.0 / cfg.temperature
    h, w, y = d["hidden"].to(dev), d["weight"].to(dev), d["labels"].to(dev)
    g = d["dlogprobs"].to(dev)
    q = d["dentropy"].to(dev) if cfg.entropy_grad else None
    f32 = dict(dtype=torch.float32, device=dev)
    lse, pz, lp, ent = (torch.empty(T, **f32) for _ in range(4))
    junk = [torch.empty(T, **f32) for _ in range(4)]       # forward outputs of the variants
    dh = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    dw = torch.empty(V, H, **f32)
    P = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    stream = torch.cuda.current_stream(dev).cuda_stream
    libs = {name: load_variant(variant_path(name)) for name, _, _, _ in VARIANTS}
    base = libs["product"]
    ws_f = torch.empty(base.skyrl_lmhead_fwd_workspace_bytes(T, H, V), dtype=torch.uint8, device=dev)
    ws_b = torch.empty(base.skyrl_lmhead_bwd_workspace_bytes(T, H, V, 0), dtype=torch.uint8, device=dev)

    def fwd(lib, outs):
        st = lib.skyrl_lmhead_fwd(P(h), H, P(w), H, P(y), T, H, V, rt, P(outs[0]), P(outs[1]), P(outs[2]), P(outs[3]), P(ws_f),
                                  ws_f.numel(), stream)
        assert st == 0, st

    def bwd(lib, options=0):
        st = lib.skyrl_lmhead_bwd(P(h), H, P(w), H, P(y), P(lse), P(pz) if q is not None else None, P(g), P(q), T, H, V, rt, P(dh),
                                  P(dw), options, 0, P(ws_b), ws_b.numel(), stream)
        assert st == 0, st

    fwd(base, (lp, ent, lse, pz))      # the row statistics every backward below uses
    bwd(base)
    torch.cuda.synchronize()

    def timed(lib, options=0):
        n = lib.skyrl_lmhead_num_kernel_kinds()
        hnd = lib.skyrl_lmhead_profile_begin()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fwd(lib, junk if lib is not base else (lp, ent, lse, pz))
            bwd(lib, options)
        e1.record()
        torch.cuda.synchronize()
        ms, cnt = (ctypes.c_double * n)(), (ctypes.c_int64 * n)()
        assert lib.skyrl_lmhead_profile_end(hnd, ms, cnt) == 0
        per = {lib.skyrl_lmhead_kernel_name(k).decode(): ms[k] / args.steps for k in range(n) if cnt[k]}
        per["step"] = e0.elapsed_time(e1) / args.steps
        return per

    rows = {name: [] for name in libs}
    rows["product + tiny dz flushed"] = []
    for _ in range(2):
        timed(base)
    for _ in range(args.rounds):
        for name, lib in libs.items():
            rows[name].append(timed(lib))
        rows["product + tiny dz flushed"].append(timed(base, ops.FLUSH_TINY_DZ_BIT))
    fwd(base, (lp, ent, lse, pz))
    bwd(base)

    def med(name, key):
        v = sorted(r[key] for r in rows[name])
        return v[len(v) // 2]

    kernels = ("lmhead_fwd_tiles", "lmhead_bwd_dz", "lmhead_bwd_gemm")
    flop = {"lmhead_fwd_tiles": 2.0 * T * V * H, "lmhead_bwd_dz": 2.0 * T * V * H, "lmhead_bwd_gemm": 4.0 * T * V * H}
    print(f"workload {cfg.name}: T={T} H={H} V={V}, {args.rounds} rounds x {args.steps} steps per variant, medians, ms per step "
          f"(fraction of 2.5 PFLOP/s)")
    print(f"{'variant':<28}" + "".join(f"{k:>26}" for k in kernels) + f"{'whole step':>14}   left out")
    for name, _, touched, what in VARIANTS + [("product + tiny dz flushed", 0, ("lmhead_bwd_gemm",), "nothing: p < 2^-24 is written as 0 into the dz panel")]:
        cells = []
        for k in kernels:
            ms = med(name, k)
            mark = "*" if (k in touched) else " "
            cells.append(f"{ms:>14.3f} ({flop[k] / (ms * 1e-3) / 2.5e15:.3f}){mark}  ")
        print(f"{name:<28}" + "".join(cells) + f"{med(name, 'step'):>12.3f}   {what}")
    print("* the kernel the variant changes; the other columns show the run-to-run spread of unchanged kernels")

    extra = {}

    def product_step():
        fwd(base, (lp, ent, lse, pz))
        bwd(base)

    extra["power_product_steps"] = bench_py.power_while(product_step, 10)
    extra["power_flushed_steps"] = bench_py.power_while(lambda: (fwd(base, (lp, ent, lse, pz)), bwd(base, ops.FLUSH_TINY_DZ_BIT)), 10)
    extra["mfma_probe"] = bench_py.mfma_probe(base, dev)

    # Board power by kind of work: which launches sit at the board's cap, and what the matrix pipe alone, HBM alone draw.
    def watts(fn, n):
        p = bench_py.power_while(fn, n)
        return None if p is None else round(p["avg_watts"], 1)

    watts_by = {"idle": watts(lambda: time.sleep(0.05), 10)}
    sink = torch.empty(256 * 256, **f32)
    for name, operands in (("mfma_only_zero_operands", torch.zeros(65536)), ("mfma_only_random_operands", torch.randn(65536))):
        o = operands.to(torch.bfloat16).to(dev)
        watts_by[name] = watts(lambda: _lib.check(base.skyrl_lmhead_mfma_probe(o.data_ptr(), 256, 20000, sink.data_ptr(), stream), "probe"), 12)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    watts_by["hbm_copy"] = watts(lambda: dst.copy_(src), 400)
    del src, dst
    watts_by["forward_launches"] = watts(lambda: fwd(base, (lp, ent, lse, pz)), 30)
    watts_by["backward_launches"] = watts(lambda: bwd(base), 10)
    watts_by["backward_launches_l2_only_gemm"] = watts(lambda: bwd(libs["l2_only_gemm"]), 10)
    fwd(base, (lp, ent, lse, pz))
    bwd(base)
    extra["avg_watts_by_kind"] = watts_by
    extra["vendor_gemm"] = bench_py.vendor_gemm(h, w)
    # the atomic traffic of a fully fused backward, alone
    dh32 = torch.zeros(T, H, **f32)
    ms = []
    for _ in range(2):
        dw.zero_()
        dh32.zero_()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        st = base.skyrl_lmhead_atomic_floor_probe(P(dw), P(dh32), T // 256 * 256, H, V // 256 * 256, stream)
        e1.record()
        torch.cuda.synchronize()
        assert st == 0, st
        ms.append(e0.elapsed_time(e1))
    adds = 2.0 * (T // 256) * (V // 256) * 256 * H
    extra["fused_backward_atomic_floor"] = {
        "ms": min(ms), "fp32_atomic_adds": adds, "bytes": 4 * adds, "TB_per_s": 4 * adds / (min(ms) * 1e-3) / 1e12,
        "exact": bool(float(dw[0, 0]) == T // 256 and float(dh32[0, 0]) == V // 256),
        "split_backward_ms": med("product", "lmhead_bwd_dz") + med("product", "lmhead_bwd_gemm"),
    }
    print(json.dumps(extra, indent=1))
    return 0


if __name__ == "__main__":
    sys.exit(main())

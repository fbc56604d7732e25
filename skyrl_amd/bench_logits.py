"""Benchmark of the logits-input kernels (``python -m skyrl_amd.bench_logits``): log-probability + entropy forward and the
backward from a materialised ``[T, V]`` logits matrix, Qwen2.5-7B-sized by default (T = 16384, V = 152064), synthetic data,
one GPU.  Prints one JSON line: per variant the time, the algorithmic bytes (``T * V * es`` read in the forward, read + written
in the backward) per second and their fraction of the MI355X's 8 TB/s; with ``--eager`` also what the same statistics cost
through plain torch operations on the same GPU (``log_softmax`` + ``gather`` + entropy, and their autograd backward).
"""

from __future__ import annotations

import argparse
import json
import sys

import torch

from . import torch_utils as TU

PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, published


def _time(fn, steps: int, warmup: int) -> float:
    for _ in range(warmup):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--tokens", type=int, default=16384)
    ap.add_argument("--vocab", type=int, default=152064)
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--eager", action="store_true", help="also time plain torch operations on the same logits")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        print("bench_logits needs a ROCm GPU: there is no CPU implementation of this path", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    T, V = args.tokens, args.vocab
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    es = 2 if args.dtype == "bf16" else 4
    gen = torch.Generator(device=dev).manual_seed(2000)
    logits = torch.empty(T, V, dtype=dtype, device=dev)
    for r in range(0, T, 2048):
        n = min(2048, T - r)
        logits[r:r + n] = (torch.randn(n, V, device=dev, generator=gen) * 3).to(dtype)
    labels = torch.randint(0, V, (T,), device=dev, generator=gen)
    g = torch.randn(T, device=dev, generator=gen)
    q = torch.randn(T, device=dev, generator=gen) * 0.01
    lp, ent, lse, pz = TU.logits_fwd(logits, labels, 1.0, True)
    out = torch.empty_like(logits)
    scratch = logits.clone()
    matrix = T * V * es

    def report(ms: float, nbytes: int) -> dict:
        gbs = nbytes / ms / 1e6
        return {"ms": ms, "GB/s": gbs, "frac_of_hbm_peak": gbs / PEAK_HBM_GBS}

    variants = {
        "fwd logprob+entropy": (lambda: TU.logits_fwd(logits, labels, 1.0, True), matrix),
        "fwd logprob": (lambda: TU.logits_fwd(logits, labels, 1.0, False), matrix),
        "bwd dlogprobs": (lambda: TU._bwd_into(out, logits, labels, lse, None, g, None, 1.0), 2 * matrix),
        "bwd dlogprobs+dentropy": (lambda: TU._bwd_into(out, logits, labels, lse, pz, g, q, 1.0), 2 * matrix),
        # timing only: after the first call the buffer holds gradients, not logits; the arithmetic per element is the same
        "bwd in place": (lambda: TU._bwd_into(scratch, scratch, labels, lse, None, g, None, 1.0), 2 * matrix),
    }
    result = {name: report(_time(fn, args.steps, args.warmup), nbytes) for name, (fn, nbytes) in variants.items()}
    del scratch, out
    eager = None
    if args.eager:
        def eager_fwd():
            lsm = torch.log_softmax(logits.float(), dim=-1)
            return lsm.gather(-1, labels[:, None])[:, 0], -(lsm.exp() * lsm).sum(-1)

        def eager_fwd_bwd():
            x = logits.detach().requires_grad_(True)
            lsm = torch.log_softmax(x.float(), dim=-1)
            a, b = lsm.gather(-1, labels[:, None])[:, 0], -(lsm.exp() * lsm).sum(-1)
            (a * g + b * q).sum().backward()
            return x.grad

        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        f = _time(eager_fwd, max(2, args.steps // 3), 1)
        fb = _time(eager_fwd_bwd, max(2, args.steps // 3), 1)
        eager = {"fwd ms": f, "fwd+bwd ms": fb, "peak_extra_bytes": torch.cuda.max_memory_allocated() - base}
    fwd, bwd = result["fwd logprob+entropy"], result["bwd dlogprobs+dentropy"]
    print(json.dumps({
        "metric": "logits-input logprob+entropy fwd+bwd tokens/sec on 1 MI355X; fraction of HBM peak",
        "value": T / (fwd["ms"] + bwd["ms"]) * 1e3, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": fwd["ms"] + bwd["ms"], "higher_is_better": True, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": f"logits [T={T}, V={V}] {args.dtype}: log-probability + entropy forward, backward with both upstream gradients"},
        "roofline": {"kernel": "logits_bwd_rows", "bound": "hbm", "achieved": bwd["GB/s"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": bwd["frac_of_hbm_peak"], "traffic": None},
        "variants": result, "eager_torch_same_gpu": eager, "extra_memory_bytes": 16 * T}))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

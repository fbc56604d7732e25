"""Benchmark of the fused MTP soft cross-entropy (``python -m skyrl_amd.bench_soft_ce``): forward + backward from hidden
states at a Qwen2.5-7B-shaped LM head by default, synthetic data, one GPU.  Prints one JSON line with the step time, the
rate on the 10*T*V*H flop of a step (two forward products, their recomputation, the student's input gradient) and the
library's own per-kernel HIP-event times.  With ``--topk K`` the top-k variant runs instead (one forward product of
2*T*V*H flop with the candidate filter in its epilogue, then K gathered weight rows per token in each direction).
"""

from __future__ import annotations

import argparse
import ctypes
import json
import sys
import time

import torch

from . import _lib
from .mtp_soft_ce import softce_bwd, softce_fwd, softce_topk_bwd, softce_topk_fwd, topk_logits

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16, published


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--tokens", type=int, default=16384)
    ap.add_argument("--hidden", type=int, default=3584)
    ap.add_argument("--vocab", type=int, default=152064)
    ap.add_argument("--depth", type=int, default=0, help="MTP depth: the teacher is rolled by depth + 1 positions")
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--vocab-chunk", type=int, default=0)
    ap.add_argument("--topk", type=int, default=0, help="distill only the teacher's K largest logits (draft_soft_ce_topk)")
    ap.add_argument("--data", choices=["gaussian", "peaked"], default="gaussian",
                    help="peaked: teacher hidden states close to a weight row, so that a few logits stand out as in a trained model")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        print("bench_soft_ce needs a ROCm GPU: there is no CPU implementation of this path", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    T, H, V = args.tokens, args.hidden, args.vocab
    gen = torch.Generator().manual_seed(2000)
    student = torch.randn(T, H, generator=gen).bfloat16().to(dev)
    teacher = torch.randn(T, H, generator=gen).bfloat16().to(dev)
    weight = (torch.randn(V, H, generator=gen) * 3.0 / H ** 0.5).bfloat16().to(dev)
    dloss = torch.randn(T, generator=gen).to(dev)
    if args.data == "peaked":
        rows = torch.randint(0, V, (T,), generator=gen).to(dev)
        teacher = (teacher.float() + 4.0 * H ** 0.5 / 3.0 * weight[rows].float()).bfloat16()
    lib = _lib.load()

    def step_topk():
        values, columns = topk_logits(teacher, weight, args.topk, 1.0)
        loss, coef, used = softce_topk_fwd(student, weight, values, columns, T, args.depth + 1, 1.0)
        return loss, softce_topk_bwd(weight, coef, used, dloss, 1.0)

    def step():
        if args.topk:
            return step_topk()
        loss, lse_s, lse_t = softce_fwd(student, teacher, weight, T, args.depth + 1, 1.0)
        return loss, softce_bwd(student, teacher, weight, lse_s, lse_t, dloss, T, args.depth + 1, 1.0, args.vocab_chunk)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize(dev)
    handle = lib.skyrl_lmhead_profile_begin()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss, d_student = step()
    torch.cuda.synchronize(dev)
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    n = lib.skyrl_lmhead_num_kernel_kinds()
    total, count = (ctypes.c_double * n)(), (ctypes.c_int64 * n)()
    _lib.check(lib.skyrl_lmhead_profile_end(handle, total, count), "skyrl_lmhead_profile_end")
    kernels = {lib.skyrl_lmhead_kernel_name(k).decode(): {"ms_per_step": total[k] / args.steps,
                                                          "launches_per_step": count[k] / args.steps}
               for k in range(n) if count[k]}
    flop = (2.0 * T * V * H + 4.0 * T * args.topk * H) if args.topk else 10.0 * T * V * H
    tflops = flop / ms / 1e9
    print(json.dumps({
        "metric": "fused MTP soft cross-entropy fwd+bwd tokens/sec on 1 MI355X", "value": T / ms * 1e3, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "dtype": "bf16",
        "data": "synthetic", "config": {"workload": f"mtp-soft-ce{'-top' + str(args.topk) if args.topk else ''}: T={T} H={H} V={V} depth={args.depth}, "
                               f"{args.data} data, forward+backward"},
        "tflops": tflops, "pct_of_bf16_mfma_peak": 100.0 * tflops / PEAK_BF16_TFLOPS, "kernels": kernels,
        "loss_mean": loss.mean().item(), "scratch_bytes": (
            {"forward": int(lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, args.topk)), "backward": 0} if args.topk else
            {"forward": int(lib.skyrl_softce_fwd_workspace_bytes(T, H, V)),
             "backward": int(lib.skyrl_softce_bwd_workspace_bytes(T, H, V, args.vocab_chunk))})}))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

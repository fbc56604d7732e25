"""Times of the per-token loss kernels and the packed-sequence index kernels (``python -m skyrl_amd.bench_small_kernels``).

Each kernel is called through the C ABI 200 times on ``[rows, cols]`` fp32 inputs of three sizes; the table gives the mean
time per call and the rate on the bytes the call has to move.  At the sizes of one micro-batch these kernels are bound by
launch latency, not by HBM.
"""

from __future__ import annotations

import sys

import torch

from . import _lib


def _time_us(fn, n: int = 200) -> float:
    for _ in range(10):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(n):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / n * 1e3


def main() -> int:
    if not torch.cuda.is_available():
        print("bench_small_kernels needs a ROCm GPU: there is no CPU implementation of these kernels", file=sys.stderr)
        return 2
    lib = _lib.load()
    dev = "cuda"
    p = lambda t: t.data_ptr()  # noqa: E731
    for rows, cols in ((8, 2048), (64, 8192), (512, 8192)):
        n = rows * cols
        g = torch.Generator(device=dev).manual_seed(0)
        lp = torch.randn(rows, cols, device=dev, generator=g) * 0.5 - 2
        old = lp + torch.randn(rows, cols, device=dev, generator=g) * 0.3
        base = lp + torch.randn(rows, cols, device=dev, generator=g) * 0.3
        adv = torch.randn(rows, cols, device=dev, generator=g)
        ent = torch.rand(rows, cols, device=dev, generator=g)
        mask = (torch.rand(rows, cols, device=dev, generator=g) > 0.4).float()
        f = lambda *shape: torch.empty(*shape, device=dev)  # noqa: E731
        part, out3, grad, out6, row_sums, dlp, dent = f(768), f(3), f(n), f(6), f(rows, 6), f(n), f(n)
        kld, row_mean, mean = f(n), f(rows), f(())
        cu = (torch.arange(rows + 1, device=dev) * cols).to(torch.int64)
        tokens = torch.randint(0, 150000, (n,), device=dev, generator=g)
        labels = torch.empty_like(tokens)
        packed = torch.randn(n, device=dev, generator=g)
        out = f(rows, cols - 1)
        am = torch.ones(rows, cols, dtype=torch.uint8, device=dev)
        import ctypes
        keep, tis, wgt, met, rstat, parts5 = f(n), f(n), f(n), f(16), f(rows * 20), f(5 * 256)
        c_f = lambda v: ctypes.byref(ctypes.c_float(v))  # noqa: E731
        cases = {  # name: (call, bytes the call reads and writes)
            "ppo_policy_loss": (lambda: lib.skyrl_ppo_policy_loss(p(lp), p(old), p(adv), p(mask), None, n, 0.2, 0.2, 3.0, 0, p(out3),
                                                                  p(grad), p(part), None), 20 * n),
            "approx_kl + gradient": (lambda: lib.skyrl_approx_kl(p(lp), p(base), p(mask), rows, cols, 3, p(kld), p(row_mean), p(mean),
                                                                 2, p(grad), None), 20 * n),
            "masked_mean + gradient": (lambda: lib.skyrl_masked_mean(p(lp), p(mask), rows, cols, p(row_mean), p(grad), None), 12 * n),
            "actor_loss, all terms": (lambda: lib.skyrl_actor_loss(p(lp), p(old), p(adv), p(mask), None, p(base), p(ent), rows, cols, 0,
                                                                   0.2, 0.2, 3.0, 3, 1.0, 1.0, 0.01, 0.01, p(row_sums), p(out6), p(dlp),
                                                                   p(dent), None), 36 * n),
            "off_policy_correction, all steps": (lambda: lib.skyrl_off_policy_correction(
                p(old), p(lp), p(mask), rows, cols, 1, 1.5, 1, 0.9, 1.1, c_f(0.5), c_f(3.0), c_f(0.7), c_f(1.5), p(keep), p(tis), p(wgt),
                p(met), p(rstat), None), 36 * n),
            "logprob_diff_metrics": (lambda: lib.skyrl_logprob_diff_metrics(p(lp), p(old), p(mask), n, p(out6), p(parts5), None), 12 * n),
            "packed_next_token_labels": (lambda: lib.skyrl_packed_next_token_labels(p(tokens), p(cu), rows, n, p(labels), None), 16 * n),
            "packed_scatter, plain": (lambda: lib.skyrl_packed_scatter_logprobs(p(packed), p(cu), rows, n, None, None, None, None, rows,
                                                                                cols - 1, p(out), None), 12 * n),
            "packed_scatter, attention mask": (lambda: lib.skyrl_packed_scatter_logprobs(p(packed), p(cu), rows, n, None, None, None, p(am),
                                                                                         rows, cols - 1, p(out), None), 10 * n),
            "packed_gather_grad, plain": (lambda: lib.skyrl_packed_gather_grad(p(out), p(cu), rows, n, None, None, None, None, rows,
                                                                               cols - 1, p(packed), None), 8 * n),
        }
        print(f"[{rows}, {cols}] = {n} tokens")
        for name, (call, nbytes) in cases.items():
            us = _time_us(call)
            print(f"   {name:32s} {us:8.1f} us  {nbytes / us / 1e3:8.1f} GB/s", flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

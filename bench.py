#!/usr/bin/env python3
"""Benchmark of the fused LM-head log-probability path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME] [--no-cpu-baseline]

A step is one forward + backward pass of the path over one synthetic micro-batch that is already resident in HBM: the
Qwen2.5-7B-shaped LM head (T=16384 packed tokens, H=3584, V=152064, temperature 0.6, upstream gradients on both the
log-probabilities and the entropy).  The step goes through the C ABI (``skyrl_lmhead_fwd`` then ``skyrl_lmhead_bwd``), exactly
as the torch custom ops call it.  One JSON line is printed:

  value / unit   tokens per second of forward + backward (whole job; one GPU)
  roofline       the dominant kernel (``lmhead_bwd_gemm``: the dHidden and dWeight products of every vocab chunk, 4*T*V*H of
                 the 8*T*V*H flop and half of the step) against the dense bf16 MFMA peak of 2.5 PFLOP/s; its time is measured
                 live with HIP events on the launch stream
  step_roofline  the whole step (8*T*V*H algorithmic flop / step time) against the same peak
  kernels        live HIP-event time per kernel and step
  cpu_baseline   the CPU restatement of the reference's torch implementation, timed on this host on a bounded sample
  mfma_probe     what the matrix pipe of this GPU sustains with the mainloop's MFMA sequence alone (operands in registers, no
                 memory access), on N(0,1) operands and on zeros: with random operands the chip is power-limited well below
                 the published peak, which bounds every bf16 kernel on this benchmark's data
  vendor_gemm    one ``torch.matmul`` (hipBLASLt) of the same [T,H] x [V,H]^T bf16 product on the same data, HIP-event timed
  power          board power from the driver's hwmon file while the same steps run again, next to the board's power cap
  autograd       the same step through ``linear_cross_entropy(...)`` and ``loss.backward()`` on fresh tensors, wall-clock
                 and peak allocated bytes (the protocol of the reference's own harness)
The last three legs run after the timed region.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_DENSE_FLOPS = 2.5e15  # MI355X dense bf16 MFMA
METRIC = "fused LM-head fwd+bwd tokens/sec on 1 MI355X; % bf16 MFMA peak"

def measured_traffic(config_name: str, kernel: str):
    """Bytes beyond L2 per launch of ``kernel`` in workload ``config_name``, or None when that workload has not been profiled.

    Not measurable live: it comes from two ``rocprofv3 --pmc`` passes (FETCH_SIZE, then WRITE_SIZE), each scaled by what the
    same counter reads for the 1 GiB copy of --copy-probe.  The summary of those passes under profiles/ ends with one line per
    kernel, ``traffic_bytes_per_launch <workload> <kernel> <bytes>``; this reads it back, so the figure in the benchmark line
    changes when, and only when, the profile is regenerated.  Returns ``(bytes, file name)``.
    """
    import glob

    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*hbm_traffic*.txt"))):
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 4 and parts[0] == "traffic_bytes_per_launch" and parts[1] == config_name and parts[2] == kernel:
                    return int(float(parts[3])), os.path.basename(path)
    return None, None


def cpu_baseline(cfg, sample_tokens: int):
    """Time the oracle's reference-faithful torch path (bf16 matmul, fp32 softmax, 1 chunk) on ``sample_tokens`` tokens."""
    import torch

    from oracle import lmhead_oracle as O
    from skyrl_amd.bench_inputs import make_inputs
    import dataclasses

    small = dataclasses.replace(cfg, T=sample_tokens, layout="dense", n_seqs=1, mask="none")
    d = make_inputs(small)
    g = d.get("dlogprobs") if cfg.backward else None
    warm = {k: (v[:8] if k in ("hidden", "labels", "dlogprobs") else v) for k, v in d.items()}
    O.reference_faithful_fwd_bwd(warm["hidden"], warm["weight"][:4096], warm["labels"] % 4096, cfg.temperature,
                                 warm.get("dlogprobs") if cfg.backward else None, chunk_size=8, want_entropy=cfg.entropy)
    t0 = time.perf_counter()
    chunk = min(sample_tokens, 1024)  # the reference's default logprobs_chunk_size (skyrl/train/config/config.py:1482)
    O.reference_faithful_fwd_bwd(d["hidden"], d["weight"], d["labels"], cfg.temperature, g, chunk_size=chunk,
                                 want_entropy=cfg.entropy)
    dt = time.perf_counter() - t0
    cpu_model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {
        "value": sample_tokens / dt,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "cpu_model": cpu_model,
        "torch_version": torch.__version__,
        "kind": "port",
        "sample": f"{sample_tokens} of {cfg.T} tokens at full H={cfg.H}, V={cfg.V}: logprob forward + entropy metric"
                  f"{' + backward' if cfg.backward else ''} in chunks of {chunk}, bf16 torch.matmul on CPU, {dt:.1f} s; the algorithm is a"
                  " loop over independent token chunks, so tokens/s carries over to the full batch",
    }


def mfma_probe(lib, dev):
    """Pure-MFMA rate (TFLOP/s) of the GEMM mainloop's instruction sequence on random and on zero operands."""
    import torch

    from skyrl_amd import _lib

    wgs, iters = 256, 50000
    flop = 4.0 * wgs * iters * 128 * 16384
    sink = torch.empty(256 * wgs, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    out = {"mfma": "v_mfma_f32_16x16x32_bf16", "workgroups": wgs}
    gen = torch.Generator().manual_seed(7)
    for name in ("random", "zero"):
        ops_ = (torch.randn(65536, generator=gen) if name == "random" else torch.zeros(65536)).to(torch.bfloat16).to(dev)
        ms = []
        for it in (iters // 10, iters, iters):  # short warm-up, then two timed launches
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(lib.skyrl_lmhead_mfma_probe(ops_.data_ptr(), wgs, it, sink.data_ptr(), stream), "skyrl_lmhead_mfma_probe")
            e1.record()
            torch.cuda.synchronize()
            ms.append(e0.elapsed_time(e1))
        out[f"{name}_operands_tflops"] = flop / (min(ms[1:]) * 1e-3) / 1e12
    return out


def vendor_gemm(hidden, weight):
    """TFLOP/s of the vendor library on the forward's product, same operands: ``hidden @ weight.T`` in bf16 (one [T, V] bf16
    result, allocated once and freed before returning)."""
    import torch

    T, H = hidden.shape
    V = weight.shape[0]
    out = torch.empty(T, V, dtype=torch.bfloat16, device=hidden.device)
    wt = weight.t()
    ms = []
    for _ in range(4):  # the first call picks the algorithm
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        torch.matmul(hidden, wt, out=out)
        e1.record()
        torch.cuda.synchronize()
        ms.append(e0.elapsed_time(e1))
    del out
    best = min(ms[1:])
    return {"op": f"torch.matmul bf16 [{T},{H}] x [{V},{H}]^T -> bf16 [{T},{V}]", "ms": best,
            "tflops": 2.0 * T * V * H / (best * 1e-3) / 1e12, "frac_of_peak": 2.0 * T * V * H / (best * 1e-3) / PEAK_BF16_DENSE_FLOPS}


def _hwmon(name: str):
    import glob

    found = sorted(glob.glob(f"/sys/class/drm/card*/device/hwmon/hwmon*/{name}"))
    return found[0] if found else None


def power_while(step, steps: int):
    """Average board power (W) over ``steps`` more steps, read from the amdgpu hwmon file every few milliseconds by a second
    thread, and the board's power cap.  None when the files are not readable."""
    import threading

    import torch

    path = _hwmon("power1_input") or _hwmon("power1_average")
    cap = _hwmon("power1_cap")
    if not path:
        return None
    samples, stop = [], threading.Event()

    def sample():
        while not stop.is_set():
            try:
                with open(path) as f:
                    samples.append(int(f.read()) / 1e6)
            except (OSError, ValueError):
                pass
            time.sleep(0.003)

    for _ in range(3):  # reach the steady thermal / power state first
        step()
    torch.cuda.synchronize()
    th = threading.Thread(target=sample, daemon=True)
    th.start()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    stop.set()
    th.join()
    if not samples:
        return None
    out = {"avg_watts": sum(samples) / len(samples), "max_watts": max(samples), "samples": len(samples), "source": path}
    if cap:
        try:
            with open(cap) as f:
                out["cap_watts"] = int(f.read()) / 1e6
        except (OSError, ValueError):
            pass
    return out


def autograd_leg(cfg, hidden, weight, labels, g, q, reps: int = 3):
    """The step as the trainer calls it, timed as skyrl/benchmarks/bench_fused_linear_logprob.py:83-108 times the reference:
    fresh leaf tensors, ``linear_cross_entropy`` -> a scalar loss -> ``backward()``, synchronize, wall clock; median of ``reps``
    after one warm-up, and the peak of ``torch.cuda.max_memory_allocated`` above what was allocated before the call."""
    import torch

    from skyrl_amd.fused_linear_logprob_hip import linear_cross_entropy

    times, peak = [], 0
    for it in range(reps + 1):
        h = hidden.detach().clone().requires_grad_(True)
        w = weight.detach().clone().requires_grad_(True)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        t0 = time.perf_counter()
        logprobs, entropy = linear_cross_entropy(h, w, labels, float(cfg.temperature), "none", None)
        loss = (logprobs * g).sum()
        if q is not None:
            loss = loss + (entropy * q).sum()
        loss.backward()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if it > 0:
            times.append(dt * 1e3)
            peak = max(peak, torch.cuda.max_memory_allocated() - base)
        del h, w, logprobs, entropy, loss
    times.sort()
    return {"call": "linear_cross_entropy(hidden, weight, labels, temperature, 'none', None); (logprobs*g + entropy*q).sum().backward()",
            "ms_per_step": times[len(times) // 2], "ms_all": times, "peak_bytes_above_inputs": int(peak),
            "grad_weight_dtype": "bf16 (the weight's dtype, as the reference returns it)"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default="qwen2.5-7b-fwdbwd")
    ap.add_argument("--vocab-chunk", type=int, default=0)
    ap.add_argument("--cpu-sample-tokens", type=int, default=6144)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-mfma-probe", action="store_true")
    ap.add_argument("--no-extra-legs", action="store_true",
                    help="skip the legs that run after the timed region: vendor GEMM, board power, the autograd call")
    ap.add_argument("--skip-masked-rows", action="store_true",
                    help="run the backward pass through skyrl_lmhead_bwd_active_rows, which drops the tokens whose upstream "
                         "gradients are zero on the device (the configurations with a response mask); value stays tokens/s "
                         "over all T tokens, the roofline figures count the flop actually executed")
    ap.add_argument("--frozen-lm-head", action="store_true",
                    help="the weight takes no gradient (adapter training): d_weight = NULL, the dW product is skipped")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 1 GiB device-to-device copy (a kernel of known HBM traffic) so that rocprofv3 "
                         "--pmc FETCH_SIZE / WRITE_SIZE readings of the same run can be scaled to bytes")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the fused LM-head path on ONE GPU; --gpus N with N > 1 is not supported "
              "(every GPU box of this project has one GPU, and the path has no collectives at tensor-parallel size 1).",
              file=sys.stderr)
        return 2

    import torch

    from skyrl_amd import _lib, ops
    from skyrl_amd.bench_inputs import CONFIGS, make_inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback.", file=sys.stderr)
        return 3
    cfg = CONFIGS[args.config]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.load()

    d = make_inputs(cfg)
    T, H, V = cfg.T, cfg.H, cfg.V
    rcp_t = 1.0 / cfg.temperature
    want_ent = cfg.entropy or cfg.entropy_grad
    hidden, weight, labels = d["hidden"].to(dev), d["weight"].to(dev), d["labels"].to(dev)
    g = d["dlogprobs"].to(dev) if cfg.backward else None
    q = d["dentropy"].to(dev) if cfg.entropy_grad else None

    # Outputs and scratch are allocated once, outside the timed region, and passed by pointer: the timed region is the C ABI.
    f32 = dict(dtype=torch.float32, device=dev)
    logprobs, row_lse = torch.empty(T, **f32), torch.empty(T, **f32)
    entropy = torch.empty(T, **f32) if want_ent else None
    row_pz = torch.empty(T, **f32) if want_ent else None
    ws_f = torch.empty(ops.fwd_workspace_bytes(T, H, V), dtype=torch.uint8, device=dev)
    if cfg.backward:
        d_hidden = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
        d_weight = torch.empty(V, H, **f32)
        skip_rows = bool(args.skip_masked_rows)
        bwd_query = lib.skyrl_lmhead_bwd_active_rows_workspace_bytes if skip_rows else lib.skyrl_lmhead_bwd_workspace_bytes
        bwd_entry = lib.skyrl_lmhead_bwd_active_rows if skip_rows else lib.skyrl_lmhead_bwd
        ws_b = torch.empty(int(bwd_query(T, H, V, args.vocab_chunk)), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731

    skip = bool(args.skip_masked_rows and cfg.backward)
    t_active = int(((g != 0) | ((q != 0) if q is not None else False)).sum().item()) if skip else T

    def step(bwd_options: int = 0):
        st = lib.skyrl_lmhead_fwd(hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0), labels.data_ptr(),
                                  T, H, V, rcp_t, logprobs.data_ptr(), ptr(entropy), row_lse.data_ptr(), ptr(row_pz),
                                  ws_f.data_ptr(), ws_f.numel(), stream)
        _lib.check(st, "skyrl_lmhead_fwd")
        if cfg.backward:
            st = bwd_entry(hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0),
                                      labels.data_ptr(), row_lse.data_ptr(), ptr(row_pz) if q is not None else None,
                                      g.data_ptr(), ptr(q), T, H, V, rcp_t, d_hidden.data_ptr(),
                                      None if args.frozen_lm_head else d_weight.data_ptr(), bwd_options,
                                      args.vocab_chunk, ws_b.data_ptr(), ws_b.numel(), stream)
            _lib.check(st, "skyrl_lmhead_bwd")

    if args.copy_probe:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)  # 1 GiB read + 1 GiB written
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # Timed region: exactly K steps, bracketed by synchronize on both sides; per-kernel HIP events ride along.
    with _lib.KernelProfile() as prof:
        torch.cuda.synchronize()
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]  # per-step times ride along
        t0 = time.perf_counter()
        marks[0].record()
        for k in range(args.steps):
            step()
            marks[k + 1].record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    per_step = sorted(marks[k].elapsed_time(marks[k + 1]) for k in range(args.steps))
    ms_per_step = elapsed * 1e3 / args.steps
    tokens_per_s = T * args.steps / elapsed

    kernels = {k: {"ms_per_step": ms / args.steps, "launches_per_step": n / args.steps, "avg_launch_ms": ms / n}
               for k, (ms, n) in prof.results.items() if n}
    # Executed flop: forward over all T tokens, backward over the tokens that were not dropped.
    bwd_gemms = 2.0 if args.frozen_lm_head else 3.0  # logits recompute + dHidden (+ dWeight)
    step_flop = 2.0 * T * V * H + (2.0 * bwd_gemms * t_active * V * H if cfg.backward else 0.0)
    step_roofline = {"bound": "mfma", "achieved": step_flop / (ms_per_step * 1e-3) / 1e12, "peak": PEAK_BF16_DENSE_FLOPS / 1e12,
                     "unit": "TFLOP/s"}
    step_roofline["frac"] = step_roofline["achieved"] / step_roofline["peak"]

    # Dominant kernel: lmhead_bwd_gemm with a backward pass (one launch per vocab chunk carries the chunk's dHidden and dWeight
    # products: over a step 4*T*V*H flop, 2*T*V*H for a frozen LM head); forward-only workloads are all lmhead_fwd_tiles.
    if cfg.backward:
        k = kernels["lmhead_bwd_gemm"]
        dom_name, dom_flop = "lmhead_bwd_gemm", 2.0 * (bwd_gemms - 1.0) * t_active * V * H
        dom_ms, dom_launches = k["ms_per_step"], k["launches_per_step"]
    else:
        k = kernels["lmhead_fwd_tiles"]
        dom_name, dom_ms, dom_launches, dom_flop = "lmhead_fwd_tiles", k["ms_per_step"], k["launches_per_step"], 2.0 * T * V * H
    achieved = dom_flop / (dom_ms * 1e-3) / 1e12
    traffic, traffic_source = measured_traffic(cfg.name, dom_name)
    roofline = {
        "kernel": dom_name,
        "bound": "mfma",
        "achieved": achieved,
        "peak": PEAK_BF16_DENSE_FLOPS / 1e12,
        "unit": "TFLOP/s",
        "frac": achieved / (PEAK_BF16_DENSE_FLOPS / 1e12),
        "traffic": traffic,
        "traffic_source": traffic_source,
        "flop_per_launch": dom_flop / dom_launches,
        "avg_launch_ms": dom_ms / dom_launches,
        "launches_per_step": dom_launches,
    }

    import ctypes
    cus, khz = ctypes.c_int(0), ctypes.c_int(0)
    _lib.check(lib.skyrl_lmhead_device_info(ctypes.byref(cus), ctypes.byref(khz)), "skyrl_lmhead_device_info")
    box_cus, box_khz = cus.value, khz.value
    out = {
        "metric": METRIC,
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_median": per_step[len(per_step) // 2],
        "ms_per_step_min": per_step[0],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{cfg.name}: LM head T={T} H={H} V={V}, temperature {cfg.temperature}, "
                        f"{'forward+backward' if cfg.backward else 'forward'}"
                        f"{', entropy with upstream grad' if cfg.entropy_grad else (', entropy' if cfg.entropy else '')}"
                        f"{', frozen LM head (no dW)' if args.frozen_lm_head and cfg.backward else ''}",
            "T": T, "H": H, "V": V, "temperature": cfg.temperature,
            "vocab_chunk": args.vocab_chunk or "library default",
            "backward_tokens": t_active,
            "device": torch.cuda.get_device_name(0),
            "compute_units": torch.cuda.get_device_properties(0).multi_processor_count,
            # the box's own figure for the denominator: CUs x 4096 bf16 flop per clock per CU x the maximum shader clock
            "max_clock_mhz": box_khz / 1e3,
            "peak_from_box_tflops": box_cus * 4096 * box_khz * 1e3 / 1e12,
        },
        "scratch_bytes": {"forward": ws_f.numel(), "backward": ws_b.numel() if cfg.backward else 0,
                          "one_bf16_TxV_buffer_would_be": 2 * T * V},
        "tflops": step_roofline["achieved"],
        "pct_of_bf16_mfma_peak": 100.0 * step_roofline["frac"],
        "roofline": roofline,
        "step_roofline": step_roofline,
        "kernels": kernels,
    }
    # Each MFMA kernel against the published peak and against what the matrix pipe of this box sustains on random operands
    # with nothing else in the loop (the power-limited ceiling of any bf16 kernel on this data).
    kind_flop = {"lmhead_fwd_tiles": 2.0 * T * V * H}
    if cfg.backward:
        kind_flop["lmhead_bwd_dz"] = 2.0 * t_active * V * H
        kind_flop["lmhead_bwd_gemm"] = 2.0 * (bwd_gemms - 1.0) * t_active * V * H
    probe = None if args.no_mfma_probe else mfma_probe(lib, dev)
    per_kernel = {}
    for name, fl in kind_flop.items():
        if name in kernels:
            tf = fl / (kernels[name]["ms_per_step"] * 1e-3) / 1e12
            per_kernel[name] = {"tflops": tf, "frac_of_peak": tf / (PEAK_BF16_DENSE_FLOPS / 1e12),
                                "frac_of_mfma_probe_random": (tf / probe["random_operands_tflops"]) if probe else None}
    out["mfma_kernels"] = per_kernel
    if probe:
        out["mfma_probe"] = probe
        out["step_frac_of_mfma_probe_random"] = step_roofline["achieved"] / probe["random_operands_tflops"]
    if not args.no_extra_legs:
        power = power_while(step, max(5, args.steps))
        if power:
            out["power"] = power
        if cfg.backward:
            # The same K steps with the backward's optional flush of softmax probabilities below 2^-24 (SKYRL_BWD_FLUSH_TINY_DZ,
            # off in `value`): same products, a dz panel that is mostly zeros, and with it a higher clock under the power limit.
            for _ in range(2):
                step(ops.FLUSH_TINY_DZ_BIT)
            torch.cuda.synchronize()
            with _lib.KernelProfile() as prof_f:
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    step(ops.FLUSH_TINY_DZ_BIT)
                torch.cuda.synchronize()
                ms_f = (time.perf_counter() - t0) * 1e3 / args.steps
            out["with_tiny_dz_flushed"] = {
                "option": "SKYRL_BWD_FLUSH_TINY_DZ: p < 2^-24 taken as 0 when dz is formed; not part of `value`",
                "ms_per_step": ms_f, "tokens_per_s": T * 1e3 / ms_f,
                "pct_of_bf16_mfma_peak": 100.0 * step_flop / (ms_f * 1e-3) / PEAK_BF16_DENSE_FLOPS,
                "kernels_ms_per_step": {k: ms / args.steps for k, (ms, n) in prof_f.results.items() if n},
            }
        if cfg.backward and not skip and not args.frozen_lm_head:
            del d_weight, ws_b  # the autograd call allocates its own
            out["autograd"] = autograd_leg(cfg, hidden, weight, labels, g, q)
            out["autograd"]["vs_c_abi_step"] = out["autograd"]["ms_per_step"] / ms_per_step
        out["vendor_gemm"] = vendor_gemm(hidden, weight)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, args.cpu_sample_tokens)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())

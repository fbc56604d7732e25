"""Seeded synthetic inputs for the five benchmark configurations of the fused LM-head path, plus a small twin of each.

Generation is on the CPU with one ``torch.Generator`` per configuration (seed = 1000 + index), in fp32 then cast, so a CPU
checker and the GPU see identical bits.  hidden ~ N(0,1) -> bf16; weight ~ N(0, (3/sqrt(H))^2) -> bf16; labels uniform in
[0, V); masks and upstream gradients as each configuration states.
"""

from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional

import torch


@dataclasses.dataclass(frozen=True)
class LmHeadConfig:
    name: str
    index: int
    T: int
    H: int
    V: int
    temperature: float = 1.0
    backward: bool = True
    entropy: bool = True          # entropy output requested
    entropy_grad: bool = False    # entropy carries its own upstream gradient
    layout: str = "dense"         # "dense": n_seqs x seq_len; "packed": variable lengths
    n_seqs: int = 1
    mask: str = "none"            # "none" | "prefix50" | "suffix30_90"
    weight_scale: float = 3.0     # weight ~ N(0, (weight_scale / sqrt(H))^2)
    upstream: str = "randn"       # "randn": dlogprobs ~ N(0,1) * mask; "minus_one": the gradient of (-logprobs).sum()

    @property
    def fwd_flop(self) -> float:
        return 2.0 * self.T * self.V * self.H

    @property
    def total_flop(self) -> float:
        """Algorithmic work of one step: forward GEMM, and for training steps the logits recompute, dHidden and dW GEMMs."""
        return (8.0 if self.backward else 2.0) * self.T * self.V * self.H


CONFIGS: Dict[str, LmHeadConfig] = {
    c.name: c
    for c in [
        LmHeadConfig("qwen2.5-0.5b-fwd", 0, T=2048, H=896, V=151936, backward=False, n_seqs=4),
        LmHeadConfig("qwen2.5-1.5b-fwdbwd", 1, T=8192, H=1536, V=151936, n_seqs=8, mask="prefix50", entropy=False),
        LmHeadConfig("qwen2.5-7b-fwdbwd", 2, T=16384, H=3584, V=152064, temperature=0.6, entropy_grad=True, layout="packed"),
        LmHeadConfig("llama3.1-8b-fwdbwd", 3, T=32768, H=4096, V=128256, n_seqs=8, mask="suffix30_90", entropy=False),
        LmHeadConfig("qwen3-32b-fwd", 4, T=32768, H=5120, V=151936, backward=False, entropy=False, n_seqs=16),
    ]
}

# The long-context sweep of the reference's own harness (skyrl/benchmarks/bench_fused_linear_logprob.py:39-47, 90-97):
# H = 2048, the vocabulary of one TP=4 shard (62080) or the full one (248320), one sequence of S tokens,
# hidden ~ N(0,1), weight ~ N(0, 1/H), loss = (-logprobs).sum().  Not part of the five benchmark configurations; these
# are the shapes for which the fused path exists ("what makes 262k fit", model_utils.py:289-293).
for _i, (_s, _v) in enumerate([(65536, 62080), (262144, 62080), (65536, 248320), (262144, 248320)]):
    _c = LmHeadConfig(f"longctx-s{_s}-v{_v}", 5 + _i, T=_s, H=2048, V=_v, entropy=False, weight_scale=1.0, upstream="minus_one")
    CONFIGS[_c.name] = _c

# Same structure (masks, temperature, packing, ragged edges) at sizes a CPU checker finishes in seconds.
SMALL_TWINS: Dict[str, LmHeadConfig] = {
    "qwen2.5-0.5b-fwd": dataclasses.replace(CONFIGS["qwen2.5-0.5b-fwd"], T=4 * 96, H=128, V=1187 * 4),
    "qwen2.5-1.5b-fwdbwd": dataclasses.replace(CONFIGS["qwen2.5-1.5b-fwdbwd"], T=8 * 64, H=192, V=2374 * 2),
    "qwen2.5-7b-fwdbwd": dataclasses.replace(CONFIGS["qwen2.5-7b-fwdbwd"], T=700, H=256, V=594 * 8),
    "llama3.1-8b-fwdbwd": dataclasses.replace(CONFIGS["llama3.1-8b-fwdbwd"], T=8 * 80, H=256, V=501 * 8),
    "qwen3-32b-fwd": dataclasses.replace(CONFIGS["qwen3-32b-fwd"], T=16 * 40, H=320, V=1187 * 4),
}


def _packed_lengths(T: int, gen: torch.Generator, lo: int, hi: int) -> List[int]:
    lens: List[int] = []
    total = 0
    while total < T:
        n = int(torch.randint(lo, hi + 1, (1,), generator=gen).item())
        n = min(n, T - total)
        lens.append(n)
        total += n
    return lens


def make_inputs(cfg: LmHeadConfig, seed: Optional[int] = None) -> Dict[str, torch.Tensor]:
    """CPU tensors: hidden [T,H] bf16, weight [V,H] bf16, labels [T] int64, mask [T] fp32, dlogprobs [T] fp32 (if backward),
    dentropy [T] fp32 (if entropy_grad), cu_seqlens [n+1] int64."""
    gen = torch.Generator().manual_seed(1000 + cfg.index if seed is None else seed)
    T, H, V = cfg.T, cfg.H, cfg.V
    rows = max(1, (1 << 24) // H)  # generate hidden and weight in slabs: no [T,H] or [V,H] fp32 temporary
    hidden = torch.empty(T, H, dtype=torch.bfloat16)
    if T <= rows:  # (one draw for the sizes that existed before the slabs, so their bits stay what they were)
        hidden.copy_(torch.randn(T, H, generator=gen, dtype=torch.float32))
    else:
        for r0 in range(0, T, rows):
            r1 = min(T, r0 + rows)
            hidden[r0:r1] = torch.randn(r1 - r0, H, generator=gen, dtype=torch.float32).to(torch.bfloat16)
    weight = torch.empty(V, H, dtype=torch.bfloat16)
    for r0 in range(0, V, rows):
        r1 = min(V, r0 + rows)
        weight[r0:r1] = (torch.randn(r1 - r0, H, generator=gen, dtype=torch.float32) * (cfg.weight_scale / H**0.5)).to(torch.bfloat16)
    labels = torch.randint(0, V, (T,), generator=gen, dtype=torch.int64)

    if cfg.layout == "packed":
        scale = max(1, 16384 // T)
        lens = _packed_lengths(T, gen, max(2, 256 // scale), max(4, 4096 // scale))
    else:
        assert T % cfg.n_seqs == 0
        lens = [T // cfg.n_seqs] * cfg.n_seqs
    cu = torch.zeros(len(lens) + 1, dtype=torch.int64)
    cu[1:] = torch.tensor(lens, dtype=torch.int64).cumsum(0)

    mask = torch.ones(T, dtype=torch.float32)
    if cfg.mask == "prefix50":
        for i, n in enumerate(lens):
            mask[int(cu[i]) : int(cu[i]) + n // 2] = 0.0
    elif cfg.mask == "suffix30_90":
        fr = torch.rand(len(lens), generator=gen) * 0.6 + 0.3
        for i, n in enumerate(lens):
            keep = int(round(float(fr[i]) * n))
            mask[int(cu[i]) : int(cu[i]) + n - keep] = 0.0

    out = {"hidden": hidden, "weight": weight, "labels": labels, "mask": mask, "cu_seqlens": cu}
    if cfg.backward and cfg.upstream == "minus_one":
        out["dlogprobs"] = -mask
    elif cfg.backward:
        out["dlogprobs"] = torch.randn(T, generator=gen, dtype=torch.float32) * mask
    if cfg.entropy_grad:
        out["dentropy"] = torch.randn(T, generator=gen, dtype=torch.float32) * 0.01
    return out

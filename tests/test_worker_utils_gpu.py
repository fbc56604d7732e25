"""GPU parity of the fused log-probability drift statistics (skyrl_logprob_diff_metrics, skyrl_amd/worker_utils.py) against the
oracle's restatement of workers/worker_utils.py:34-58 in fp64, and against plain torch reductions at a size the oracle is not
needed for.  Maximum and minimum are compared exactly (they are fp32 values of the inputs), the means to fp32 accuracy."""

from __future__ import annotations

import ctypes

import pytest
import torch

from oracle import lmhead_oracle as O
from skyrl_amd import _lib
from skyrl_amd import worker_utils as WU

pytestmark = pytest.mark.gpu

PRE = "minibatch_rollout_logprobs_abs_diff"
ERR_NULL, ERR_SHAPE = -1, -2   # include/skyrl_lmhead.h


def _batch(shape, seed, masked=True):
    gen = torch.Generator().manual_seed(seed)
    rollout = torch.randn(shape, generator=gen) * 0.7 - 1.5
    lp = rollout + torch.randn(shape, generator=gen) * 0.05
    mask = (torch.rand(shape, generator=gen) > 0.3).float() if masked else None
    return lp, rollout, mask


@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (9, 57), (4, 1023), (2, 8192), (5, 8193), (64, 4099)])
@pytest.mark.parametrize("masked", [True, False])
def test_logprob_diff_metrics_match_oracle(shape, masked, cuda_device):
    lp, rollout, mask = _batch(shape, seed=shape[0] * 131 + shape[1], masked=masked)
    want = O.minibatch_rollout_logprob_diff_metrics(lp.double(), rollout.double(), None if mask is None else mask.double())
    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    got = WU.compute_minibatch_rollout_logprob_diff_metrics(to(lp), to(rollout), to(mask))
    assert list(got) == [f"{PRE}_mean", f"{PRE}_sq_mean", f"{PRE}_max", f"{PRE}_min"] and all(isinstance(v, float) for v in got.values())
    assert got[f"{PRE}_mean"] == pytest.approx(want[f"{PRE}_mean"], rel=2e-6, abs=1e-9)
    assert got[f"{PRE}_sq_mean"] == pytest.approx(want[f"{PRE}_sq_mean"], rel=2e-6, abs=1e-9)
    weighted = (lp - rollout).abs() * (1 if mask is None else mask)            # fp32, as the kernel forms it
    assert got[f"{PRE}_max"] == weighted.max().item() and got[f"{PRE}_min"] == weighted.min().item()
    lazy = WU.compute_minibatch_rollout_logprob_diff_metrics(to(lp), to(rollout), to(mask), sync_metrics=False)
    assert all(isinstance(v, torch.Tensor) and v.dim() == 0 and v.item() == got[k] for k, v in lazy.items())


def test_logprob_diff_metrics_special_cases(cuda_device):
    lp, rollout, mask = (t.to(cuda_device) for t in _batch((6, 40), seed=3))
    assert WU.compute_minibatch_rollout_logprob_diff_metrics(lp, None, mask) == {}
    # nothing counts: the clamped denominators give zeros, as in the reference
    zero = WU.compute_minibatch_rollout_logprob_diff_metrics(lp, rollout, torch.zeros_like(mask))
    assert list(zero.values()) == [0.0, 0.0, 0.0, 0.0]
    # fractional weights weigh the means and scale the extremes
    half = WU.compute_minibatch_rollout_logprob_diff_metrics(lp, rollout, torch.full_like(mask, 0.5))
    full = WU.compute_minibatch_rollout_logprob_diff_metrics(lp, rollout, None)
    assert half[f"{PRE}_mean"] == pytest.approx(full[f"{PRE}_mean"], rel=1e-6) and half[f"{PRE}_max"] == 0.5 * full[f"{PRE}_max"]
    # a NaN log-probability reaches every statistic, as with Tensor.max() / .sum()
    bad = lp.clone()
    bad[2, 5] = float("nan")
    got = WU.compute_minibatch_rollout_logprob_diff_metrics(bad, rollout, None)
    assert all(v != v for v in got.values())
    # [B, G, S] inputs, bf16 inputs, a mask that broadcasts, non-contiguous views
    cube = WU.compute_minibatch_rollout_logprob_diff_metrics(lp.reshape(2, 3, 40), rollout.reshape(2, 3, 40), mask.reshape(2, 3, 40))
    assert cube == WU.compute_minibatch_rollout_logprob_diff_metrics(lp, rollout, mask)
    col = WU.compute_minibatch_rollout_logprob_diff_metrics(lp, rollout, mask[:, :1])
    assert col == WU.compute_minibatch_rollout_logprob_diff_metrics(lp, rollout, mask[:, :1].expand(6, 40).contiguous())
    view = WU.compute_minibatch_rollout_logprob_diff_metrics(lp.t().contiguous().t(), rollout, mask)
    assert view == WU.compute_minibatch_rollout_logprob_diff_metrics(lp, rollout, mask)
    low = WU.compute_minibatch_rollout_logprob_diff_metrics(lp.bfloat16(), rollout.bfloat16(), mask)
    assert low == WU.compute_minibatch_rollout_logprob_diff_metrics(lp.bfloat16().float(), rollout.bfloat16().float(), mask)
    with pytest.raises(RuntimeError):
        WU.compute_minibatch_rollout_logprob_diff_metrics(lp.cpu(), rollout.cpu(), None)
    with pytest.raises(ValueError):
        WU.compute_minibatch_rollout_logprob_diff_metrics(lp[:0], rollout[:0], None)
    torch.library.opcheck(WU.logprob_diff_terms, (lp, rollout, mask), test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(WU.logprob_diff_terms, (lp, rollout, None), test_utils=("test_schema", "test_faketensor"))


def test_logprob_diff_c_abi_argument_errors(cuda_device):
    lib = _lib.load()
    x = torch.zeros(64, device=cuda_device)
    out, part = torch.empty(4, device=cuda_device), torch.empty(5 * 256, device=cuda_device)
    stream = torch.cuda.current_stream(cuda_device).cuda_stream
    call = lambda a=x.data_ptr(), b=x.data_ptr(), n=64, o=out.data_ptr(), p=part.data_ptr(): lib.skyrl_logprob_diff_metrics(  # noqa: E731
        a, b, None, n, o, p, stream)
    assert call() == 0
    torch.cuda.synchronize()
    assert out.tolist() == [0.0, 0.0, 0.0, 0.0]
    assert call(a=None) == ERR_NULL and call(b=None) == ERR_NULL and call(o=None) == ERR_NULL and call(p=None) == ERR_NULL
    assert call(n=0) == ERR_SHAPE and call(n=-3) == ERR_SHAPE
    assert isinstance(ctypes.c_int(call()).value, int)


def test_logprob_diff_metrics_full_size_and_graph_replay(cuda_device):
    """4.2 M tokens against torch reductions in fp64; bit-identical on a second call; captured once and replayed on new data
    with eager work in between, every replay equal to the eager result."""
    gen = torch.Generator(device=cuda_device).manual_seed(9)
    shape = (1024, 4096)
    rollout = torch.randn(shape, device=cuda_device, generator=gen) - 1.5
    lp = rollout + torch.randn(shape, device=cuda_device, generator=gen) * 0.03
    mask = (torch.rand(shape, device=cuda_device, generator=gen) > 0.4).float()
    got = WU.logprob_diff_terms(lp, rollout, mask)
    d = (lp - rollout).abs()
    assert got[0].item() == pytest.approx(((d.double() * mask).sum() / mask.sum()).item(), rel=1e-6)
    assert got[1].item() == pytest.approx(((d.double() ** 2 * mask).sum() / mask.sum()).item(), rel=1e-6)
    assert got[2].item() == (d * mask).max().item() and got[3].item() == (d * mask).min().item()
    assert torch.equal(got, WU.logprob_diff_terms(lp, rollout, mask))
    a, b, m = lp[:16].clone(), rollout[:16].clone(), mask[:16].clone()
    side = torch.cuda.Stream(device=cuda_device)
    side.wait_stream(torch.cuda.current_stream(cuda_device))
    with torch.cuda.stream(side):
        for _ in range(2):
            WU.logprob_diff_terms(a, b, m)
    torch.cuda.current_stream(cuda_device).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = WU.logprob_diff_terms(a, b, m)
    for r in (16, 32, 48):
        a.copy_(lp[r:r + 16]), b.copy_(rollout[r:r + 16]), m.copy_(mask[r:r + 16])
        graph.replay()
        torch.cuda.synchronize()
        eager = WU.logprob_diff_terms(lp[r:r + 16].contiguous(), rollout[r:r + 16].contiguous(), mask[r:r + 16].contiguous())
        torch.cuda.synchronize()
        assert torch.equal(captured, eager), r

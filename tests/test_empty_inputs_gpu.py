"""Empty micro-batches through the public wrappers: no launch, no misleading error -- the shapes and values that the
reference's torch expressions give on empty tensors (sums 0, clamped denominators 1, the mean of nothing NaN)."""

from __future__ import annotations

import math
from types import SimpleNamespace

import pytest
import torch

pytestmark = pytest.mark.gpu

V, H = 512, 128


def test_empty_inputs_through_the_wrappers(cuda_device):
    from skyrl_amd import model_utils as MU
    from skyrl_amd import model_wrapper as MW
    from skyrl_amd import mtp_soft_ce as M
    from skyrl_amd import off_policy_correction as OPC
    from skyrl_amd import policy_loss as PL
    from skyrl_amd import torch_utils as TU
    dev = cuda_device
    W = torch.randn(V, H, device=dev).bfloat16()
    z = lambda *s: torch.zeros(*s, device=dev)  # noqa: E731
    ids = lambda *s: torch.zeros(*s, dtype=torch.long, device=dev)  # noqa: E731
    hid = lambda *s: torch.zeros(*s, device=dev).bfloat16()  # noqa: E731
    cfg = SimpleNamespace(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.2, clip_ratio_c=3.0, off_policy_correction=None,
                          use_kl_loss=False, use_entropy_loss=False)
    # materialised logits
    assert TU.logprobs_from_logits(z(0, 5, V), ids(0, 5)).shape == (0, 5)
    assert TU.logprobs_from_logits(z(2, 0, V), ids(2, 0)).shape == (2, 0)
    assert TU.chunked_entropy_from_logits(z(0, 4, V)).shape == (0, 4) and TU.vocab_parallel_entropy(z(0, 4, V)).shape == (0, 4)
    assert MW.action_log_probs_from_logits(z(0, 6, V), ids(0, 6), 2, torch.ones(0, 6, dtype=torch.long, device=dev), 1.0).shape == (0, 2)
    # hidden states
    assert MU.from_parallel_hidden_to_logprobs(hid(0, 4, H), W, ids(0, 4), 0, V, None).shape == (0, 3)
    assert M.soft_ce_from_hidden(hid(0, 4, H), hid(0, 4, H), W).shape == (0, 4)
    values, columns = M.topk_logits_from_hidden(hid(0, H), W, 8)
    assert values.shape == (0, 8) and columns.shape == (0, 8) and columns.dtype == torch.int64
    assert M.soft_ce_topk_from_hidden(hid(0, 4, H), hid(0, 4, H), W, 8).shape == (0, 4)
    with pytest.raises(ValueError, match="bad k"):
        M.topk_logits_from_hidden(hid(0, H), W, 0)
    # the consumers
    for shape in ((0, 4), (3, 0)):
        loss, metrics = PL.ppo_policy_loss(z(*shape), z(*shape), z(*shape), cfg, z(*shape))
        assert loss.item() == 0.0 and metrics["clip_ratio"] == 0.0
        kld = PL.compute_approx_kl(z(*shape), z(*shape), z(*shape))
        assert kld.shape == shape and kld.dtype == torch.float32
        assert PL.masked_mean(z(*shape), z(*shape)).item() == 0.0 and math.isnan(PL.masked_mean(z(*shape), None).item())
        assert PL.masked_mean(z(*shape), z(*shape), dim=-1).shape == shape[:1]
        tis, metrics, mask = OPC.compute_off_policy_correction(z(*shape), z(*shape), z(*shape),
                                                               SimpleNamespace(tis_ratio_type="token", token_tis_ratio_clip_high=2.0))
        assert tis.shape == shape and mask.shape == shape and metrics["is_ratio_mean"] == 0.0
        with pytest.raises(ValueError, match="at least one token"):
            PL.actor_loss(z(*shape), z(*shape), z(*shape), cfg, z(*shape))
    assert math.isnan(PL.approx_kl_loss(z(0, 4), z(0, 4), z(0, 4)).item())          # the mean over no rows
    assert PL.approx_kl_loss(z(3, 0), z(3, 0), z(3, 0)).item() == 0.0               # rows without tokens count as 0
    assert PL.masked_mean(z(3, 0), z(3, 0), dim=-1).tolist() == [0.0, 0.0, 0.0]
    # gradients flow (as zeros of the right shape) through the empty results
    x = z(0, 4).requires_grad_(True)
    (PL.compute_approx_kl(x, z(0, 4), None).sum() + PL.masked_mean(x, z(0, 4))).backward()
    assert x.grad.shape == (0, 4)

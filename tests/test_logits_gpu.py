"""GPU parity of the logits-input kernels (skyrl_logits_fwd / skyrl_logits_bwd and their reference-shaped wrappers) against
the oracle's restatements of logprobs_from_logits_v2, chunked_entropy_from_logits (skyrl/backends/skyrl_train/utils/
torch_utils.py:58-177), DistributedLogprob (distributed/megatron/model_utils.py:66-138) and the entropy gradient of
_VocabParallelEntropy (:1316-1345), computed in fp64 from the same bf16 / fp32 logits.

Tolerances: log-probabilities 1e-4 absolute and entropy 1e-4 relative on fp32 logits (2e-2 / 1e-2 are the path's stated bounds);
gradients 1e-5 relative to the row's largest entry for fp32 logits, half a bf16 ulp of it for bf16 logits.
"""

from __future__ import annotations

import ctypes
import math

import pytest
import torch

from oracle import lmhead_oracle as O
from skyrl_amd import _lib, torch_utils as TU

pytestmark = pytest.mark.gpu

ERR_NULL, ERR_SHAPE, ERR_ALIGN, ERR_ARG = -1, -2, -3, -5   # include/skyrl_lmhead.h


def _case(T, V, dtype, seed, scale=3.0):
    gen = torch.Generator().manual_seed(seed)
    logits = (torch.randn(T, V, generator=gen) * scale).to(dtype)
    labels = torch.randint(0, V, (T,), generator=gen)
    g = torch.randn(T, generator=gen)
    q = torch.randn(T, generator=gen) * 0.1
    return logits, labels, g, q


def _exact(logits, labels, g, q, temperature):
    """fp64 values and gradient of sum(g * logprob + q * entropy) for logits / temperature."""
    x = logits.double().requires_grad_(True)
    lsm = torch.log_softmax(x / temperature, -1)
    lp = lsm.gather(-1, labels[:, None])[:, 0]
    ent = torch.distributions.Categorical(logits=x / temperature).entropy()
    (lp * g.double() + ent * q.double()).sum().backward()
    return lp.detach(), ent.detach(), x.grad


@pytest.mark.parametrize("T,V,dtype,temperature", [
    (37, 5000, torch.float32, 1.0),
    (130, 20011, torch.bfloat16, 0.7),     # a vocabulary that is not a multiple of a 16-byte piece
    (5, 151936, torch.bfloat16, 1.0),      # a full-size row
    (64, 7, torch.float32, 1.3),           # rows shorter than one piece
    (3, 2049, torch.bfloat16, 1.0),
    (1, 1, torch.float32, 1.0),
])
def test_logits_forward_and_backward_match_fp64(T, V, dtype, temperature, cuda_device):
    logits, labels, g, q = _case(T, V, dtype, seed=T + V)
    want_lp, want_ent, want_grad = _exact(logits, labels, g, q, temperature)
    d, y = logits.to(cuda_device), labels.to(cuda_device)
    lp, ent, lse, pz = TU.logits_fwd(d, y, 1.0 / temperature, True)
    assert (lp.cpu().double() - want_lp).abs().max() <= 1e-4
    assert ((ent.cpu().double() - want_ent).abs() / want_ent.abs().clamp_min(1e-3)).max() <= 1e-4
    assert (lse.cpu().double() - torch.logsumexp(logits.double() / temperature, -1)).abs().max() <= 1e-4
    grad = TU.logits_bwd(d, y, lse, pz, g.to(cuda_device), q.to(cuda_device), 1.0 / temperature)
    assert grad.dtype == dtype and grad.shape == (T, V)
    # errors are measured against the size of the row's terms g / temperature and p * g / temperature, not against their
    # difference: where the label's probability is close to 1 the two nearly cancel, in any fp32 evaluation
    row_scale = torch.maximum(want_grad.abs().amax(-1, keepdim=True), ((g.abs() + q.abs()) / temperature).double()[:, None]).clamp_min(1e-30)
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -8
    assert ((grad.cpu().double() - want_grad).abs() / row_scale).max() <= tol
    # the gradient written over the logits themselves is the same, bit for bit
    clone = d.clone()
    TU.logits_bwd_(clone, y, lse, pz, g.to(cuda_device), q.to(cuda_device), 1.0 / temperature)
    assert torch.equal(clone, grad)
    # log-probability alone (no entropy statistics), entropy alone (no labels)
    lp2, ent2, lse2, _ = TU.logits_fwd(d, y, 1.0 / temperature, False)
    assert torch.equal(lp2, lp) and torch.equal(lse2, lse) and float(ent2.abs().max()) == 0.0
    lp3, ent3, _, _ = TU.logits_fwd(d, None, 1.0 / temperature, True)
    assert torch.equal(ent3, ent) and float(lp3.abs().max()) == 0.0


def test_logits_rows_that_do_not_allow_vector_loads_and_strided_rows(cuda_device):
    """A row pitch that is not a multiple of 16 bytes, a base that is not 16-byte aligned, rows with padding between them."""
    T, V = 33, 3001
    logits, labels, g, q = _case(T, V, torch.bfloat16, seed=4)
    want_lp, want_ent, want_grad = _exact(logits, labels, g, q, 1.0)
    padded = torch.zeros(T, V + 7, dtype=torch.bfloat16, device=cuda_device)      # pitch 3008 * 2 bytes: 16-byte pieces
    padded[:, :V] = logits.to(cuda_device)
    odd = torch.zeros(T * (V + 3) + 1, dtype=torch.bfloat16, device=cuda_device)[1:].reshape(T, V + 3)   # 2-byte aligned base
    odd[:, :V] = logits.to(cuda_device)
    y, gd, qd = labels.to(cuda_device), g.to(cuda_device), q.to(cuda_device)
    ref = None
    for view in (padded[:, :V], odd[:, :V]):
        lp, ent, lse, pz = TU.logits_fwd(view, y, 1.0, True)
        assert (lp.cpu().double() - want_lp).abs().max() <= 1e-4 and (ent.cpu().double() - want_ent).abs().max() <= 1e-3
        grad = TU.logits_bwd(view, y, lse, pz, gd, qd, 1.0)
        row_scale = want_grad.abs().amax(-1, keepdim=True)
        assert ((grad.cpu().double() - want_grad).abs() / row_scale).max() <= 2.0 ** -8
        if ref is not None:   # the two load paths add the same numbers in different orders
            assert (lp - ref[0]).abs().max() <= 1e-5 and (grad.float() - ref[1].float()).abs().max() <= 2.0 ** -8 * float(row_scale.max())
        ref = (lp, grad)
        before = view.clone()
        TU.logits_bwd_(view, y, lse, pz, gd, qd, 1.0)                # in place into a strided view: the padding stays untouched
        assert torch.equal(view, grad)
    assert float(padded[:, V:].abs().max()) == 0.0 and float(odd[:, V:].abs().max()) == 0.0 and before.shape == (T, V)


def test_logits_extreme_rows(cuda_device):
    """Rows of equal logits (-ln V), a row with one dominant logit, very negative rows (no underflow to log 0), -inf entries
    (masked vocabulary: probability exactly 0), rows without upstream gradient (exact zeros)."""
    V = 4099
    rows = torch.zeros(6, V)
    rows[1, 17] = 80.0
    rows[2] = -300.0                                                    # exp(-300) is 0 in fp32: a maximum that started at 0 would give log 0
    rows[3] = torch.linspace(-50, 50, V)
    rows[4, ::2] = -math.inf
    rows[5] = torch.randn(V, generator=torch.Generator().manual_seed(0)) * 10
    labels = torch.tensor([5, 17, 9, V - 1, 1, 3])
    d = rows.to(cuda_device)
    lp, ent, lse, pz = TU.logits_fwd(d, labels.to(cuda_device), 1.0, True)
    want_lp = torch.log_softmax(rows.double(), -1).gather(-1, labels[:, None])[:, 0]
    want_ent = torch.distributions.Categorical(logits=rows.double()).entropy()
    assert torch.isfinite(lp).all() and torch.isfinite(ent).all()
    assert (lp.cpu().double() - want_lp).abs().max() <= 1e-4 and (ent.cpu().double() - want_ent).abs().max() <= 1e-4
    assert lp[0].item() == pytest.approx(-math.log(V), abs=1e-5) and ent[0].item() == pytest.approx(math.log(V), abs=1e-5)
    assert lp[2].item() == pytest.approx(-math.log(V), abs=1e-4)
    assert ent[4].item() == pytest.approx(math.log((V - 1) // 2), abs=1e-5)
    g = torch.tensor([1.0, -2.0, 0.5, 0.0, 1.0, 0.0], device=cuda_device)
    grad = TU.logits_bwd(d, labels.to(cuda_device), lse, None, g, None, 1.0)
    assert float(grad[3].abs().max()) == 0.0 and float(grad[5].abs().max()) == 0.0
    assert float(grad[4, ::2].abs().max()) == 0.0                       # masked columns get no gradient
    assert torch.isfinite(grad).all()
    assert grad.sum(-1).abs().max() <= 1e-4                              # rows of (onehot - p) * g sum to zero


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_reference_shaped_wrappers_match_oracle(dtype, cuda_device):
    gen = torch.Generator().manual_seed(3)
    B, S, V = 3, 41, 2500
    logits = (torch.randn(B, S, V, generator=gen) * 2).to(dtype)
    labels = torch.randint(0, V, (B, S), generator=gen)
    mask = (torch.rand(B, S, generator=gen) > 0.3).to(dtype)
    d, y = logits.to(cuda_device), labels.to(cuda_device)
    want = O.logprobs_from_logits_v2(logits.double(), labels)
    got = TU.logprobs_from_logits(d, y, inplace_backward=False)
    assert got.dtype == torch.float32 and got.shape == (B, S) and (got.cpu().double() - want).abs().max() <= 1e-4
    v2 = TU.logprobs_from_logits_v2(d, y)
    assert v2.dtype == dtype and (v2.cpu().double() - want).abs().max() <= (1e-4 if dtype == torch.float32 else 0.05)
    if dtype == torch.bfloat16:      # inside the error ball of the reference's own bf16 path around the exact value
        ref_bf16 = O.logprobs_from_logits_v2(logits, labels)
        assert (v2.cpu().double() - want).abs().max() <= (ref_bf16.double() - want).abs().max() + 1e-6
    ent_want = O.chunked_entropy_from_logits(logits.double(), mask.double())
    ent = TU.chunked_entropy_from_logits(d, attention_mask=mask.to(cuda_device), chunk_size=7)
    assert ent.dtype == dtype and not ent.requires_grad
    assert (ent.cpu().double() - ent_want).abs().max() <= (1e-4 if dtype == torch.float32 else 0.05)
    assert bool((ent.cpu()[mask == 0] == 0).all())
    with pytest.raises(ValueError):
        TU.chunked_entropy_from_logits(d, attention_mask=mask.to(cuda_device)[:, :-1])
    with pytest.raises(ValueError):
        TU.chunked_entropy_from_logits(d, chunk_size=0)
    # gradients through autograd: out of place, and in place over a non-leaf logits tensor
    g = torch.randn(B, S, generator=gen)
    x = logits.double().requires_grad_(True)
    (O.logprobs_from_logits_v2(x, labels) * g.double()).sum().backward()
    leaf = d.clone().requires_grad_(True)
    (TU.logprobs_from_logits(leaf, y, inplace_backward=False) * g.to(cuda_device)).sum().backward()
    scale = x.grad.abs().amax(-1, keepdim=True)
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -8
    assert ((leaf.grad.cpu().double() - x.grad).abs() / scale).max() <= tol
    leaf2 = d.clone().requires_grad_(True)
    mid = leaf2 * 1.0                                                     # what a model's output is: not a leaf
    (TU.logprobs_from_logits(mid, y, inplace_backward=True) * g.to(cuda_device)).sum().backward()
    assert torch.equal(leaf2.grad, leaf.grad) and torch.equal(mid.detach(), leaf.grad)   # the logits now hold their gradient
    # entropy with gradient, and both outputs of one pass
    leaf3 = d.clone().requires_grad_(True)
    ent_g = TU.chunked_entropy_from_logits(leaf3, requires_grad=True)
    (ent_g.float() * g.to(cuda_device)).sum().backward()
    x2 = logits.double().requires_grad_(True)
    (torch.distributions.Categorical(logits=x2).entropy() * g.double()).sum().backward()
    scale2 = x2.grad.abs().amax(-1, keepdim=True)
    assert ((leaf3.grad.cpu().double() - x2.grad).abs() / scale2).max() <= (1e-5 if dtype == torch.float32 else 2.0 ** -7)
    both_lp, both_ent = TU.logprobs_and_entropy_from_logits(d, y, temperature=0.6)
    assert (both_lp.cpu().double() - O.logprobs_from_logits_v2(logits.double() / 0.6, labels)).abs().max() <= 1e-4
    assert (both_ent.cpu().double() - O.chunked_entropy_from_logits(logits.double() / 0.6)).abs().max() <= 1e-4


def test_distributed_logprob_adapters_match_oracle(cuda_device):
    gen = torch.Generator().manual_seed(8)
    B, S, V, start = 2, 33, 1800, 500
    logits = torch.randn(B, S, V, generator=gen).bfloat16()
    target = torch.randint(start, start + V, (B, S), generator=gen)
    target[0, :4] = torch.tensor([0, start - 1, start + V, 10 ** 9])       # outside the shard on either side
    g = torch.randn(B, S, generator=gen)
    lp_want, softmax, tmask, masked = O.distributed_logprob_forward(logits.double(), target, start, start + V)
    grad_want = O.distributed_logprob_backward(softmax, tmask, masked, g.double())
    for chunked in (False, True):
        leaf = logits.to(cuda_device).requires_grad_(True)
        if chunked:
            lp = TU.ChunkedDistributedLogprob.apply(leaf, target.to(cuda_device), start, start + V, 8, None, False)
        else:
            lp = TU.DistributedLogprob.apply(leaf, target.to(cuda_device), start, start + V, None, False)
        assert lp.dtype == torch.float32 and lp.shape == (B, S)
        assert (lp.cpu().double() - lp_want).abs().max() <= 1e-4 and bool((lp.cpu()[tmask] == 0).all())
        (lp * g.to(cuda_device)).sum().backward()
        assert leaf.grad.dtype == torch.bfloat16
        scale = grad_want.abs().amax(-1, keepdim=True)
        assert ((leaf.grad.cpu().double() - grad_want).abs() / scale).max() <= 2.0 ** -8
    with torch.no_grad():
        out = TU.DistributedLogprob.apply(logits.to(cuda_device), target.to(cuda_device), start, start + V, None, True)
    assert torch.equal(out, lp.detach())
    rolled_want = O.distributed_logprob_forward(logits.double(), target.roll(-1, -1), start, start + V)[0][:, :-1]
    got = TU.from_parallel_logits_to_logprobs(logits.to(cuda_device), target.to(cuda_device), start, start + V, None, inference_only=True)
    assert got.shape == (B, S - 1) and (got.cpu().double() - rolled_want).abs().max() <= 1e-4


def test_logits_c_abi_argument_errors(cuda_device):
    lib = _lib.load()
    T, V = 8, 640
    x = torch.randn(T, V, device=cuda_device)
    y = torch.zeros(T, dtype=torch.int64, device=cuda_device)
    out = torch.empty(T, device=cuda_device)
    p = lambda t: t.data_ptr()  # noqa: E731
    fwd = lambda **kw: lib.skyrl_logits_fwd(kw.get("logits", p(x)), kw.get("dtype", 1), kw.get("ld", V), kw.get("labels", p(y)), kw.get("T", T),  # noqa: E731
                                            V, kw.get("rt", 1.0), kw.get("lp", p(out)), None, None, None, None)
    assert fwd() == 0
    assert fwd(logits=ctypes.c_void_p(0)) == ERR_NULL and fwd(labels=None) == ERR_NULL and fwd(lp=None) == ERR_NULL
    assert fwd(dtype=2) == ERR_ARG and fwd(rt=0.0) == ERR_ARG and fwd(rt=float("nan")) == ERR_ARG
    assert fwd(ld=V - 1) == ERR_SHAPE and fwd(T=0) == ERR_SHAPE
    assert fwd(logits=p(x) + 2) == ERR_ALIGN
    grad = torch.empty(T, V, device=cuda_device)
    bwd = lambda dst, ldd, g=p(out): lib.skyrl_logits_bwd(p(x), 1, V, p(y), p(out), None, g, None, T, V, 1.0, dst, ldd, None)  # noqa: E731
    assert bwd(p(grad), V) == 0 and bwd(p(x), V) == 0                     # apart, or exactly in place
    assert bwd(p(x) + 4 * V, V) == ERR_ARG                                # overlapping the logits any other way
    assert bwd(p(grad), V - 1) == ERR_SHAPE and bwd(None, V) == ERR_NULL and bwd(p(grad), V, None) == ERR_NULL
    torch.cuda.synchronize()


def test_logits_ops_opcheck(cuda_device):
    x = torch.randn(12, 300, device=cuda_device).bfloat16()
    y = torch.randint(0, 300, (12,), device=cuda_device)
    torch.library.opcheck(TU.logits_fwd, (x, y, 1.0, True), test_utils=("test_schema", "test_faketensor"))
    lp, ent, lse, pz = TU.logits_fwd(x, y, 1.0, True)
    torch.library.opcheck(TU.logits_bwd, (x, y, lse, pz, lp, ent, 1.0), test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(TU.logits_bwd_, (x.clone(), y, lse, pz, lp, ent, 1.0), test_utils=("test_schema", "test_faketensor"))


def test_logits_full_size_properties(cuda_device):
    """16384 rows of 152064 bf16 logits (4.6 GiB): sampled rows against fp64, the entropy bounds, rows of the gradient that
    sum to zero, nothing of the matrix's size allocated by the forward or by the in-place backward."""
    T, V = 16384, 152064
    gen = torch.Generator(device=cuda_device).manual_seed(0)
    logits = torch.empty(T, V, dtype=torch.bfloat16, device=cuda_device)
    for r in range(0, T, 2048):
        logits[r:r + 2048] = (torch.randn(2048, V, device=cuda_device, generator=gen) * 3).bfloat16()
    labels = torch.randint(0, V, (T,), device=cuda_device, generator=gen)
    g = torch.randn(T, device=cuda_device, generator=gen)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    lp, ent, lse, pz = TU.logits_fwd(logits, labels, 1.0, True)
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated() - base < (1 << 20)
    rows = torch.randperm(T, generator=torch.Generator().manual_seed(1))[:16].to(cuda_device)
    z = logits[rows].double()
    want_lp = torch.log_softmax(z, -1).gather(-1, labels[rows][:, None])[:, 0]
    assert (lp[rows].double() - want_lp).abs().max() <= 1e-4
    assert (ent[rows].double() - torch.distributions.Categorical(logits=z).entropy()).abs().max() <= 1e-4
    assert bool((lp <= 0).all()) and bool((ent >= 0).all()) and bool((ent <= math.log(V) + 1e-3).all())
    want_grad = (torch.nn.functional.one_hot(labels[rows], V) - torch.softmax(z, -1)) * g[rows].double()[:, None]
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    TU.logits_bwd_(logits, labels, lse, None, g, None, 1.0)
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated() - base < (1 << 20)
    got = logits[rows].double()
    assert ((got - want_grad).abs() / want_grad.abs().amax(-1, keepdim=True)).max() <= 2.0 ** -8
    assert bool(torch.isfinite(logits[:512]).all())


def test_vocab_parallel_entropy_wrappers_match_library(cuda_device):
    """vocab_parallel_entropy / _weighted_sum (model_utils.py:1316-1440): values and the gradient
    softmax * (sum softmax * logits - logits) * grad, against torch.distributions in fp64."""
    gen = torch.Generator().manual_seed(12)
    S, V = 57, 3000
    logits = (torch.randn(1, S, V, generator=gen) * 2).bfloat16()
    weights = (torch.rand(S, generator=gen) > 0.4).float()
    x = logits.double().requires_grad_(True)
    ent64 = torch.distributions.Categorical(logits=x).entropy()
    (ent64[0] * weights.double()).sum().backward()
    leaf = logits.to(cuda_device).requires_grad_(True)
    ent = TU.vocab_parallel_entropy(leaf, chunk_size=0, chunk_memory_mb=64)
    assert ent.shape == (1, S) and ent.dtype == torch.bfloat16
    assert (ent.detach().cpu().double() - ent64.detach()).abs().max() <= 0.05
    total = TU.vocab_parallel_entropy_weighted_sum(leaf, weights.to(cuda_device), chunk_size=16)
    total.backward()
    scale = x.grad.abs().amax(-1, keepdim=True).clamp_min(1e-30)
    assert ((leaf.grad.cpu().double() - x.grad).abs() / scale)[0][weights > 0].max() <= 2.0 ** -7
    assert float(leaf.grad[0][(weights == 0).to(cuda_device)].abs().max()) == 0.0
    with pytest.raises(ValueError):
        TU.vocab_parallel_entropy(leaf, chunk_size=-1)
    with pytest.raises(ValueError):
        TU.vocab_parallel_entropy(leaf, chunk_size=0, chunk_memory_mb=0)


@pytest.mark.parametrize("layout", ["attention_mask", "sub_sequences"])
@pytest.mark.parametrize("with_loss_mask", [False, True])
def test_vocab_parallel_entropy_packed_sequences_matches_oracle(layout, with_loss_mask, cuda_device):
    """The packed action-token entropy on materialised logits (model_utils.py:1001-1087): value and gradient against the
    oracle's restatement of the reference's packed-weight route applied to fp64 entropies."""
    import numpy as np

    gen = torch.Generator().manual_seed(34)
    V = 900
    if layout == "attention_mask":
        L, num_actions = 40, 17
        real = [40, 23, 31, 5, 1]
        am = torch.zeros(len(real), L, dtype=torch.long)
        am[0] = 1
        am[1, L - 23:] = 1
        am[2, :31] = 1
        am[3, 10:15] = 1
        am[4, L - 1] = 1
        padded = [r + (-r) % 8 for r in real]
        sub = None
    else:
        L, num_actions = 48, 30
        sub = [[9, 1, 14], [20, 6], [33]]
        padded = [16, 8, 16, 24, 8, 40]
        am = torch.ones(len(sub), L, dtype=torch.long)
    B = am.shape[0]
    cu = torch.tensor([0] + list(np.cumsum(padded)))
    T = int(cu[-1])
    logits = (torch.randn(1, T, V, generator=gen) * 2).float()
    loss_mask = (torch.rand(B, num_actions, generator=gen) > 0.35).float() if with_loss_mask else None
    x = logits.double().requires_grad_(True)
    ent64 = torch.distributions.Categorical(logits=x).entropy().squeeze(0)
    want, want_loss = O.packed_action_entropy(ent64, cu, L, num_actions, am, None if loss_mask is None else loss_mask.double(), sub)
    want_loss.backward()
    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    leaf = logits.to(cuda_device).requires_grad_(True)
    got, got_loss = TU.vocab_parallel_entropy_packed_sequences(leaf, to(cu), L, num_actions, to(am), to(loss_mask), None,
                                                               sub_seq_lengths=sub, chunk_size=0)
    assert got.dim() == 0 and not got.requires_grad and got_loss.requires_grad
    assert want.item() > 0.5
    assert got.item() == pytest.approx(want.item(), rel=1e-4) and got_loss.item() == pytest.approx(want.item(), rel=1e-4)
    got_loss.backward()
    err = (leaf.grad.cpu().double() - x.grad).abs().max().item()
    assert err <= 1e-5 * x.grad.abs().max().item(), err
    assert bool(((leaf.grad.cpu() != 0).any(-1) == (x.grad != 0).any(-1)).all())       # the same tokens carry gradient


def test_packed_logits_wrapper_all_layouts_with_gradient(cuda_device):
    """from_parallel_logits_to_logprobs_packed_sequences (model_utils.py:566-710) end to end -- labels kernel, logits kernel,
    scatter kernel -- in the three layouts, against the oracle's statement of the same pipeline (per-sequence roll, the
    materialised-logits log-probability, scatter-back), values and gradient."""
    dev = cuda_device
    V = 515
    gen = torch.Generator().manual_seed(52)
    true_lens = [9, 1, 17, 13, 6]
    padded = [10, 2, 17, 16, 6]
    cu = torch.cat([torch.zeros(1, dtype=torch.long), torch.tensor(padded).cumsum(0)])
    T = int(cu[-1])
    logits = (torch.randn(1, T, V, generator=gen) * 2).float()
    tokens = torch.randint(0, V, (1, T), generator=gen)
    rolled = O.packed_rolled_targets(tokens[0], cu)
    L = 20
    am = torch.zeros(len(true_lens), L, dtype=torch.bool)
    for b, n in enumerate(true_lens):
        am[b, L - n:] = True
    sub = [[9, 1], [17], [13, 6]]
    cases = {"plain": (dict(), len(padded), L), "mask": (dict(attention_mask=am), len(padded), L),
             "sub": (dict(sub_seq_lengths=sub), len(sub), 30)}
    for name, (kw, rows, seqlen) in cases.items():
        x = logits.double().requires_grad_(True)
        probs = O.distributed_logprob_forward(x, rolled[None], 0, V)[0][0]
        want = O.packed_scatter_back(probs, cu, rows, seqlen, **kw)
        G = torch.randn(want.shape, generator=gen)
        (want * G.double()).sum().backward()
        leaf = logits.to(dev).requires_grad_(True)
        dkw = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in kw.items()}
        got = TU.from_parallel_logits_to_logprobs_packed_sequences(leaf, tokens.to(dev), cu.to(dev), seqlen, 0, V, None, **dkw)
        assert got.shape == want.shape and got.dtype == torch.float32, name
        assert (got.detach().cpu().double() - want.detach()).abs().max() <= 1e-4, name
        assert torch.equal(got.detach().cpu() == 0, want.detach() == 0), name
        (got * G.to(dev)).sum().backward()
        err = (leaf.grad.cpu().double() - x.grad).abs().max().item()
        assert err <= 1e-5 * max(1.0, x.grad.abs().max().item()), (name, err)


def test_logits_entry_points_replay_from_a_hip_graph(cuda_device):
    """Forward, backward and the in-place backward captured in one HIP graph; three replays on new logits, with eager work in
    between, each reproduce the eager results bit for bit."""
    T, V = 200, 5003
    logits = torch.zeros(T, V, dtype=torch.bfloat16, device=cuda_device)
    labels = torch.zeros(T, dtype=torch.int64, device=cuda_device)
    g = torch.zeros(T, device=cuda_device)
    q = torch.zeros(T, device=cuda_device)

    def step():
        lp, ent, lse, pz = TU.logits_fwd(logits, labels, 0.9, True)
        grad = TU.logits_bwd(logits, labels, lse, pz, g, q, 0.9)
        over = logits.clone()
        TU.logits_bwd_(over, labels, lse, None, g, None, 0.9)
        return lp, ent, grad, over

    def refill(seed):
        gen_ = torch.Generator().manual_seed(seed)
        logits.copy_((torch.randn(T, V, generator=gen_) * 3).bfloat16())
        labels.copy_(torch.randint(0, V, (T,), generator=gen_))
        g.copy_(torch.randn(T, generator=gen_))
        q.copy_(torch.randn(T, generator=gen_) * 0.1)

    refill(0)
    side = torch.cuda.Stream(device=cuda_device)
    side.wait_stream(torch.cuda.current_stream(cuda_device))
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream(cuda_device).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for seed in (1, 2, 3):
        refill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_logits_random_shapes_against_fp64(cuda_device):
    """Thirty random (T, V, dtype, temperature, row pitch) cases, ragged ends and unaligned pitches included."""
    rng = torch.Generator().manual_seed(2024)
    for case in range(30):
        T = int(torch.randint(1, 70, (1,), generator=rng))
        V = int(torch.randint(1, 9000, (1,), generator=rng))
        dtype = torch.bfloat16 if case % 2 else torch.float32
        temperature = float(torch.rand(1, generator=rng)) * 1.5 + 0.3
        pad = int(torch.randint(0, 9, (1,), generator=rng))
        logits, labels, g, q = _case(T, V, dtype, seed=1000 + case)
        want_lp, want_ent, want_grad = _exact(logits, labels, g, q, temperature)
        wide = torch.zeros(T, V + pad, dtype=dtype, device=cuda_device)
        wide[:, :V] = logits.to(cuda_device)
        view, y = wide[:, :V], labels.to(cuda_device)
        lp, ent, lse, pz = TU.logits_fwd(view, y, 1.0 / temperature, True)
        tag = (case, T, V, dtype, pad)
        assert (lp.cpu().double() - want_lp).abs().max() <= 1e-4, tag
        assert (ent.cpu().double() - want_ent).abs().max() <= 1e-4 * max(1.0, float(want_ent.max())), tag
        grad = TU.logits_bwd(view, y, lse, pz, g.to(cuda_device), q.to(cuda_device), 1.0 / temperature)
        scale = torch.maximum(want_grad.abs().amax(-1, keepdim=True), ((g.abs() + q.abs()) / temperature).double()[:, None])
        assert ((grad.cpu().double() - want_grad).abs() / scale).max() <= (1e-5 if dtype == torch.float32 else 2.0 ** -8), tag


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("compute_entropy,entropy_grad", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fsdp_forward_tail_from_logits(cuda_device, packed, compute_entropy, entropy_grad, dtype):
    """action_log_probs_from_logits against the reference's forward tail (workers/model_wrapper.py:291, 333-393, restated in
    the oracle) on the same logits in fp64: values, shapes, the zero padding, the gradient into the logits -- out of place
    and written over a non-leaf logits tensor."""
    from skyrl_amd.model_wrapper import action_log_probs_from_logits
    dev = cuda_device
    gen = torch.Generator().manual_seed(61)
    B, S, V, A, t = 3, 24, 700, 7, 0.8
    seqs = torch.randint(0, V, (B, S), generator=gen)
    am = torch.ones(B, S, dtype=torch.long)
    am[0, :5] = 0
    am[1, :2] = 0
    nnz = am.flatten().nonzero().flatten() if packed else None
    n_tok = int(am.sum()) if packed else B * S
    logits = (torch.randn(1 if packed else B, n_tok if packed else S, V, generator=gen) * 2).to(dtype)
    x = logits.double().requires_grad_(True)
    want_alp, want_ent = O.hf_wrapper_tail(x, seqs, A, am.double(), t, nnz_indices=nnz)
    G = torch.randn(B, A, generator=gen).double()
    Q = torch.randn(B, S, generator=gen).double() * 0.1
    ((want_alp * G).sum() + ((want_ent * Q).sum() if entropy_grad else 0.0)).backward()
    grads = []
    for inplace in (False, True):
        leaf = logits.to(dev).requires_grad_(True)
        mid = leaf * 1.0
        alp, out = action_log_probs_from_logits(mid, seqs.to(dev), A, am.to(dev), t, return_output=True,
                                                compute_entropy=compute_entropy, entropy_requires_grad=entropy_grad,
                                                nnz_indices=None if nnz is None else nnz.to(dev), inplace_backward=inplace)
        assert alp.shape == (B, A) and alp.dtype == torch.float32
        assert (alp.detach().cpu().double() - want_alp.detach()).abs().max() <= 1e-4
        loss = (alp * G.float().to(dev)).sum()
        if compute_entropy:
            ent = out["entropy"]
            assert ent.shape == (B, S) and ent.dtype == dtype and ent.requires_grad == entropy_grad
            assert (ent.detach().cpu().double() - want_ent.detach()).abs().max() <= (1e-4 if dtype == torch.float32 else 0.05)
            assert bool((ent.detach().cpu()[am == 0] == 0).all())
            if entropy_grad:
                loss = loss + (ent.float() * Q.float().to(dev)).sum()
        else:
            assert out == {}
        loss.backward()
        grads.append(leaf.grad.clone())
        if inplace:
            assert torch.equal(mid.detach(), leaf.grad)       # the logits' storage now holds the gradient
    assert torch.equal(grads[0], grads[1])
    scale = x.grad.abs().amax(-1, keepdim=True).clamp_min(1e-6)
    live = x.grad.abs().amax(-1) > 0
    tol = 1e-4 if dtype == torch.float32 else 2.0 ** -6        # bf16: the entropy reaches the loss rounded to bf16
    assert ((grads[0].cpu().double() - x.grad).abs() / scale)[live].max() <= tol
    assert float(grads[0].cpu()[~live].abs().max() if bool((~live).any()) else 0.0) == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("view", ["drop_last", "drop_first", "narrow_vocab", "both"])
def test_sliced_logits_are_walked_where_they_lie(view, dtype, cuda_device):
    """``logits[:, :-1]`` and its relatives (what a caller that shifts the logits instead of the labels passes): rows equally
    pitched inside a batch entry, the entries not adjacent.  No copy is made -- the kernels run once per batch entry -- so the
    results equal those of a contiguous copy bit for bit, and with ``inplace_backward`` the gradient lands in the caller's own
    storage, the rows outside the view untouched."""
    from skyrl_amd import torch_utils as TU
    gen = torch.Generator(device=cuda_device).manual_seed(5)
    B, S, V = 3, 9, 1000
    base = (torch.randn(B, S, V, device=cuda_device, generator=gen) * 2).to(dtype)
    cut = {"drop_last": (slice(None), slice(0, S - 1), slice(None)), "drop_first": (slice(None), slice(1, S), slice(None)),
           "narrow_vocab": (slice(None), slice(None), slice(0, V - 8)), "both": (slice(None), slice(1, S - 1), slice(8, V))}[view]
    sub = base[cut]
    assert not sub.is_contiguous()
    b, s, v = sub.shape
    labels = torch.randint(0, v, (b, s), device=cuda_device, generator=gen)
    g = torch.randn(b, s, device=cuda_device, generator=gen)
    q = torch.randn(b, s, device=cuda_device, generator=gen) * 0.1
    # reference run on a contiguous copy
    copy = sub.clone().requires_grad_(True)
    lp0, ent0 = TU.logprobs_and_entropy_from_logits(copy, labels, temperature=0.7)
    ((lp0 * g).sum() + (ent0 * q).sum()).backward()
    # the view itself, out of place
    leaf = base.clone().requires_grad_(True)
    lp1, ent1 = TU.logprobs_and_entropy_from_logits(leaf[cut], labels, temperature=0.7)
    ((lp1 * g).sum() + (ent1 * q).sum()).backward()
    assert torch.equal(lp1, lp0) and torch.equal(ent1, ent0)
    assert torch.equal(leaf.grad[cut], copy.grad)
    outside = torch.ones_like(base, dtype=torch.bool)
    outside[cut] = False
    assert bool((leaf.grad[outside] == 0).all())
    # in place: the gradient is written over the view's rows of a non-leaf tensor, the rest of its storage keeps the logits
    leaf2 = base.clone().requires_grad_(True)
    mid = leaf2 * 1.0
    before = mid.detach().clone()
    lp2 = TU.logprobs_from_logits(mid[cut], labels, inplace_backward=True)
    (lp2 * g).sum().backward()
    plain = base.clone().requires_grad_(True)
    (TU.logprobs_from_logits(plain[cut].clone(), labels, inplace_backward=False) * g).sum().backward()
    assert torch.equal(leaf2.grad, plain.grad)
    assert torch.equal(mid.detach()[cut], plain.grad[cut]) and torch.equal(mid.detach()[outside], before[outside])
    # the other wrappers take the same views
    assert torch.equal(TU.chunked_entropy_from_logits(sub), TU.chunked_entropy_from_logits(sub.clone()))
    assert torch.equal(TU.logprobs_from_logits_v2(sub, labels), TU.logprobs_from_logits_v2(sub.clone(), labels))
    assert torch.equal(TU.DistributedLogprob.apply(sub, labels, 0, v, None, True), TU.DistributedLogprob.apply(sub.clone(), labels, 0, v, None, True))

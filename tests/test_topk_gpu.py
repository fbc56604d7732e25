"""GPU parity of the top-k draft loss from hidden states (the HIP stand-in for draft_soft_ce_topk,
skyrl/backends/skyrl_train/mtp/soft_ce.py:243-341) against the oracle's restatement on fp64 logits of the same bf16 operands.

Where fp32 and fp64 may rank two logits differently (the k-th and (k+1)-th of a row closer than 1e-4) the row is left out of
the set comparison and only held to the loss tolerance; bit-exact cases use logits that are exact in bf16.
"""

from __future__ import annotations

import ctypes
import math

import numpy as np
import pytest
import torch

from oracle import lmhead_oracle as O
from skyrl_amd import _lib, mtp_soft_ce as M

pytestmark = pytest.mark.gpu

ERR_NULL, ERR_SHAPE, ERR_WORKSPACE, ERR_ARG = -1, -2, -4, -5   # include/skyrl_lmhead.h
LOSS_ATOL = 2e-3      # per-token loss (fp32 logits of bf16 operands against fp64 ones)
GRAD_REL_L2 = 1e-2    # d student hidden is stored in bf16
GRAD_ROW_REL_L2 = 5e-2


def _operands(T, H, V, seed, scale=3.0):
    gen = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * scale / H**0.5).to(torch.bfloat16)
    return hidden, weight


@pytest.mark.parametrize("T,H,V,k,temperature", [
    (300, 256, 5000, 8, 1.0),        # chunks of 1024, 2048 and a ragged rest; ragged token tile
    (513, 128, 1000, 64, 0.7),       # one chunk narrower than the first chunk width
    (70, 64, 300, 300, 1.0),         # k = V: every column is kept
    (1000, 192, 20011, 32, 1.0),     # all chunk widths up to 8192 and a ragged last tile
    (257, 64, 9000, 1, 1.3),         # k = 1: the arg-max
    (64, 64, 2100, 1024, 1.0),       # the largest k
])
def test_topk_logits_match_fp64(T, H, V, k, temperature, cuda_device):
    hidden, weight = _operands(T, H, V, seed=T + V)
    z = (hidden.double() @ weight.double().t()) / temperature
    want_vals, want_idx = z.topk(min(k + 1, V), dim=-1)
    vals, idx = M.topk_logits_from_hidden(hidden.to(cuda_device), weight.to(cuda_device), k, temperature=temperature)
    vals, idx = vals.cpu(), idx.cpu()
    assert vals.shape == (T, k) and idx.shape == (T, k) and idx.dtype == torch.int64 and vals.dtype == torch.float32
    # every reported value is the logit of its column, the lists are sorted and hold no column twice
    assert (vals.double() - z.gather(-1, idx)).abs().max() <= 1e-4 * max(1.0, float(z.abs().max()))
    assert bool((vals[:, 1:] <= vals[:, :-1]).all())
    assert all(len(set(r)) == k for r in idx.tolist())
    # the same set of columns wherever fp64 separates the k-th from the (k+1)-th logit
    if k < V:
        clear = (want_vals[:, k - 1] - want_vals[:, k]) > 1e-4
        assert int(clear.sum()) >= 0.9 * T
    else:
        clear = torch.ones(T, dtype=torch.bool)
    got_sets = idx.sort(-1).values
    want_sets = want_idx[:, :k].sort(-1).values
    assert torch.equal(got_sets[clear], want_sets[clear])


def test_topk_logits_random_shapes(cuda_device):
    """Twenty random (T, H, V, k) cases: the column sets of fp64 wherever fp64 separates the k-th from the (k+1)-th logit."""
    rng = torch.Generator().manual_seed(77)
    for case in range(20):
        T = int(torch.randint(1, 600, (1,), generator=rng))
        H = 64 * int(torch.randint(1, 5, (1,), generator=rng))
        V = int(torch.randint(2, 12000, (1,), generator=rng))
        k = int(torch.randint(1, min(V, 200), (1,), generator=rng))
        hidden, weight = _operands(T, H, V, seed=500 + case)
        z = hidden.double() @ weight.double().t()
        want = z.topk(k + 1, dim=-1)
        clear = (want.values[:, k - 1] - want.values[:, k]) > 1e-4
        vals, idx = M.topk_logits_from_hidden(hidden.to(cuda_device), weight.to(cuda_device), k)
        tag = (case, T, H, V, k)
        assert torch.equal(idx.cpu().sort(-1).values[clear], want.indices[:, :k].sort(-1).values[clear]), tag
        assert (vals.cpu().double() - z.gather(-1, idx.cpu())).abs().max() <= 1e-4 * max(1.0, float(z.abs().max())), tag
        assert bool((vals[:, 1:] <= vals[:, :-1]).all()), tag


def test_topk_logits_ties_and_the_worst_case_order_bit_exact(cuda_device):
    """Logits that are exact in bf16 and ascend with the column -- every logit is a candidate in every chunk, the worst case of
    the filter -- with many equal values: equal values come out lower column first, results bit-exact."""
    T, H, V, k = 130, 64, 19000, 40
    hidden = torch.zeros(T, H, dtype=torch.bfloat16)
    hidden[:, 0] = 1.0
    hidden[:, 1] = torch.arange(T).to(torch.bfloat16)          # a per-token offset through a second column
    weight = torch.zeros(V, H, dtype=torch.bfloat16)
    weight[:, 0] = (torch.arange(V, dtype=torch.float32) / 64.0).to(torch.bfloat16)   # ascending, 8 mantissa bits: runs of ties
    weight[:, 1] = 1.0
    z = hidden.float() @ weight.float().t()                     # exact: two products of bf16 values, sums below 2^24 ulps
    order = np.lexsort((np.arange(V)[None, :].repeat(T, 0), -z.numpy()), axis=-1)[:, :k]
    vals, idx = M.topk_logits_from_hidden(hidden.to(cuda_device), weight.to(cuda_device), k)
    assert np.array_equal(idx.cpu().numpy(), order)
    assert torch.equal(vals.cpu(), z.gather(-1, torch.from_numpy(order)))
    # descending logits: after the first chunk nothing passes the filter
    weight[:, 0] = -weight[:, 0]
    z = hidden.float() @ weight.float().t()
    order = np.lexsort((np.arange(V)[None, :].repeat(T, 0), -z.numpy()), axis=-1)[:, :k]
    vals, idx = M.topk_logits_from_hidden(hidden.to(cuda_device), weight.to(cuda_device), k)
    assert np.array_equal(idx.cpu().numpy(), order) and torch.equal(vals.cpu(), z.gather(-1, torch.from_numpy(order)))


def test_topk_logits_in_token_blocks_and_with_strided_rows(cuda_device):
    """More tokens than one block of 16384 (the per-token scratch is reused by the second block), hidden rows and weight rows
    with a pitch larger than H: bit-identical to the calls on contiguous halves."""
    T, H, V, k = 16384 + 300, 64, 1500, 8
    hidden, weight = _operands(T, H, V, seed=21)
    wide_h = torch.zeros(T, H + 24, dtype=torch.bfloat16, device=cuda_device)
    wide_h[:, :H] = hidden.to(cuda_device)
    wide_w = torch.zeros(V, H + 8, dtype=torch.bfloat16, device=cuda_device)
    wide_w[:, :H] = weight.to(cuda_device)
    vals, idx = M.topk_logits(wide_h[:, :H], wide_w[:, :H], k, 1.0)
    h, w = hidden.to(cuda_device), weight.to(cuda_device)
    a_vals, a_idx = M.topk_logits(h[:16384], w, k, 1.0)
    b_vals, b_idx = M.topk_logits(h[16384:].contiguous(), w, k, 1.0)
    assert torch.equal(vals, torch.cat([a_vals, b_vals])) and torch.equal(idx, torch.cat([a_idx, b_idx]))
    z = hidden[-300:].double() @ weight.double().t()
    want = z.topk(k + 1, dim=-1)
    clear = (want.values[:, k - 1] - want.values[:, k]) > 1e-4
    assert torch.equal(idx[-300:].cpu().long().sort(-1).values[clear], want.indices[:, :k].sort(-1).values[clear])


def test_topk_logits_with_infinite_logits_in_a_ragged_tile(cuda_device):
    """The last token of a ragged token tile has logits of +-inf: the tile's padding rows repeat that token and must not
    reach any list; the token's own list holds the first k columns of +inf."""
    T, H, V, k = 300, 64, 1300, 4
    hidden, weight = _operands(T, H, V, seed=5)
    hidden[T - 1] = 0
    hidden[T - 1, 0] = 3.0e38
    weight[:, 0] = torch.where(torch.arange(V) % 3 == 0, 2.0, -2.0).bfloat16()
    vals, idx = M.topk_logits_from_hidden(hidden.to(cuda_device), weight.to(cuda_device), k)
    assert torch.isinf(vals[T - 1]).all() and bool((vals[T - 1] > 0).all()) and idx[T - 1].tolist() == [0, 3, 6, 9]
    z = hidden[: T - 1].double() @ weight.double().t()
    want = z.topk(k + 1, dim=-1)
    clear = (want.values[:, k - 1] - want.values[:, k]) > 1e-4
    assert torch.equal(idx[: T - 1].cpu().sort(-1).values[clear], want.indices[:, :k].sort(-1).values[clear])
    again = M.topk_logits_from_hidden(hidden.to(cuda_device), weight.to(cuda_device), k)
    assert torch.equal(again[1], idx)


def test_topk_logits_are_reproducible(cuda_device):
    hidden, weight = _operands(700, 128, 12000, seed=3)
    h, w = hidden.to(cuda_device), weight.to(cuda_device)
    a = M.topk_logits_from_hidden(h, w, 50)
    for _ in range(3):
        b = M.topk_logits_from_hidden(h, w, 50)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def _soft_ce_case(B, S, H, V, k, shift, seed):
    gen = torch.Generator().manual_seed(seed)
    student = torch.randn(B, S, H, generator=gen).to(torch.bfloat16)
    teacher = (student.float() + 0.7 * torch.randn(B, S, H, generator=gen)).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * 3.0 / H**0.5).to(torch.bfloat16)
    w64 = weight.double()
    x = student.double().requires_grad_(True)
    z_t = teacher.double() @ w64.t()
    per_token, _, _, cols = O.soft_ce_topk_per_token(x @ w64.t(), z_t, k, roll_shift=shift)
    top = z_t.topk(min(k + 1, V), dim=-1).values
    clear = (top[..., k - 1] - top[..., k]) > 1e-4 if k < V else torch.ones(B, S, dtype=torch.bool)
    clear = torch.roll(clear, shifts=-shift, dims=1) if shift else clear
    return student, teacher, weight, x, per_token, cols, clear


@pytest.mark.parametrize("B,S,H,V,k,shift", [
    (2, 150, 256, 5000, 8, 1),
    (1, 300, 128, 3000, 64, 0),
    (3, 85, 64, 20011, 20, 2),
    (4, 9, 64, 257, 257, 3),          # k = V: the full-vocabulary soft cross-entropy
    (1, 1, 64, 1500, 5, 4),           # one position: the roll wraps onto itself
])
def test_soft_ce_topk_from_hidden_matches_oracle(B, S, H, V, k, shift, cuda_device):
    student, teacher, weight, x, per_token, cols, clear = _soft_ce_case(B, S, H, V, k, shift, seed=B * 100 + S)
    gen = torch.Generator().manual_seed(1)
    g = torch.randn(B, S, generator=gen).double() * clear        # rows fp32 may rank differently take no part in the gradient
    (per_token * g).sum().backward()
    hs = student.to(cuda_device).requires_grad_(True)
    got = M.soft_ce_topk_from_hidden(hs, teacher.to(cuda_device), weight.to(cuda_device), k, shift=shift)
    assert got.shape == (B, S) and got.dtype == torch.float32
    (got * g.float().to(cuda_device)).sum().backward()
    err = (got.detach().cpu().double() - per_token.detach()).abs()
    assert float(err[clear].max()) <= LOSS_ATOL, float(err[clear].max())
    assert float(err.max()) <= 0.05            # a swapped near-tie at the k-th place moves the loss by next to nothing
    assert int(clear.sum()) >= 0.9 * B * S
    want, have = x.grad.reshape(-1, H), hs.grad.double().cpu().reshape(-1, H)
    assert float((have - want).norm() / want.norm()) < GRAD_REL_L2
    norms = want.norm(dim=1)
    floor = 1e-3 * float(norms.max())
    assert float(((have - want).norm(dim=1) / norms.clamp_min(floor)).max()) < GRAD_ROW_REL_L2
    assert bool((hs.grad.cpu().reshape(-1, H)[g.reshape(-1) == 0] == 0).all())
    if k == V:   # the limit in which it is the full soft cross-entropy of the tile kernels
        full = M.soft_ce_from_hidden(student.to(cuda_device), teacher.to(cuda_device), weight.to(cuda_device), shift=shift)
        assert float((full - got.detach()).abs().max()) <= LOSS_ATOL


def test_draft_soft_ce_topk_from_hidden_reductions_and_checks(cuda_device):
    B, S, H, V, k, shift = 2, 40, 64, 2000, 16, 1
    student, teacher, weight, x, per_token, cols, clear = _soft_ce_case(B, S, H, V, k, shift, seed=77)
    mask = torch.ones(B, S)
    mask[0, 25:] = 0
    mask = O.shift_mask_for_mtp(mask, 0) * clear
    args = (student.to(cuda_device), teacher.to(cuda_device), weight.to(cuda_device), mask.to(cuda_device), k)
    want = O.draft_soft_ce_topk_from_hidden(student.double(), teacher.double(), weight.double(), mask.double(), k, roll_shift=shift)
    assert M.draft_soft_ce_topk_from_hidden(*args, roll_shift=shift).item() == pytest.approx(want.item(), abs=LOSS_ATOL)
    norm = torch.tensor(123.0)
    want = O.draft_soft_ce_topk_from_hidden(student.double(), teacher.double(), weight.double(), mask.double(), k, norm.double(),
                                            roll_shift=shift)
    got = M.draft_soft_ce_topk_from_hidden(*args, norm.to(cuda_device), roll_shift=shift)
    assert got.item() == pytest.approx(want.item(), abs=LOSS_ATOL)
    # k beyond the vocabulary is the whole vocabulary (k_eff = min(k, V), soft_ce.py:267)
    small_w = weight[:200].to(cuda_device)
    a = M.soft_ce_topk_from_hidden(args[0], args[1], small_w, 5000, shift=shift)
    b = M.soft_ce_topk_from_hidden(args[0], args[1], small_w, 200, shift=shift)
    assert torch.equal(a, b)
    with pytest.raises(AssertionError):
        M.soft_ce_topk_from_hidden(args[0], args[1].clone().requires_grad_(True), args[2], k)
    with pytest.raises(ValueError):
        M.soft_ce_topk_from_hidden(args[0], args[1], args[2], 0)
    with pytest.raises(ValueError):
        M.topk_logits(args[0].reshape(-1, H), args[2], 1025, 1.0)
    empty = M.soft_ce_topk_from_hidden(args[0][:, :0], args[1][:, :0], args[2], k)
    assert empty.shape == (B, 0)


def test_topk_c_abi_argument_errors(cuda_device):
    lib = _lib.load()
    T, H, V, k = 64, 64, 512, 4
    hidden, weight = _operands(T, H, V, seed=0)
    h, w = hidden.to(cuda_device), weight.to(cuda_device)
    vals = torch.empty(T, k, device=cuda_device)
    cols = torch.empty(T, k, dtype=torch.int32, device=cuda_device)
    need = lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, k)
    assert need > 0 and lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, V + 1) == 0
    assert lib.skyrl_lmhead_topk_workspace_bytes(T, H, 5000, 1025) == 0 and lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, 0) == 0
    ws = torch.empty(need, dtype=torch.uint8, device=cuda_device)

    def call(hp=None, kk=k, ws_bytes=need, vp=None, HH=H):
        return lib.skyrl_lmhead_topk_logits(h.data_ptr() if hp is None else hp, H, w.data_ptr(), H, T, HH, V, kk, 1.0,
                                            vals.data_ptr() if vp is None else vp, cols.data_ptr(), ws.data_ptr(), ws_bytes, None)

    assert call() == 0
    assert call(hp=ctypes.c_void_p(0)) == ERR_NULL and call(vp=ctypes.c_void_p(0)) == ERR_NULL
    assert call(kk=0) == ERR_ARG and call(kk=V + 1) == ERR_ARG
    assert call(ws_bytes=need - 1) == ERR_WORKSPACE
    assert call(HH=40) == ERR_SHAPE
    loss = torch.empty(T, device=cuda_device)
    coef = torch.empty(T, k, device=cuda_device)
    used = torch.empty(T, k, dtype=torch.int32, device=cuda_device)
    fwd = lambda seq, shift: lib.skyrl_softce_topk_fwd(h.data_ptr(), H, w.data_ptr(), H, vals.data_ptr(), cols.data_ptr(), T, seq,  # noqa: E731
                                                       shift, H, V, k, 1.0, loss.data_ptr(), coef.data_ptr(), used.data_ptr(), None)
    assert fwd(16, 1) == 0 and fwd(7, 1) == ERR_SHAPE and fwd(16, -1) == ERR_SHAPE
    dh = torch.empty(T, H, dtype=torch.bfloat16, device=cuda_device)
    bwd = lambda ld: lib.skyrl_softce_topk_bwd(w.data_ptr(), H, coef.data_ptr(), used.data_ptr(), loss.data_ptr(), T, H, V, k, 1.0,  # noqa: E731
                                               dh.data_ptr(), ld, None)
    assert bwd(H) == 0 and bwd(H - 8) == ERR_SHAPE
    torch.cuda.synchronize()


def test_topk_ops_opcheck(cuda_device):
    hidden, weight = _operands(96, 64, 700, seed=9)
    h, w = hidden.to(cuda_device), weight.to(cuda_device)
    torch.library.opcheck(M.topk_logits, (h, w, 6, 1.0), test_utils=("test_schema", "test_faketensor"))
    vals, cols = M.topk_logits(h, w, 6, 1.0)
    torch.library.opcheck(M.softce_topk_fwd, (h, w, vals, cols, 32, 1, 1.0), test_utils=("test_schema", "test_faketensor"))
    loss, coef, used = M.softce_topk_fwd(h, w, vals, cols, 32, 1, 1.0)
    torch.library.opcheck(M.softce_topk_bwd, (w, coef, used, loss, 1.0), test_utils=("test_schema", "test_faketensor"))


def test_topk_full_size_properties(cuda_device):
    """The 7B shape (T = 16384, H = 3584, V = 152064), k = 32: sampled rows against logits computed row by row, the workspace
    far below one T x V buffer, loss and gradient finite and bounded."""
    T, H, V, k = 16384, 3584, 152064, 32
    gen = torch.Generator(device=cuda_device).manual_seed(0)
    student = torch.randn(T, H, device=cuda_device, generator=gen).to(torch.bfloat16)
    teacher = (student.float() + 0.5 * torch.randn(T, H, device=cuda_device, generator=gen)).to(torch.bfloat16)
    weight = (torch.randn(V, H, device=cuda_device, generator=gen) * (3.0 / H**0.5)).to(torch.bfloat16)
    lib = _lib.load()
    assert lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, k) < 2 * T * V / 4
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    vals, idx = M.topk_logits_from_hidden(teacher, weight, k)
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated() - base < lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, k) + 16 * T * k + (64 << 20)
    rows = torch.randperm(T, generator=torch.Generator().manual_seed(1))[:24].to(cuda_device)
    z = teacher[rows].double() @ weight.double().t()
    want_vals, want_idx = z.topk(k + 1, dim=-1)
    clear = (want_vals[:, k - 1] - want_vals[:, k]) > 1e-4
    assert torch.equal(idx[rows].sort(-1).values[clear], want_idx[:, :k].sort(-1).values[clear]) and int(clear.sum()) >= 20
    assert float((vals[rows].double() - z.gather(-1, idx[rows])).abs().max()) <= 1e-3
    hs = student.requires_grad_(True)
    loss = M.soft_ce_topk_from_hidden(hs.reshape(4, T // 4, H), teacher.reshape(4, T // 4, H), weight, k, shift=1)
    loss.sum().backward()
    assert bool(torch.isfinite(loss).all()) and float(loss.detach().min()) >= 0.0 and float(loss.detach().max()) <= 30.0
    assert bool(torch.isfinite(hs.grad).all())
    # sampled rows of the loss against the oracle on fp64 logits
    for t in rows.tolist()[:6]:
        b, s = divmod(t, T // 4)
        tt = b * (T // 4) + (s + 1) % (T // 4)
        zt = teacher[tt].double() @ weight.double().t()
        zs = student[t].detach().double() @ weight.double().t()
        want = O.soft_ce_topk_per_token(zs[None, None].cpu(), zt[None, None].cpu(), k)[0]
        assert float(loss.detach().reshape(-1)[t]) == pytest.approx(float(want), abs=5e-3)


def test_topk_draft_loss_replays_from_a_hip_graph(cuda_device):
    """The top-k entry points launch kernels and nothing else (the per-token counters are cleared by a kernel, not by a
    memset), so a forward + backward of the draft loss can be captured; three replays on new inputs, with eager work in
    between, each reproduce the eager result bit for bit."""
    T, S, H, V, k = 320, 80, 128, 3000, 16
    gen = torch.Generator().manual_seed(5)
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).bfloat16().to(cuda_device)
    student = torch.zeros(T, H, dtype=torch.bfloat16, device=cuda_device)
    teacher = torch.zeros(T, H, dtype=torch.bfloat16, device=cuda_device)
    g = torch.zeros(T, device=cuda_device)

    def step():
        values, columns = M.topk_logits(teacher, weight, k, 1.0)
        loss, coef, used = M.softce_topk_fwd(student, weight, values, columns, S, 1, 1.0)
        return values, columns, loss, M.softce_topk_bwd(weight, coef, used, g, 1.0)

    def refill(seed):
        gen_ = torch.Generator().manual_seed(seed)
        student.copy_(torch.randn(T, H, generator=gen_).bfloat16())
        teacher.copy_(torch.randn(T, H, generator=gen_).bfloat16())
        g.copy_(torch.randn(T, generator=gen_))

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


def test_topk_of_a_nan_row_is_nan(cuda_device):
    """A token whose hidden row holds a NaN has NaN logits everywhere: torch.topk ranks NaN first, and the reference's draft loss
    on it is NaN (mtp/soft_ce.py:258-305).  No logit of such a row passes the kernel's comparisons; the ranks it cannot fill
    come back as NaN with column 0, never as uninitialised memory, and the rows around it are untouched."""
    T, H, V, k = 130, 64, 3000, 16
    hidden, weight = _operands(T, H, V, seed=3)
    clean_vals, clean_idx = M.topk_logits_from_hidden(hidden.to(cuda_device), weight.to(cuda_device), k)
    hidden[77, 5] = float("nan")
    vals, idx = M.topk_logits_from_hidden(hidden.to(cuda_device), weight.to(cuda_device), k)
    assert bool(torch.isnan(vals[77]).all()) and bool((idx[77] == 0).all())
    others = torch.arange(T) != 77
    assert torch.equal(vals[others.to(cuda_device)], clean_vals[others.to(cuda_device)])
    assert torch.equal(idx[others.to(cuda_device)], clean_idx[others.to(cuda_device)])

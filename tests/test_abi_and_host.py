"""CPU-only checks of the boundary: the C-ABI library loads, exports every symbol the header declares, rejects bad arguments
before touching a device, and the Python host layer mirrors the reference's interface and error behaviour.  No kernel is
launched here."""

import inspect
import os
import re

import pytest
import torch

from skyrl_amd import _lib, model_utils, ops
from skyrl_amd.fused_linear_logprob_hip import FusedLinearLogprobHip, LinearCrossEntropy, linear_cross_entropy

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "skyrl_lmhead.h")
BENCH_HEADER = os.path.join(ROOT, "include", "skyrl_lmhead_bench.h")  # measurement aids, no reference counterpart


def _read(path):
    with open(path) as f:
        return f.read()


def _declared_functions(*headers):
    text = "".join(_read(h) for h in (headers or (HEADER, BENCH_HEADER)))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(skyrl_(?:lmhead|ppo|packed|approx|masked|actor|softce|logits|off|logprob)_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_functions()
    assert names == sorted(_lib.SIGNATURES), "ctypes table and header disagree"
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.skyrl_lmhead_version() == _lib.ABI_VERSION


def test_library_is_in_tree_and_has_no_torch_dependency():
    assert _lib.lib_path().startswith(ROOT)
    import subprocess
    out = subprocess.run(["ldd", _lib.lib_path()], capture_output=True, text=True).stdout
    assert "libamdhip64" in out and "torch" not in out and "libc10" not in out


def test_strerror_table():
    for code in (0, -1, -2, -3, -4, -5, -6):
        assert _lib.strerror(code) and "unknown" not in _lib.strerror(code)
    assert "unknown" in _lib.strerror(-99)


def test_workspace_queries():
    lib = _lib.load()
    T, H, V = 16384, 3584, 152064
    fwd = lib.skyrl_lmhead_fwd_workspace_bytes(T, H, V)
    assert 3 * 4 * T * 2 * 594 <= fwd <= 3 * 4 * T * 2 * 594 + 4096
    bwd = lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, 4096)
    # hidden^T + fp32 dHidden + one dz panel; nothing of size T*V, and no copy of the weight (V is a multiple of 64)
    expect = 2 * H * T + 4 * T * H + 2 * T * 4096
    assert expect <= bwd <= expect + (8 << 20)  # + 128 B of row padding per scratch row
    # a vocabulary that is not a multiple of the k-tile needs the transposed, zero-padded weight as well
    odd = lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V - 8, 4096)
    assert expect + 2 * H * (V - 8) <= odd <= expect + 2 * H * V + (8 << 20)
    assert bwd < 2 * T * V
    assert lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, 100) == 0  # not a multiple of 256
    assert lib.skyrl_lmhead_fwd_workspace_bytes(0, H, V) == 0
    # top-k: a candidate list of one chunk (8192 slots of 8 bytes) and k running keys per token of a 16384-token block,
    # whatever T and V are beyond that
    k = 32
    topk = lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, k)
    assert 8 * T * (8192 + k) <= topk <= 8 * T * (8192 + k) + 12 * T + 4096
    assert lib.skyrl_lmhead_topk_workspace_bytes(16 * T, H, 2 * V, k) == topk
    assert lib.skyrl_lmhead_topk_workspace_bytes(T, H, 1000, k) < topk // 7      # a vocabulary below one chunk
    for bad_k in (0, 1025, -1):
        assert lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, bad_k) == 0
    assert lib.skyrl_lmhead_topk_workspace_bytes(T, H, 20, 21) == 0              # k beyond the vocabulary


def _call_fwd(lib, **kw):
    a = dict(hidden=0x1000, ldh=128, weight=0x2000, ldw=128, labels=0x3000, T=4, H=128, V=16, rt=1.0, lp=0x4000, ent=None,
             lse=None, pz=None, ws=0x10000, wsb=1 << 20, stream=None)
    a.update(kw)
    return lib.skyrl_lmhead_fwd(a["hidden"], a["ldh"], a["weight"], a["ldw"], a["labels"], a["T"], a["H"], a["V"], a["rt"],
                                a["lp"], a["ent"], a["lse"], a["pz"], a["ws"], a["wsb"], a["stream"])


def test_forward_argument_errors_are_reported_before_any_launch():
    lib = _lib.load()
    assert _call_fwd(lib, hidden=None) == -1
    assert _call_fwd(lib, lp=None) == -1
    assert _call_fwd(lib, H=100, ldh=104, ldw=104) == -2  # H not a multiple of 64
    assert _call_fwd(lib, T=0) == -2
    assert _call_fwd(lib, ldh=64) == -2  # leading dimension < H
    # matrices of any size are accepted (a tile is addressed from its own first row); only the row pitch is limited
    assert _call_fwd(lib, ldw=(1 << 22) + 8) == -2 and _call_fwd(lib, ldh=(1 << 22) + 8) == -2
    assert _call_fwd(lib, hidden=0x1008) == -3
    assert _call_fwd(lib, ldw=132) == -3
    assert _call_fwd(lib, ws=None) == -4
    assert _call_fwd(lib, wsb=16) == -4
    assert _call_fwd(lib, rt=0.0) == -5
    assert _call_fwd(lib, rt=float("inf")) == -5
    assert _call_fwd(lib, rt=float("nan")) == -5


def test_static_scratch_forward_argument_errors():
    """The entry point without a workspace checks its operands like the ordinary forward, and its size limit, on the host."""
    lib = _lib.load()

    def call(hidden=0x1000, weight=0x2000, labels=0x3000, lp=0x4000, T=256, H=128, V=1024, ldh=None, ldw=None, rt=1.0):
        return lib.skyrl_lmhead_fwd_static_scratch(hidden, ldh or H, weight, ldw or H, labels, T, H, V, rt, lp, None, None, None,
                                                   None)

    assert lib.skyrl_lmhead_static_scratch_bytes() == 33554432
    assert call(hidden=None) == -1 and call(lp=None) == -1
    assert call(H=100, ldh=104, ldw=104) == -2 and call(T=0) == -2
    assert call(hidden=0x1008) == -3
    assert call(rt=0.0) == -5
    assert call(V=1398017, H=64) == -6  # a 256-token tile of partials no longer fits the 32 MiB array
    assert call(V=1398017, H=64, ldw=(1 << 22) + 8) == -2  # the row-pitch limit is reported first


def test_split_operand_argument_errors():
    """fp32 operands as stacked bf16 terms: layouts, shapes and alignment are checked on the host."""
    lib = _lib.load()
    p, q = 0x10000, 0x20000
    assert lib.skyrl_lmhead_split_operand(None, 1, 128, 4, 128, 0, q, 256, None) == -1
    assert lib.skyrl_lmhead_split_operand(p, 1, 128, 4, 128, 7, q, 256, None) == -5      # no such layout
    assert lib.skyrl_lmhead_split_operand(p, 1, 128, 4, 128, 0, q, 128, None) == -2      # destination rows too short for 2 terms
    assert lib.skyrl_lmhead_split_operand(p, 1, 128, 4, 128, 2, q, 256, None) == -2      # ... for 3 terms
    assert lib.skyrl_lmhead_split_operand(p, 1, 64, 4, 128, 0, q, 256, None) == -2       # source rows shorter than H
    assert lib.skyrl_lmhead_split_operand(p, 1, 128, 0, 128, 0, q, 256, None) == -2
    assert lib.skyrl_lmhead_split_operand(p + 4, 1, 128, 4, 128, 0, q, 256, None) == -3
    assert lib.skyrl_lmhead_split_operand(p, 1, 130, 4, 128, 0, q, 256, None) == -3
    T, H, V = 300, 128, 1000
    base = lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, 0)
    assert lib.skyrl_lmhead_bwd_split_workspace_bytes(T, H, 1, V, 0, 0) == base           # one term: the ordinary backward
    # more terms only lengthen the logits GEMM; the scratch grows by one fp32 per (padded) token, the label residuals
    assert lib.skyrl_lmhead_bwd_split_workspace_bytes(T, H, 3, V, 0, 0) == base + 512 * 4
    assert lib.skyrl_lmhead_bwd_split_workspace_bytes(T, H, 1, V, 0, 1) == lib.skyrl_lmhead_bwd_active_rows_workspace_bytes(T, H, V, 0)
    assert lib.skyrl_lmhead_bwd_split_workspace_bytes(T, H, 4, V, 0, 0) == 0
    args = (p, 3 * H, p, 3 * H, p, p, None, p, None, T, H)
    tail = (V, 1.0, p, p, 0, 0, 0, p, 1 << 40, None)
    assert lib.skyrl_lmhead_bwd_split(*args, 0, *tail) == -5 and lib.skyrl_lmhead_bwd_split(*args, 4, *tail) == -5
    assert lib.skyrl_lmhead_bwd_split(p, 2 * H, p, 3 * H, p, p, None, p, None, T, H, 3, *tail) == -2   # hidden rows hold 2 of 3 terms


def test_backward_argument_errors():
    lib = _lib.load()

    def call(**kw):
        a = dict(hidden=0x1000, ldh=128, weight=0x2000, ldw=128, labels=0x3000, lse=0x4000, pz=None, g=0x5000, q=None, T=4,
                 H=128, V=16, rt=1.0, dh=0x6000, dw=0x7000, acc=0, vc=0, ws=0x10000, wsb=1 << 30, stream=None)
        a.update(kw)
        return lib.skyrl_lmhead_bwd(a["hidden"], a["ldh"], a["weight"], a["ldw"], a["labels"], a["lse"], a["pz"], a["g"],
                                    a["q"], a["T"], a["H"], a["V"], a["rt"], a["dh"], a["dw"], a["acc"], a["vc"], a["ws"],
                                    a["wsb"], a["stream"])

    assert call(lse=None) == -1
    assert call(q=0x8000, pz=None) == -1  # an entropy gradient needs row_pz
    assert call(dh=0x6004) == -3
    assert call(vc=100) == -5
    assert call(wsb=1024) == -4
    assert call(H=96, ldh=96, ldw=96) == -2


def test_mfma_probe_argument_errors():
    lib = _lib.load()
    assert lib.skyrl_lmhead_mfma_probe(None, 256, 10, 0x2000, None) == -1
    assert lib.skyrl_lmhead_mfma_probe(0x1000, 256, 10, None, None) == -1
    assert lib.skyrl_lmhead_mfma_probe(0x1000, 0, 10, 0x2000, None) == -5
    assert lib.skyrl_lmhead_mfma_probe(0x1000, 256, 0, 0x2000, None) == -5
    assert lib.skyrl_lmhead_mfma_probe(0x1008, 256, 10, 0x2000, None) == -3


def test_ppo_policy_loss_argument_errors():
    lib = _lib.load()
    call = lambda **kw: lib.skyrl_ppo_policy_loss(*[{**dict(lp=0x1000, old=0x2000, adv=0x3000, mask=None, w=None, T=8, lo=0.2,  # noqa: E731
                                                        hi=0.2, c=3.0, dual=0, out=0x4000, g=None, part=None, stream=None), **kw}[k]
                                                     for k in ("lp", "old", "adv", "mask", "w", "T", "lo", "hi", "c", "dual", "out", "g",
                                                               "part", "stream")])
    assert call(lp=None) == -1
    assert call(out=None) == -1
    assert call(T=0) == -2
    assert call(lo=float("nan")) == -5
    assert call(dual=1, c=float("inf")) == -5
    assert call(T=8193) == -4 and call(T=8193, part=None, lp=None) == -1   # several workgroups need the partial-sum scratch


def test_ppo_policy_loss_mirror_contract():
    from types import SimpleNamespace

    from skyrl_amd.policy_loss import ppo_policy_loss

    x = torch.zeros(2, 4)
    cfg = SimpleNamespace(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.2, clip_ratio_c=3.0)
    with pytest.raises(AssertionError):
        ppo_policy_loss(x, x, x, SimpleNamespace(policy_loss_type="gspo", eps_clip_low=0.2, eps_clip_high=0.2))
    # rollout log-probabilities are used for off-policy correction only: computed on the device when the config switches one
    # on (a cap that is missing is named), ignored (as in the reference) when it does not
    cfg.off_policy_correction = SimpleNamespace(tis_ratio_type="token")
    with pytest.raises(ValueError, match="token_tis_ratio_clip_high"):
        ppo_policy_loss(x, x, x, cfg, rollout_logprobs=x)
    cfg.off_policy_correction = SimpleNamespace(tis_ratio_type="token", token_tis_ratio_clip_high=2.0)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ppo_policy_loss(x, x, x, cfg, rollout_logprobs=x)
    cfg.off_policy_correction = {"tis_ratio_type": None, "sequence_mask_metric": None}
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ppo_policy_loss(x, x, x, cfg, rollout_logprobs=x)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ppo_policy_loss(x, x, x, cfg)


def test_status_to_exception_mapping():
    with pytest.raises(ValueError, match="NULL"):
        _lib.check(-1, "x")
    with pytest.raises(_lib.LmHeadLibraryError):
        _lib.check(1, "x")
    _lib.check(0, "x")


def test_ops_refuse_cpu_tensors_and_wrong_dtypes():
    h = torch.zeros(4, 128, dtype=torch.bfloat16)
    w = torch.zeros(16, 128, dtype=torch.bfloat16)
    y = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ops.lmhead_fwd(h, w, y, 1.0, True)
    with pytest.raises(TypeError, match="bf16"):
        ops.lmhead_fwd(h.float(), w, y, 1.0, True)        # fp32 hidden with a bf16 weight would be a silent down-cast
    with pytest.raises(TypeError, match="bf16"):
        ops.lmhead_fwd(h.half(), w.half(), y, 1.0, True)
    with pytest.raises(TypeError, match="int64"):
        ops.lmhead_fwd(h, w, y.int(), 1.0, True)
    with pytest.raises(ValueError):
        ops.lmhead_fwd(h, w[:, :64], y, 1.0, True)


def test_fake_kernels_give_shapes_without_a_device():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        h = torch.empty(12, 128, dtype=torch.bfloat16)
        w = torch.empty(40, 128, dtype=torch.bfloat16)
        y = torch.empty(12, dtype=torch.int64)
        lp, ent, lse, pz = torch.ops.skyrl_amd.lmhead_fwd(h, w, y, 1.0, True)
        assert lp.shape == (12,) and ent.shape == (12,) and lp.dtype == torch.float32
        lp, ent, lse, pz = torch.ops.skyrl_amd.lmhead_fwd(h, w, y, 1.0, False)
        assert ent.numel() == 0 and pz.numel() == 0
        dh, dw = torch.ops.skyrl_amd.lmhead_bwd(h, w, y, lse, None, lp, None, 1.0, 0)
        assert dh.shape == (12, 128) and dh.dtype == torch.bfloat16 and dw.shape == (40, 128) and dw.dtype == torch.float32


def test_signatures_mirror_the_reference():
    # FusedLinearChunkedDistributedLogprob.forward / FusedLinearLogprobTriton.forward (model_utils.py:302-313)
    assert list(inspect.signature(FusedLinearLogprobHip.forward).parameters) == [
        "ctx", "hidden", "weight", "target", "vocab_start_index", "vocab_end_index", "chunk_size", "tp_group", "inference_only"]
    # LinearCrossEntropy.forward (fused_linear_logprob_triton.py:1763-1775)
    lce = inspect.signature(LinearCrossEntropy.forward).parameters
    assert list(lce)[:7] == ["ctx", "hidden", "weight", "labels", "temperature", "reduction", "dist_process_group"]
    assert list(lce)[7:] == ["want_entropy"] and lce["want_entropy"].default is True  # one trailing optional extension
    # model_utils.py:713-725
    dense = inspect.signature(model_utils.from_parallel_hidden_to_logprobs).parameters
    assert list(dense)[:11] == [
        "hidden", "lm_head_weight", "target", "vocab_start_index", "vocab_end_index", "tp_group", "inference_only",
        "cp_group", "chunk_size", "temperature", "fused_backend"]
    assert all(v.kind is inspect.Parameter.KEYWORD_ONLY and v.default is None for v in list(dense.values())[11:])
    # model_utils.py:773-789
    packed = inspect.signature(model_utils.from_parallel_hidden_to_logprobs_packed_sequences).parameters
    assert list(packed)[:15] == [
        "hidden", "lm_head_weight", "target", "cu_seqlens_padded", "unpacked_seqlen", "vocab_start_index", "vocab_end_index",
        "group", "inference_only", "cp_group", "chunk_size", "attention_mask", "sub_seq_lengths", "temperature",
        "fused_backend"]
    # anything beyond the reference's list is keyword-only and optional, so every reference call site binds unchanged
    assert all(v.kind is inspect.Parameter.KEYWORD_ONLY and v.default is None for v in list(packed.values())[15:])
    # model_utils.py:1090-1096
    assert list(inspect.signature(model_utils._fused_vocab_parallel_entropy_from_hidden).parameters) == [
        "hidden", "lm_head_weight", "tp_group", "chunk_size", "temperature"]
    # model_utils.py:431-441 (+ one trailing optional argument)
    assert list(inspect.signature(model_utils._fused_lm_head_logprob_apply).parameters)[:9] == [
        "backend", "hidden", "weight", "target", "vocab_start_index", "vocab_end_index", "chunk_size", "tp_group",
        "inference_only"]


def test_linear_cross_entropy_argument_asserts():
    h = torch.zeros(4, 128, dtype=torch.bfloat16)
    w = torch.zeros(16, 128, dtype=torch.bfloat16)
    y = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(AssertionError, match="temperature must be a float"):
        linear_cross_entropy(h, w, y, 1, "none", None)
    with pytest.raises(AssertionError, match="reduction must be a str"):
        linear_cross_entropy(h, w, y, 1.0, 0, None)
    with pytest.raises(ValueError, match="Invalid reduction"):
        linear_cross_entropy(h, w, y, 1.0, "max", None)


def test_backend_validation():
    assert model_utils.validate_fused_backend("hip") == "hip"
    for bad in ("torch", "triton", "cuda"):
        with pytest.raises(ValueError):
            model_utils.validate_fused_backend(bad)


def test_backward_method_knobs_mirror_the_reference():
    """``BackwardEnum`` / ``set_backward_method`` / ``FORCE_FP32_IEEE_PRECISION`` (fused_linear_logprob_triton.py:185-216,
    603-611): the built method is accepted, the others are refused by name, the precision flag exists and is off."""
    from skyrl_amd import fused_linear_logprob_hip as F

    assert (F.BackwardEnum._Total_Fuse_MN, F.BackwardEnum._Total_Separate, F.BackwardEnum._Split_Dlogits_N,
            F.BackwardEnum._Split_Dlogits_M) == (0, 1, 2, 3)
    F.set_backward_method(F.BackwardEnum._Split_Dlogits_N)
    for other in (F.BackwardEnum._Total_Fuse_MN, F.BackwardEnum._Total_Separate, F.BackwardEnum._Split_Dlogits_M):
        with pytest.raises(NotImplementedError):
            F.set_backward_method(other)
    assert F.FORCE_FP32_IEEE_PRECISION is False


def test_policy_loss_names_are_the_reference_registry_names():
    """ppo_utils.py:497-515: the eleven names of PolicyLossRegistry.repopulate_registry, each with six positional arguments
    (log_probs, old_log_probs, advantages, config, loss_mask, rollout_logprobs)."""
    import inspect

    from skyrl_amd import policy_loss as PL

    assert sorted(PL.POLICY_LOSS_FUNCTIONS) == sorted(["regular", "dual_clip", "gspo", "cispo", "clip_cov", "kl_cov", "sapo",
                                                       "cross_entropy", "importance_sampling", "dppo", "rollout_is"])
    for name, fn in PL.POLICY_LOSS_FUNCTIONS.items():
        params = list(inspect.signature(fn).parameters)
        assert params[:6] == ["log_probs", "old_log_probs", "advantages", "config", "loss_mask", "rollout_logprobs"], name
        assert PL.get_policy_loss(name) is fn
    with pytest.raises(ValueError):
        PL.get_policy_loss("nope")


def test_packed_index_helpers_match_brute_force():
    cu = torch.tensor([0, 4, 5, 12, 12, 20])
    _, tok, si, so, sl = model_utils._packed_sequence_indices(cu, 20, torch.device("cpu"))
    want_si, want_so = [], []
    for i in range(len(cu) - 1):
        for o in range(int(cu[i + 1] - cu[i])):
            want_si.append(i), want_so.append(o)
    assert si.tolist() == want_si and so.tolist() == want_so and sl.tolist() == [4, 1, 7, 0, 8]
    rows, offs, lens = model_utils._packed_subseq_row_indices_offsets_and_lens(
        torch.tensor([0, 4, 8, 16]), [[3, 4], [7]], torch.device("cpu"))
    assert rows.tolist() == [0, 0, 1] and offs.tolist() == [0, 4, 0] and lens.tolist() == [3, 4, 7]
    with pytest.raises(ValueError):
        model_utils._packed_subseq_row_indices_offsets_and_lens(torch.tensor([0, 4, 8]), [[3], [4], [1]], torch.device("cpu"))
    with pytest.raises(ValueError):
        model_utils._packed_subseq_row_indices_offsets_and_lens(torch.tensor([0, 4, 8, 9]), [[3], [4]], torch.device("cpu"))


def test_merge_soft_ce_shard_statistics_equals_full_vocabulary():
    """Per-slice soft cross-entropy statistics merged on the host against the full-vocabulary value, fp64."""
    from skyrl_amd.vocab_shards import merge_soft_ce_shard_statistics

    gen = torch.Generator().manual_seed(13)
    T, V = 11, 37
    zs = torch.randn(T, V, dtype=torch.float64, generator=gen) * 3
    zt = torch.randn(T, V, dtype=torch.float64, generator=gen) * 3
    bounds = [0, 1, 9, 30, 37]
    loss, ls, lt = [], [], []
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        a, b = zs[:, lo:hi], zt[:, lo:hi]
        loss.append(-(torch.softmax(b, -1) * torch.log_softmax(a, -1)).sum(-1))
        ls.append(torch.logsumexp(a, -1))
        lt.append(torch.logsumexp(b, -1))
    got, got_ls, got_lt = merge_soft_ce_shard_statistics(torch.stack(loss), torch.stack(ls), torch.stack(lt))
    want = -(torch.softmax(zt, -1) * torch.log_softmax(zs, -1)).sum(-1)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(got_ls, torch.logsumexp(zs, -1), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(got_lt, torch.logsumexp(zt, -1), rtol=1e-12, atol=1e-12)
    with pytest.raises(ValueError):
        merge_soft_ce_shard_statistics(got, got_ls, got_lt)


def test_merge_shard_statistics_equals_full_vocabulary_softmax():
    """The host-side merge of per-slice statistics (what a vocabulary-parallel group's all-reduces compute) against a plain
    log-softmax over the whole vocabulary, fp64, with a token whose target no slice owns."""
    from skyrl_amd.vocab_shards import merge_shard_statistics

    gen = torch.Generator().manual_seed(12)
    T, V = 9, 40
    z = torch.randn(T, V, dtype=torch.float64, generator=gen) * 3
    y = torch.randint(0, V, (T,), generator=gen)
    y[0] = V + 5
    bounds = [0, 7, 8, 29, 40]
    lps, lses, pzs, owners = [], [], [], []
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        zs = z[:, lo:hi]
        lse = torch.logsumexp(zs, -1)
        own = (y >= lo) & (y < hi)
        idx = (y - lo).clamp(0, hi - lo - 1)
        lps.append(torch.where(own, zs.gather(-1, idx[:, None])[:, 0] - lse, torch.zeros(T, dtype=torch.float64)))
        lses.append(lse)
        pzs.append((torch.softmax(zs, -1) * zs).sum(-1))
        owners.append(own)
    lp, ent, lse, pz = merge_shard_statistics(torch.stack(lps), torch.stack(lses), torch.stack(pzs), torch.stack(owners))
    full = torch.log_softmax(z, -1)
    want_lp = full.gather(-1, y.clamp(max=V - 1)[:, None])[:, 0]
    want_lp[0] = 0.0
    torch.testing.assert_close(lp, want_lp, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(ent, -(full.exp() * full).sum(-1), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(lse, torch.logsumexp(z, -1), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(pz, (full.exp() * z).sum(-1), rtol=1e-12, atol=1e-12)
    with pytest.raises(ValueError):
        merge_shard_statistics(lp, lse, pz, torch.stack(owners))


def test_default_vocab_chunk_respects_the_panel_cap():
    """With vocab_chunk = 0 the library picks the dz panel width itself: whatever the shape, the panel holds at most 1.5 GiB
    of dz values (plus row padding), the choice is a multiple of 256 columns no wider than the padded vocabulary, and the
    same query gives the same answer twice."""
    lib = _lib.load()
    for T, H, V in [(16384, 3584, 152064), (32768, 4096, 128256), (8192, 1536, 151936), (300, 128, 1001), (1, 64, 8),
                    (100000, 1024, 50257), (2048, 8192, 262144)]:
        Tb = min(T, 32768)  # the backward walks the tokens in blocks; the scratch is sized by the block
        Tp, Vp, Hp = -(-Tb // 256) * 256, -(-V // 256) * 256, -(-H // 256) * 256
        total = lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, 0)
        assert total == lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, 0)
        fixed = (0 if V % 64 == 0 else 2 * H * (Vp + 64)) + 2 * H * (Tp + 64) + 4 * Tp * Hp
        if T > Tb:  # several blocks: the fp32 matrix in which a bf16 dW is summed over the blocks
            fixed += -(-4 * V * H // 256) * 256
        # the row-compacting variant adds the gathered copies: two [T, H] bf16 matrices and 28 bytes per token (+ counters)
        extra = lib.skyrl_lmhead_bwd_active_rows_workspace_bytes(T, H, V, 0) - total
        assert 4 * T * H + 28 * T <= extra <= 4 * T * H + 28 * T + 4 * (T // 32768 + 2) + 9 * 256, (T, H, V, extra)
        panel = total - fixed
        assert 0 < panel <= (3 << 29) + 2 * Tp * 64 + 4096 or panel <= 2 * Tp * (2048 + 64) + 4096, (T, H, V, panel)
        vc = (panel - 1024) // (2 * Tp) - 64          # the alignment slack is below one row
        vc = -(-vc // 256) * 256
        assert 256 <= vc <= Vp and lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, vc) == total, (T, H, V, vc)


def test_product_never_touches_the_oracle_or_the_working_folder():
    """The checker stays test infrastructure: no module of the package imports, reads or names ``oracle`` or ``_work``, and
    of the two scripts at the root only ``smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` import the oracle."""
    import ast

    def imports(path):
        tree = ast.parse(_read(path))
        found = set()
        for node in ast.walk(tree):
            if isinstance(node, ast.Import):
                found.update(a.name.split(".")[0] for a in node.names)
            elif isinstance(node, ast.ImportFrom) and node.module and node.level == 0:
                found.add(node.module.split(".")[0])
        return found

    pkg = os.path.join(ROOT, "skyrl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                path = os.path.join(dirpath, f)
                text = _read(path)
                assert "_work" not in text.replace("_workspace", "").replace("_workgroup", ""), path
                if f.endswith(".py"):
                    assert "oracle" not in imports(path), path
    for script, allowed in (("bench.py", "cpu_baseline"), ("__graft_entry__.py", "smoke")):
        tree = ast.parse(_read(os.path.join(ROOT, script)))
        for fn in [n for n in ast.walk(tree) if isinstance(n, ast.FunctionDef)]:
            uses = any(isinstance(n, ast.ImportFrom) and n.module == "oracle" for n in ast.walk(fn))
            assert not uses or fn.name == allowed, f"{script}:{fn.name} imports the oracle"
        top_level = [n for n in tree.body if isinstance(n, (ast.Import, ast.ImportFrom))]
        assert not any(isinstance(n, ast.ImportFrom) and n.module == "oracle" for n in top_level)


def test_reduction_enum_of_the_verl_interface():
    """EntropyReductionEnum and its two helpers (fused_linear_logprob_triton.py:146-180): same numbers, same errors."""
    from skyrl_amd import fused_linear_logprob_hip as F

    assert (F.EntropyReductionEnum._None, F.EntropyReductionEnum._Sum, F.EntropyReductionEnum._Mean) == (0, 1, 2)
    assert [F.get_entropy_reduction_enum_number(r) for r in ("none", "sum", "mean")] == [0, 1, 2]
    assert [F.get_entropy_reduction_enum(n) for n in (0, 1, 2)] == [0, 1, 2]
    for bad in ("NONE", "max", ""):
        with pytest.raises(ValueError, match="Invalid reduction"):
            F.get_entropy_reduction_enum_number(bad)
    with pytest.raises(ValueError, match="Invalid ce_reduction"):
        F.get_entropy_reduction_enum(3)


def test_ablation_variants_name_bits_the_kernel_sources_test_for():
    """The timing-only variants of skyrl_amd/bench_ablations.py: unique names, the product first and unmodified, every bit a
    variant sets is tested for by the kernel sources, and the sources default to no ablation."""
    import re

    from skyrl_amd import bench_ablations as A

    names = [v[0] for v in A.VARIANTS]
    assert len(set(names)) == len(names) and A.VARIANTS[0][:2] == ("product", 0)
    csrc = os.path.join(ROOT, "skyrl_amd", "csrc")
    sources = _read(os.path.join(csrc, "lmhead_kernels.hip")) + _read(os.path.join(csrc, "gemm_core.hpp"))
    known = {int(b) for b in re.findall(r"LMHEAD_ABLATE & (\d+)", sources)}
    assert known == {1, 2, 4, 8, 16, 32, 64}
    for name, bits, touched, what in A.VARIANTS:
        assert all(bits & b == 0 or b in known for b in (1 << i for i in range(16))), name
        assert bits < 2 * max(known) and what
        assert set(touched) <= {"lmhead_fwd_tiles", "lmhead_bwd_dz", "lmhead_bwd_gemm"}
        assert A.variant_path(name).startswith(os.path.join(csrc, "ablations"))
    assert sources.count("#define LMHEAD_ABLATE 0") == 2  # each file's default, under #ifndef


def test_bench_refuses_more_than_one_gpu():
    """bench.py --gpus N with N > 1 exits with a message instead of measuring anything."""
    import subprocess
    import sys

    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert proc.returncode != 0
    assert "ONE GPU" in (proc.stdout + proc.stderr)

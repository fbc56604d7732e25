"""The forward entry point that allocates nothing (``skyrl_lmhead_fwd_static_scratch``) against ``skyrl_lmhead_fwd``.

Both are called through the raw C ABI with ctypes.  The static-scratch variant keeps its partial statistics in a fixed array
inside the library's device image and walks the tokens in blocks that fit it; block boundaries are tile boundaries, so the
results must equal the workspace variant's bit for bit.  Two calls in a row share the array, the second on a smaller input.
"""

import pytest
import torch

from oracle import lmhead_oracle as O
from skyrl_amd import _lib

pytestmark = pytest.mark.gpu


def _inputs(T, H, V, seed, dev, oov_every=0):
    gen = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * 3 / H**0.5).to(torch.bfloat16)
    labels = torch.randint(0, V, (T,), generator=gen)
    if oov_every:
        labels[::oov_every] = torch.iinfo(torch.int64).max
    return hidden, weight, labels, hidden.to(dev), weight.to(dev), labels.to(dev)


def _call(lib, static, h, w, y, rcp_temperature, want_entropy=True):
    T, H = h.shape
    V = w.shape[0]
    f32 = dict(dtype=torch.float32, device=h.device)
    out = [torch.full((T,), float("nan"), **f32) for _ in range(4)]  # logprobs, entropy, row_lse, row_pz
    ptr = [t.data_ptr() for t in out]
    if not want_entropy:
        ptr[1] = ptr[3] = None
    stream = torch.cuda.current_stream(h.device).cuda_stream
    common = (h.data_ptr(), h.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), T, H, V, float(rcp_temperature), *ptr)
    if static:
        # Device memory in use, as the driver sees it (this catches an allocation made behind torch's back), must not move.
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(h.device)[0]
        st = lib.skyrl_lmhead_fwd_static_scratch(*common, stream)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(h.device)[0] == free_before, "the static-scratch forward allocated device memory"
    else:
        nbytes = int(lib.skyrl_lmhead_fwd_workspace_bytes(T, H, V))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=h.device)
        st = lib.skyrl_lmhead_fwd(*common, ws.data_ptr(), nbytes, stream)
    _lib.check(st, "forward")
    torch.cuda.synchronize()
    return out


def test_static_scratch_forward_equals_the_workspace_forward(cuda_device):
    lib = _lib.load()
    dev = cuda_device
    assert lib.skyrl_lmhead_static_scratch_bytes() == 32 << 20
    # The library's device image (code and the static array) is loaded on the first launch: do that before memory is watched.
    _, _, _, h, w, y = _inputs(64, 64, 256, 1, dev)
    _call(lib, False, h, w, y, 1.0)
    # First call: three blocks of the 32 MiB array (24 * ceil(V/256) bytes of partials per token: 2353 tokens fit at
    # V = 152064, so blocks of 2304 = 9 tiles), a ragged last tile and out-of-range labels.  Second call: smaller in every extent.
    cases = [((5000, 256, 152064), 0.6, 11, 7), ((300, 128, 5000), 1.0, 12, 0)]
    for (T, H, V), temperature, seed, oov_every in cases:
        hidden, weight, labels, h, w, y = _inputs(T, H, V, seed, dev, oov_every)
        got = _call(lib, True, h, w, y, 1.0 / temperature)
        want = _call(lib, False, h, w, y, 1.0 / temperature)
        for name, a, b in zip(("logprobs", "entropy", "row_lse", "row_pz"), got, want):
            assert torch.equal(a, b), f"{name} differs at T={T}, V={V}"
        # and against the oracle, on the rows either side of every block boundary and at both ends
        rows = torch.tensor(sorted({r for c in (0, 2304, 4608, T) for r in range(c - 40, c + 40) if 0 <= r < T}))
        ref = O.exact_fwd_bwd(hidden[rows], weight, labels[rows], temperature, None, None)
        assert (got[0].cpu()[rows].double() - ref["logprobs"]).abs().max().item() <= 2e-2
        assert ((got[1].cpu()[rows].double() - ref["entropy"]).abs() / ref["entropy"].abs()).max().item() <= 1e-2
    # Without the entropy outputs (the other kernel instantiation), on the array the calls above left behind.
    hidden, weight, labels, h, w, y = _inputs(700, 192, 9000, 13, dev)
    got = _call(lib, True, h, w, y, 1.0, want_entropy=False)
    want = _call(lib, False, h, w, y, 1.0, want_entropy=False)
    assert torch.equal(got[0], want[0]) and torch.equal(got[2], want[2])
    assert torch.isnan(got[1]).all() and torch.isnan(got[3]).all()  # NULL outputs are not written


def test_static_scratch_forward_refuses_what_does_not_fit(cuda_device):
    lib = _lib.load()
    dev = cuda_device
    T, H = 256, 64
    V = 1398016 + 1  # one 256-token tile of partials no longer fits 32 MiB
    h = torch.zeros(T, H, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(V, H, dtype=torch.bfloat16, device=dev)
    y = torch.zeros(T, dtype=torch.int64, device=dev)
    out = torch.empty(T, dtype=torch.float32, device=dev)
    st = lib.skyrl_lmhead_fwd_static_scratch(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), T, H, V, 1.0, out.data_ptr(), None,
                                             None, None, None)
    assert st == -6 and "STATIC_SCRATCH_MAX_V" in _lib.strerror(st)
    with pytest.raises(ValueError):
        _lib.check(st, "skyrl_lmhead_fwd_static_scratch")

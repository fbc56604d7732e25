"""Writes the golden vectors for the fused LM-head path.

The reference stores no golden vectors for this path (its tests are differential), so these are produced from what the
mathematics fixes, with library routines only and in fp64: ``torch.log_softmax`` + ``gather`` for the log-probabilities,
``-(p * log p).sum()`` for the entropy, and ``torch.autograd`` of ``sum(g * logprob) + sum(q * entropy)`` for the gradients.
Neither the oracle (``oracle/``) nor the HIP path is involved, so both can be checked against the files.

Out-of-vocabulary labels follow the reference's contract (model_utils.py:337, 405-411): log-probability 0, gradient keeps the
``-softmax * g`` term.  That is expressed here as ``logprob = z_y * in_vocab - logsumexp(z)`` for the gradient and a masked
fill for the value.

Run from the repository root:  python tests/golden/make_golden.py
"""

import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = [
    # name, T, H, V, temperature, out-of-vocab stride (0 = none), seed
    ("tiny_t1", 1, 64, 8, 1.0, 0, 11),
    ("ragged_tau06", 45, 64, 523, 0.6, 0, 12),
    ("oov_every3", 70, 128, 300, 1.0, 3, 13),
    ("wide_tau13", 130, 128, 700, 1.3, 5, 14),
]


def make(name, T, H, V, temperature, oov_stride, seed):
    gen = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * 3.0 / H**0.5).to(torch.bfloat16)
    labels = torch.randint(0, V, (T,), generator=gen)
    if oov_stride:
        labels[::oov_stride] = torch.iinfo(torch.int64).max
    g = torch.randn(T, generator=gen, dtype=torch.float64)
    q = torch.randn(T, generator=gen, dtype=torch.float64) * 0.3

    h = hidden.double().requires_grad_(True)
    w = weight.double().requires_grad_(True)
    z = (h @ w.t()) / temperature
    lsm = torch.log_softmax(z, dim=-1)
    in_vocab = (labels >= 0) & (labels < V)
    safe = labels.clamp(0, V - 1)
    logprobs = lsm.gather(-1, safe[:, None])[:, 0].masked_fill(~in_vocab, 0.0)
    entropy = -(lsm.exp() * lsm).sum(-1)
    lp_for_grad = z.gather(-1, safe[:, None])[:, 0] * in_vocab - torch.logsumexp(z, dim=-1)
    ((lp_for_grad * g).sum() + (entropy * q).sum()).backward()

    np.savez_compressed(
        os.path.join(HERE, f"{name}.npz"),
        hidden_bits=hidden.view(torch.int16).numpy(),
        weight_bits=weight.view(torch.int16).numpy(),
        labels=labels.numpy(),
        temperature=np.float64(temperature),
        dlogprobs=g.float().numpy(),
        dentropy=q.float().numpy(),
        logprobs=logprobs.detach().numpy(),
        entropy=entropy.detach().numpy(),
        d_hidden=h.grad.float().numpy(),
        d_weight=w.grad.float().numpy(),
    )


if __name__ == "__main__":
    for case in CASES:
        make(*case)
        print("wrote", case[0])

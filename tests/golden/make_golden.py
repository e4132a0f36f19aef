"""Writes the golden vectors ``tests/golden/*.npz``.

Each file holds one small case: the eight inputs (q, k, v, their tangents, the two incoming
gradients; drawn in fp32 and rounded to bf16-representable values, so that every element type of
the kernels sees exactly these numbers), the mask, and the expected outputs computed in fp64 by a
library routine -- PyTorch's math ``scaled_dot_product_attention`` under ``torch.func.jvp``, with
``torch.autograd.grad`` of ``<gO,O> + <gT,O'>`` for the six gradients.  This is the route the
reference's own tests take for O and O' (its ``tests/test_jvp_attention.py:548-561``, ``:595-597``);
the reference holds no vectors on disk.  The row statistics are ``M = log2(sum_j exp(S_ij))`` and
``mu = rowsum(P * S')`` from fp64 torch operations written out here.

Run from the repository root:  ``python tests/golden/make_golden.py [names]``  (CPU, a few seconds).
Expected outputs are stored as float32.
"""
import math
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import sdpa_jvp  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

# name: (Z, H, L, D, mask mode, seed[, key/value heads, key length])
CASES = {
    "dense_L72_D64": (1, 1, 72, 64, "none", 101),
    "causal_L72_D64": (1, 1, 72, 64, "causal", 102),
    "keypad_L72_D32": (2, 1, 72, 32, "keypad", 103),
    "bias_L72_D32": (1, 2, 72, 32, "bias", 104),
    "blockdiag_L136_D64": (1, 1, 136, 64, "blockdiag", 105),
    # beyond the reference's shapes: 4 query heads over 2 key/value heads, 40 queries over 56 keys
    "grouped_cross_L40x56_D32": (1, 4, 40, 32, "random", 106, 2, 56),
}


def _bf16_round(x):
    return x.to(torch.bfloat16).to(torch.float64)


def make_case(Z, H, L, D, mode, seed, Hk=None, Lk=None):
    g = torch.Generator().manual_seed(seed)
    Hk, Lk = Hk or H, Lk or L
    q, qt, go, gt = [_bf16_round(torch.randn(Z, H, L, D, generator=g)) for _ in range(4)]
    k, v, kt, vt = [_bf16_round(torch.randn(Z, Hk, Lk, D, generator=g)) for _ in range(4)]
    if (Hk, Lk) == (H, L):  # the draw order the first five files were written with
        g = torch.Generator().manual_seed(seed)
        q, k, v, qt, kt, vt, go, gt = [_bf16_round(torch.randn(Z, H, L, D, generator=g)) for _ in range(8)]
    scale = 1.0 / math.sqrt(D)
    mask, causal = None, mode == "causal"
    if mode == "keypad":
        lens = torch.tensor([L, L // 2 + 5])[:Z]
        mask = (torch.arange(L)[None, :] < lens[:, None]).view(Z, 1, 1, L)
    elif mode == "bias":
        mask = _bf16_round(torch.randn(Z, H, L, L, generator=g))
    elif mode == "blockdiag":
        seg = torch.bucketize(torch.arange(L), torch.tensor([40, 100]), right=True)
        mask = (seg[:, None] == seg[None, :]).view(1, 1, L, L)
    elif mode == "random":
        mask = torch.rand(Z, 1, L, Lk, generator=g) > 0.4
        mask[..., 0] = True
    if Hk == H:
        o, ot, grads = sdpa_jvp.forward_backward(q, k, v, qt, kt, vt, go, gt, attn_mask=mask, causal=causal, sm_scale=scale)
        ke, kte = k, kt
    else:  # grouped heads: repeat the key/value heads; autograd sums their gradients over each group
        leaves = [x.clone().requires_grad_() for x in (q, k, v, qt, kt, vt)]
        rep = lambda x: x.repeat_interleave(H // Hk, dim=1)  # noqa: E731
        o, ot = sdpa_jvp.forward(leaves[0], rep(leaves[1]), rep(leaves[2]), leaves[3], rep(leaves[4]), rep(leaves[5]),
                                 attn_mask=mask, causal=causal, sm_scale=scale)
        grads = torch.autograd.grad((o * go).sum() + (ot * gt).sum(), leaves)
        o, ot, ke, kte = o.detach(), ot.detach(), rep(k), rep(kt)
    # row statistics, from plain fp64 operations
    s = torch.einsum("zhid,zhjd->zhij", q, ke) * scale
    sp = (torch.einsum("zhid,zhjd->zhij", qt, ke) + torch.einsum("zhid,zhjd->zhij", q, kte)) * scale
    if mask is not None:
        s = s.masked_fill(~mask, float("-inf")) if mask.dtype == torch.bool else s + mask
    if causal:
        s = s.masked_fill(torch.arange(Lk)[None, :] > torch.arange(L)[:, None], float("-inf"))
    M = torch.logsumexp(s, dim=-1) / math.log(2.0)
    mu = (torch.softmax(s, dim=-1) * sp).sum(-1)
    out = dict(q=q, k=k, v=v, qt=qt, kt=kt, vt=vt, go=go, gt=gt, O=o, Ot=ot, M=M, mu=mu,
               dq=grads[0], dk=grads[1], dv=grads[2], dqt=grads[3], dkt=grads[4], dvt=grads[5])
    out = {n: t.to(torch.float32).numpy() for n, t in out.items()}
    out["scale"] = np.float64(scale)
    out["causal"] = np.bool_(causal)
    if mask is not None:
        out["mask"] = mask.numpy() if mask.dtype == torch.bool else mask.to(torch.float32).numpy()
    return out


if __name__ == "__main__":
    only = sys.argv[1:]  # optionally: the names of the files to (re)write
    for name, spec in CASES.items():
        if only and name not in only:
            continue
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **make_case(*spec))
        print("wrote", name)

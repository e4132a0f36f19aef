"""The reference's own oracle: math SDPA under forward-mode AD.  TEST INFRASTRUCTURE ONLY.

Reference ``tests/test_jvp_attention.py:548-561`` runs
``scaled_dot_product_attention`` under ``sdpa_kernel(SDPBackend.MATH)`` inside
``fwAD.dual_level()`` and takes ``unpack_dual(out).tangent`` as the tangent
oracle; ``:595-597`` does the same through ``torch.func.jvp``.  This module is
that route, on CPU, in whatever dtype the inputs have (tests use fp64 or fp32),
extended with ``torch.autograd.grad`` of ``<gO,O> + <gT,O'>`` so the tangent
path has a library-backed oracle too.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch.nn.attention import SDPBackend, sdpa_kernel


def _sdpa(q, k, v, attn_mask, causal, sm_scale):
    with sdpa_kernel(SDPBackend.MATH):
        return F.scaled_dot_product_attention(
            q, k, v, attn_mask=attn_mask, dropout_p=0.0, is_causal=causal, scale=sm_scale
        )


def forward(q, k, v, qt, kt, vt, attn_mask=None, causal=False, sm_scale=None):
    """(O, O') by ``torch.func.jvp`` of math SDPA (reference test lines 595-597)."""
    fn = lambda a, b, c: _sdpa(a, b, c, attn_mask, causal, sm_scale)  # noqa: E731
    o, ot = torch.func.jvp(fn, (q, k, v), (qt, kt, vt))
    return o, ot


def forward_backward(q, k, v, qt, kt, vt, go, gt, attn_mask=None, causal=False, sm_scale=None):
    """O, O' and the six gradients of ``sum(O*gO) + sum(O'*gT)``.

    ``gt`` may be ``None`` (first-order backward only, what the reference's
    ``backward`` implements, ``jvp_attention.py:2831``).
    """
    leaves = [t.detach().clone().requires_grad_(True) for t in (q, k, v, qt, kt, vt)]
    o, ot = forward(*leaves, attn_mask=attn_mask, causal=causal, sm_scale=sm_scale)
    loss = (o * go).sum()
    if gt is not None:
        loss = loss + (ot * gt).sum()
    grads = torch.autograd.grad(loss, leaves, allow_unused=True)
    grads = [torch.zeros_like(x) if g is None else g for g, x in zip(grads, leaves)]
    return o.detach(), ot.detach(), grads

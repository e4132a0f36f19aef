"""Tile-loop restatement of the fused dual forward and its backward.  TEST INFRASTRUCTURE ONLY.

Plain PyTorch on CPU, any float dtype (tests use fp64 and fp32).  The forward
follows the reference's online-softmax loop over key tiles
(``jvp_flash_attention/jvp_attention.py:226-335``): running max ``m`` in the
log2 domain (``qk_scale = sm_scale * log2(e)``, ``:929-930``), running sum
``l``, and the accumulators rescaled by ``alpha = exp2(m_old - m_new)``
(``:279-283``, ``:294``, ``:312-318``).  The reference keeps three accumulators
(``acc``, ``g_acc``, ``p_tv_acc``, ``:872``, ``:916-918``); ``g_acc`` and
``p_tv_acc`` share one rescale and are only ever added (``:1031-1033``), so
they are merged here into ``t_acc = sum((p*s') V + p V')``.  Epilogue
(``:1010-1033``): ``O = acc/l``, ``mu = mu_acc/l``, ``O' = t_acc/l - mu*O``,
``M = m + log2(l)``; rows with ``l == 0`` give zeros (``:1011-1015``).

The backward recomputes ``P = exp2(S*log2e - M)`` per tile pair as the
reference does (``:1509-1512``, ``:1659-1662``) with ``delta = rowsum(O*dO)``
from a pre-pass (``:1384-1411``), and adds the tangent-path terms the
reference does not have (its ``backward`` ignores the second incoming
gradient, ``:2831``).

Mask semantics follow SDPA (bool True = attend; float added after scaling).

Beyond the reference's one shape for q, k and v: k and v may be ``(Z, H_kv, L_kv, D)`` with
``H % H_kv == 0`` (query head ``h`` reads key/value head ``h // (H / H_kv)``; their gradients
are summed over the group) and any ``L_kv`` (causal = key index <= query index).
"""
from __future__ import annotations

import math

import torch

LOG2E = 1.4426950408889634


def _tile_logits(qi, kj, scale, mask, causal, i0, j0):
    """log2-domain logits of one (query tile, key tile) pair and its attend pattern."""
    s = torch.matmul(qi, kj.transpose(-1, -2)) * scale
    bi, bj = qi.shape[-2], kj.shape[-2]
    keep = torch.ones(s.shape, dtype=torch.bool)
    if causal:
        rows = torch.arange(i0, i0 + bi).unsqueeze(-1)
        cols = torch.arange(j0, j0 + bj).unsqueeze(0)
        keep = keep & (rows >= cols)
    if mask is not None:
        Lq = max(mask.shape[-2], i0 + bi)  # a mask row of extent 1 is shared by every query
        mt = mask.expand(s.shape[0], s.shape[1], Lq, mask.shape[-1])[..., i0 : i0 + bi, j0 : j0 + bj]
        if mask.dtype == torch.bool:
            keep = keep & mt
        else:
            s = s + mt.to(s.dtype)
    keep = keep & ~torch.isneginf(s)
    return s * LOG2E, keep


def _group(x, H):
    """Key/value heads repeated so that each query head finds its own at the same index."""
    return x if x is None or x.shape[1] == H else x.repeat_interleave(H // x.shape[1], dim=1)


def _ungroup(x, Hk):
    """Per-query-head key/value gradients summed over each group of heads."""
    Z, H, Lk, D = x.shape
    return x if H == Hk else x.view(Z, Hk, H // Hk, Lk, D).sum(2)


def forward(q, k, v, qt=None, kt=None, vt=None, mask=None, causal=False, scale=None, bm=32, bn=32):
    """Online-softmax dual forward.  Returns (O, O' or None, M, mu or None)."""
    Z, H, L, D = q.shape
    Lk = k.shape[2]
    k, v, kt, vt = (_group(x, H) for x in (k, v, kt, vt))
    scale = D**-0.5 if scale is None else scale
    dual = qt is not None
    o = torch.zeros_like(q)
    ot = torch.zeros_like(q) if dual else None
    M = torch.zeros(Z, H, L, dtype=q.dtype)
    mu_out = torch.zeros(Z, H, L, dtype=q.dtype) if dual else None
    for i0 in range(0, L, bm):
        i1 = min(i0 + bm, L)
        qi = q[:, :, i0:i1]
        rows = i1 - i0
        m = torch.full((Z, H, rows, 1), -math.inf, dtype=q.dtype)
        l = torch.zeros(Z, H, rows, 1, dtype=q.dtype)
        acc = torch.zeros(Z, H, rows, D, dtype=q.dtype)
        t_acc = torch.zeros_like(acc)
        mu = torch.zeros_like(l)
        hi = min(i1, Lk) if causal else Lk  # causal: tiles right of the diagonal are skipped
        for j0 in range(0, hi, bn):
            j1 = min(j0 + bn, Lk)
            s2, keep = _tile_logits(qi, k[:, :, j0:j1], scale, mask, causal, i0, j0)
            s2 = torch.where(keep, s2, torch.full_like(s2, -math.inf))
            m_new = torch.maximum(m, s2.amax(-1, keepdim=True))
            m_use = torch.where(torch.isfinite(m_new), m_new, torch.zeros_like(m_new))
            p = torch.where(keep, torch.exp2(s2 - m_use), torch.zeros_like(s2))
            alpha = torch.exp2(m - m_use)
            l = l * alpha + p.sum(-1, keepdim=True)
            acc = acc * alpha + torch.matmul(p, v[:, :, j0:j1])
            if dual:
                sp = scale * (
                    torch.matmul(qt[:, :, i0:i1], k[:, :, j0:j1].transpose(-1, -2))
                    + torch.matmul(qi, kt[:, :, j0:j1].transpose(-1, -2))
                )
                ps = p * sp
                mu = mu * alpha + ps.sum(-1, keepdim=True)
                t_acc = t_acc * alpha + torch.matmul(ps, v[:, :, j0:j1]) + torch.matmul(p, vt[:, :, j0:j1])
            m = m_new
        dead = l == 0
        l_safe = torch.where(dead, torch.ones_like(l), l)
        oi = acc / l_safe
        o[:, :, i0:i1] = oi
        M[:, :, i0:i1] = torch.where(dead, torch.full_like(l, math.inf), m + torch.log2(l_safe))[..., 0]
        if dual:
            mu_i = mu / l_safe
            ot[:, :, i0:i1] = t_acc / l_safe - mu_i * oi
            mu_out[:, :, i0:i1] = mu_i[..., 0]
    return o, ot, M, mu_out


def backward(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt=None, mask=None, causal=False, scale=None,
             bm=32, bn=32):
    """Tile-pair backward recomputing P from M.  Returns dict of six gradients.

    ``qt/kt/vt/ot/mu`` may be ``None`` when ``gt`` is ``None`` (first-order backward of a
    plain forward).
    """
    Z, H, L, D = q.shape
    Hk, Lk = k.shape[1], k.shape[2]
    k, v, kt, vt = (_group(x, H) for x in (k, v, kt, vt))
    scale = D**-0.5 if scale is None else scale
    dual = gt is not None
    g = {n: torch.zeros_like(q) for n in ("dq", "dqt")}
    g.update({n: torch.zeros_like(k) for n in ("dk", "dv", "dkt", "dvt")})
    # pre-pass row statistics (reference delta at jvp_attention.py:1384-1411, plus the tangent ones)
    d1 = (go * o).sum(-1, keepdim=True)
    if dual:
        a = (gt * o).sum(-1, keepdim=True)
        d2 = (gt * ot).sum(-1, keepdim=True) - a * mu.unsqueeze(-1)
    for i0 in range(0, L, bm):
        i1 = min(i0 + bm, L)
        hi = min(i1, Lk) if causal else Lk
        Mi = M[:, :, i0:i1].unsqueeze(-1)
        for j0 in range(0, hi, bn):
            j1 = min(j0 + bn, Lk)
            kj, vj = k[:, :, j0:j1], v[:, :, j0:j1]
            s2, keep = _tile_logits(q[:, :, i0:i1], kj, scale, mask, causal, i0, j0)
            p = torch.where(keep, torch.exp2(s2 - Mi), torch.zeros_like(s2))
            ds = p * (torch.matmul(go[:, :, i0:i1], vj.transpose(-1, -2)) - d1[:, :, i0:i1])
            g["dv"][:, :, j0:j1] += torch.matmul(p.transpose(-1, -2), go[:, :, i0:i1])
            if dual:
                ktj, vtj = kt[:, :, j0:j1], vt[:, :, j0:j1]
                sp = scale * (
                    torch.matmul(qt[:, :, i0:i1], kj.transpose(-1, -2))
                    + torch.matmul(q[:, :, i0:i1], ktj.transpose(-1, -2))
                )
                mui = mu[:, :, i0:i1].unsqueeze(-1)
                A = torch.matmul(gt[:, :, i0:i1], vj.transpose(-1, -2))
                B = torch.matmul(gt[:, :, i0:i1], vtj.transpose(-1, -2))
                ai = a[:, :, i0:i1]
                ds = ds + p * (B + A * (sp - mui) - ai * sp - d2[:, :, i0:i1])
                dsp = p * (A - ai)
                pp = p * (sp - mui)
                g["dv"][:, :, j0:j1] += torch.matmul(pp.transpose(-1, -2), gt[:, :, i0:i1])
                g["dvt"][:, :, j0:j1] += torch.matmul(p.transpose(-1, -2), gt[:, :, i0:i1])
                g["dq"][:, :, i0:i1] += scale * torch.matmul(dsp, ktj)
                g["dk"][:, :, j0:j1] += scale * torch.matmul(dsp.transpose(-1, -2), qt[:, :, i0:i1])
                g["dqt"][:, :, i0:i1] += scale * torch.matmul(dsp, kj)
                g["dkt"][:, :, j0:j1] += scale * torch.matmul(dsp.transpose(-1, -2), q[:, :, i0:i1])
            g["dq"][:, :, i0:i1] += scale * torch.matmul(ds, kj)
            g["dk"][:, :, j0:j1] += scale * torch.matmul(ds.transpose(-1, -2), q[:, :, i0:i1])
    for n in ("dk", "dv", "dkt", "dvt"):
        g[n] = _ungroup(g[n], Hk)
    return g

"""Closed-form dense fp64 statement of JVP attention.  TEST INFRASTRUCTURE ONLY.

Numpy only, no autograd.  Per (z, h):

    S  = scale * Q K^T (+ bias; -inf where masked)        P = softmax(S)
    O  = P V
    S' = scale * (Q' K^T + Q K'^T)                        mu = rowsum(P * S')
    P' = P * (S' - mu)                                    O' = P' V + P V'

which is what the reference's tile loop accumulates
(``jvp_flash_attention/jvp_attention.py:232-236`` for S and S', ``:301-318`` for
the three accumulators, ``:1030-1033`` for ``O' = g_acc/l - (mu/l) O + p_tv_acc/l``).
Masks follow SDPA: boolean True = attend, float = added to the *scaled*
logits (the reference adds it before scaling, ``:247-251``; not reproduced).
Rows with every key masked give O = O' = 0 and zero gradients, as the
reference's ``l == 0 -> l = 1`` epilogue does (``:1011-1015``).

Backward for ``Loss = <gO, O> + <gT, O'>`` (the gT = 0 case is the reference's
``dv += pT dO; dsT = pT * (dpT - delta); dk += dsT q`` at ``:1541-1553`` and
``dq += ds k`` at ``:1687-1697``):

    d1 = rowsum(gO * O)        dS1 = P * (gO V^T - d1)
    A  = gT V^T   B = gT V'^T  a = rowsum(gT * O)   d2 = rowsum(gT * O') - a * mu
    dS2 = P * (B + A * (S' - mu) - a * S' - d2)     dS' = P * (A - a)
    dS  = dS1 + dS2
    dQ = scale (dS K + dS' K')   dK = scale (dS^T Q + dS'^T Q')   dV = P^T gO + P'^T gT
    dQ' = scale dS' K            dK' = scale dS'^T Q              dV' = P^T gT

Dropout (dead code in the reference, ``:94-122``, ``:271-277``, which raises for ``dropout_p > 0`` at
``:2356-2357``; semantics here are SDPA's): a fixed matrix W = keep / (1 - p) multiplies the probabilities
wherever they meet V or V' and nowhere else, so mu stays the undropped ``rowsum(P * S')``:

    O = (P*W) V      O' = (P'*W) V + (P*W) V'
    backward: gO V^T, A and B are multiplied by W; dV = (P*W)^T gO + (P'*W)^T gT; dV' = (P*W)^T gT
"""
from __future__ import annotations

import numpy as np

LOG2E = 1.4426950408889634


def _expand_heads(x, H):
    """Grouped heads (not in the reference, which requires q, k, v of one shape, ``:2367-2378``): k, v
    may have fewer heads than q; query head h reads key/value head h // (H / Hk)."""
    Hk = x.shape[1]
    assert H % Hk == 0, "the number of query heads must be a multiple of the number of key/value heads"
    return x if Hk == H else np.repeat(x, H // Hk, axis=1)


def _reduce_heads(g, Hk):
    Z, H, L, D = g.shape
    return g if H == Hk else g.reshape(Z, Hk, H // Hk, L, D).sum(axis=2)


def _logits(q, k, mask, causal, scale):
    """Scaled, masked logits S (fp64) and the boolean 'attend' pattern.  q and k may differ in length;
    causal then means key index <= query index, as in SDPA."""
    Lq, Lk = q.shape[-2], k.shape[-2]
    s = scale * np.einsum("zhid,zhjd->zhij", q, k)
    keep = np.ones(s.shape, dtype=bool)
    if causal:
        keep &= np.tril(np.ones((Lq, Lk), dtype=bool))
    if mask is not None:
        mask = np.asarray(mask)
        if mask.dtype == np.bool_:
            keep &= np.broadcast_to(mask, s.shape)
        else:
            s = s + np.broadcast_to(mask.astype(np.float64), s.shape)
    keep &= ~np.isneginf(s)
    return s, keep


def _softmax(s, keep):
    s = np.where(keep, s, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    e = np.where(keep, np.exp(s - m_safe), 0.0)
    l = e.sum(axis=-1, keepdims=True)
    p = e / np.where(l > 0, l, 1.0)
    with np.errstate(divide="ignore"):
        lse2 = np.where(l > 0, (m_safe + np.log(np.where(l > 0, l, 1.0))) * LOG2E, np.inf)
    return p, lse2[..., 0]


def forward(q, k, v, qt=None, kt=None, vt=None, mask=None, causal=False, scale=None, keep_scale=None):
    """Returns dict with O, M and (when tangents are given) O', mu, plus P, S' for reuse.  ``keep_scale`` is
    the dropout matrix W (broadcastable to Z, H, Lq, Lk), ``None`` for no dropout."""
    q, k, v = (np.asarray(x, dtype=np.float64) for x in (q, k, v))
    D, H = q.shape[-1], q.shape[1]
    k, v = _expand_heads(k, H), _expand_heads(v, H)
    scale = D**-0.5 if scale is None else scale
    s, keep = _logits(q, k, mask, causal, scale)
    p, M = _softmax(s, keep)
    w = 1.0 if keep_scale is None else np.broadcast_to(np.asarray(keep_scale, dtype=np.float64), p.shape)
    out = {"O": (p * w) @ v, "M": M, "P": p, "scale": scale, "W": w}
    if qt is not None:
        qt, kt, vt = (np.asarray(x, dtype=np.float64) for x in (qt, kt, vt))
        kt, vt = _expand_heads(kt, H), _expand_heads(vt, H)
        sp = scale * (np.einsum("zhid,zhjd->zhij", qt, k) + np.einsum("zhid,zhjd->zhij", q, kt))
        mu = (p * sp).sum(-1, keepdims=True)
        pp = p * (sp - mu)
        out.update({"Ot": (pp * w) @ v + (p * w) @ vt, "mu": mu[..., 0], "Sp": sp, "Pp": pp})
    return out


def backward(q, k, v, qt, kt, vt, go, gt=None, mask=None, causal=False, scale=None, keep_scale=None):
    """Six gradients of <gO,O> + <gT,O'>.  ``gt=None`` means gT = 0."""
    if qt is None:
        qt, kt, vt = (np.zeros_like(np.asarray(x, dtype=np.float64)) for x in (q, k, v))
    f = forward(q, k, v, qt, kt, vt, mask=mask, causal=causal, scale=scale, keep_scale=keep_scale)
    q, k, v, qt, kt, vt, go = (np.asarray(x, dtype=np.float64) for x in (q, k, v, qt, kt, vt, go))
    H, Hk = q.shape[1], k.shape[1]
    k, v, kt, vt = (_expand_heads(x, H) for x in (k, v, kt, vt))
    p, sc, w = f["P"], f["scale"], f["W"]
    T = lambda x: np.swapaxes(x, -1, -2)  # noqa: E731
    d1 = (go * f["O"]).sum(-1, keepdims=True)
    ds = p * (w * (go @ T(v)) - d1)
    dv = T(p * w) @ go
    dsp = np.zeros_like(p)
    dvt = np.zeros_like(v)
    if gt is not None:
        gt = np.asarray(gt, dtype=np.float64)
        sp, mu = f["Sp"], f["mu"][..., None]
        A = w * (gt @ T(v))
        B = w * (gt @ T(vt))
        a = (gt * f["O"]).sum(-1, keepdims=True)
        d2 = (gt * f["Ot"]).sum(-1, keepdims=True) - a * mu
        ds = ds + p * (B + A * (sp - mu) - a * sp - d2)
        dsp = p * (A - a)
        dv = dv + T(f["Pp"] * w) @ gt
        dvt = T(p * w) @ gt
    return {
        "dq": sc * (ds @ k + dsp @ kt),
        "dk": _reduce_heads(sc * (T(ds) @ q + T(dsp) @ qt), Hk),
        "dv": _reduce_heads(dv, Hk),
        "dqt": sc * (dsp @ k),
        "dkt": _reduce_heads(sc * (T(dsp) @ q), Hk),
        "dvt": _reduce_heads(dvt, Hk),
    }

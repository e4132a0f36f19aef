"""A stand-in for the HIP backend so that the host logic (argument checks, autograd wiring,
dual-tensor handling) can be exercised on a machine without a GPU.  It computes with the oracle's
tile-loop restatement on CPU tensors.  Test infrastructure only: the shipped package never
imports it."""
import contextlib

import torch

from jvp_flash_attention_amd import _lib
from oracle import dense, dropout, tiled


class OracleBackend:
    name = "oracle-cpu"

    def __init__(self):
        self.calls = []

    @staticmethod
    def _mask(mask, kind):
        return None if kind == _lib.MASK_NONE else mask

    def fwd(self, q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p=0.0, dropout_seed=0):
        self.calls.append(("fwd", qt is not None, mask_kind, bool(causal)) + ((dropout_p, dropout_seed) if dropout_p else ()))
        if dropout_p:
            return self._fwd_dropout(q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p, dropout_seed)
        G = q.shape[1] // k.shape[1]  # grouped heads: the tile-loop restatement wants them repeated
        f = lambda t: None if t is None else (t.double() if t.shape[1] == q.shape[1] else t.double().repeat_interleave(G, 1))  # noqa: E731
        m = self._mask(mask, mask_kind)
        m = m if m is None or m.dtype == torch.bool else m.double()
        o, ot, M, mu = tiled.forward(f(q), f(k), f(v), f(qt), f(kt), f(vt), mask=m, causal=causal, scale=sm_scale)
        c = lambda t: None if t is None else t.to(q.dtype)  # noqa: E731
        return c(o), c(ot), M.float(), None if mu is None else mu.float()

    def _fwd_dropout(self, q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, p, seed):
        """With dropout the dense closed form stands in (the tile-loop restatement has no dropout)."""
        n = lambda t: None if t is None else t.double().numpy()  # noqa: E731
        W = dropout.keep_scale(q.shape[0], q.shape[1], q.shape[2], k.shape[2], p, seed)
        m = self._mask(mask, mask_kind)
        f = dense.forward(n(q), n(k), n(v), n(qt), n(kt), n(vt), mask=None if m is None else m.numpy(),
                          causal=causal, scale=sm_scale, keep_scale=W)
        c = lambda a, dt=q.dtype: torch.from_numpy(a).to(dt)  # noqa: E731
        dual = qt is not None
        return (c(f["O"]), c(f["Ot"]) if dual else None, c(f["M"], torch.float32),
                c(f["mu"], torch.float32) if dual else None)

    def _bwd_dropout(self, q, k, v, qt, kt, vt, go, gt, mask, mask_kind, causal, sm_scale, want_t, p, seed):
        n = lambda t: None if t is None else t.double().numpy()  # noqa: E731
        W = dropout.keep_scale(q.shape[0], q.shape[1], q.shape[2], k.shape[2], p, seed)
        m = self._mask(mask, mask_kind)
        g = dense.backward(n(q), n(k), n(v), n(qt), n(kt), n(vt), n(go), n(gt), mask=None if m is None else m.numpy(),
                           causal=causal, scale=sm_scale, keep_scale=W)
        c = lambda a: torch.from_numpy(a).to(q.dtype)  # noqa: E731
        tg = (c(g["dqt"]), c(g["dkt"]), c(g["dvt"])) if want_t else (None, None, None)
        return (c(g["dq"]), c(g["dk"]), c(g["dv"]), *tg)

    def bwd(self, q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale,
            want_tangent_grads=False, dropout_p=0.0, dropout_seed=0):
        self.calls.append(("bwd", gt is not None, mask_kind, bool(causal), want_tangent_grads)
                          + ((dropout_p, dropout_seed) if dropout_p else ()))
        if dropout_p:
            if go is None:
                go = torch.zeros_like(q)
            return self._bwd_dropout(q, k, v, qt, kt, vt, go, gt, mask, mask_kind, causal, sm_scale,
                                     want_tangent_grads, dropout_p, dropout_seed)
        Z, H, Hk = q.shape[0], q.shape[1], k.shape[1]
        f = lambda t: None if t is None else (t.double() if t.dim() != 4 or t.shape[1] == H else t.double().repeat_interleave(H // Hk, 1))  # noqa: E731
        m = self._mask(mask, mask_kind)
        m = m if m is None or m.dtype == torch.bool else m.double()
        if go is None:
            go = torch.zeros_like(q)
        g = tiled.backward(f(q), f(k), f(v), f(qt), f(kt), f(vt), f(o), f(ot), f(M), f(mu), f(go), f(gt),
                           mask=m, causal=causal, scale=sm_scale)
        c = lambda t: t.to(q.dtype)  # noqa: E731
        kv = lambda t: c(t if Hk == H else t.reshape(Z, Hk, H // Hk, *t.shape[2:]).sum(2))  # noqa: E731
        tg = (c(g["dqt"]), kv(g["dkt"]), kv(g["dvt"])) if want_tangent_grads else (None, None, None)
        return (c(g["dq"]), kv(g["dk"]), kv(g["dv"]), *tg)


@contextlib.contextmanager
def oracle_backend():
    saved = _lib._backend
    fake = OracleBackend()
    _lib._backend = fake
    try:
        yield fake
    finally:
        _lib._backend = saved

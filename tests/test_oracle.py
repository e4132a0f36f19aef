"""Pin the CPU oracle before anything is compared with it.

The reference holds no golden vectors (its test file has no ``test_*`` functions and no data
files); what pins results there is a live comparison with PyTorch math SDPA under forward-mode AD
(reference ``tests/test_jvp_attention.py:548-561``, ``:595-597``).  So the oracle is pinned by
(1) that same library route, (2) finite differences, which share nothing with autograd or with the
closed form, (3) invariants of the mathematics, and (4) agreement of the tile-loop restatement with
the dense closed form for several tile sizes, ragged L included.
"""
import math

import numpy as np
import pytest
import torch

from oracle import dense, sdpa_jvp, tiled

torch.manual_seed(0)


def _inputs(Z=2, H=2, L=32, D=16, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(Z, H, L, D, generator=g, dtype=dtype) for _ in range(8)]


def _masks(Z, H, L, seed=1):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(L // 2, L + 1, (Z,), generator=g)
    keypad = (torch.arange(L)[None, :] < lens[:, None]).view(Z, 1, 1, L)
    bias = torch.randn(Z, H, L, L, generator=g, dtype=torch.float64)
    rnd = torch.rand(Z, H, L, L, generator=g) > 0.7
    rnd[..., 0] = True  # no fully masked row
    return {"none": (None, False), "causal": (None, True), "keypad": (keypad, False),
            "bias": (bias, False), "random_bool": (rnd, False)}


MODES = ["none", "causal", "keypad", "bias", "random_bool"]


@pytest.mark.parametrize("mode", MODES)
def test_dense_matches_sdpa_library_route(mode):
    q, k, v, qt, kt, vt, go, gt = _inputs()
    mask, causal = _masks(2, 2, 32)[mode]
    o, ot, grads = sdpa_jvp.forward_backward(q, k, v, qt, kt, vt, go, gt, attn_mask=mask, causal=causal)
    npm = None if mask is None else mask.numpy()
    f = dense.forward(*(x.numpy() for x in (q, k, v, qt, kt, vt)), mask=npm, causal=causal)
    b = dense.backward(*(x.numpy() for x in (q, k, v, qt, kt, vt, go, gt)), mask=npm, causal=causal)
    assert np.abs(f["O"] - o.numpy()).max() < 1e-12
    assert np.abs(f["Ot"] - ot.numpy()).max() < 1e-12
    for name, ref in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert np.abs(b[name] - ref.numpy()).max() < 1e-11, name
    # gT = None is the reference's first-order backward
    _, _, g1 = sdpa_jvp.forward_backward(q, k, v, qt, kt, vt, go, None, attn_mask=mask, causal=causal)
    b1 = dense.backward(*(x.numpy() for x in (q, k, v, qt, kt, vt, go)), None, mask=npm, causal=causal)
    for name, ref in zip(("dq", "dk", "dv"), g1):
        assert np.abs(b1[name] - ref.numpy()).max() < 1e-11, name
    for name in ("dqt", "dkt", "dvt"):
        assert np.abs(b1[name]).max() == 0.0


@pytest.mark.parametrize("mode", ["none", "causal", "bool", "bias"])
@pytest.mark.parametrize("Hk,Lk", [(1, 24), (2, 40), (4, 24)])
def test_dense_with_grouped_heads_and_unequal_lengths_matches_the_library_route(mode, Hk, Lk):
    """Beyond the reference (which requires q, k, v of one shape): fewer key/value heads than query
    heads and a key length that differs from the query length.  The library route repeats the
    key/value heads explicitly, so autograd sums their gradients over each group."""
    Z, H, Lq, D = 2, 4, 24, 16
    g = torch.Generator().manual_seed(7)
    q, qt, go, gt = [torch.randn(Z, H, Lq, D, generator=g, dtype=torch.float64) for _ in range(4)]
    k, v, kt, vt = [torch.randn(Z, Hk, Lk, D, generator=g, dtype=torch.float64) for _ in range(4)]
    mask, causal = None, mode == "causal"
    if mode == "bool":
        mask = torch.rand(Z, H, Lq, Lk, generator=g) > 0.5
        mask[..., 0] = True
    if mode == "bias":
        mask = torch.randn(Z, 1, Lq, Lk, generator=g, dtype=torch.float64)
    leaves = [x.clone().requires_grad_() for x in (q, k, v, qt, kt, vt)]
    rep = lambda x: x.repeat_interleave(H // Hk, dim=1)  # noqa: E731
    o, ot = sdpa_jvp.forward(leaves[0], rep(leaves[1]), rep(leaves[2]), leaves[3], rep(leaves[4]), rep(leaves[5]),
                             attn_mask=mask, causal=causal)
    grads = torch.autograd.grad((o * go).sum() + (ot * gt).sum(), leaves)
    npm = None if mask is None else mask.numpy()
    f = dense.forward(*(x.numpy() for x in (q, k, v, qt, kt, vt)), mask=npm, causal=causal)
    b = dense.backward(*(x.numpy() for x in (q, k, v, qt, kt, vt, go, gt)), mask=npm, causal=causal)
    assert np.abs(f["O"] - o.detach().numpy()).max() < 1e-12
    assert np.abs(f["Ot"] - ot.detach().numpy()).max() < 1e-12
    for name, ref in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert b[name].shape == tuple(ref.shape), name
        assert np.abs(b[name] - ref.numpy()).max() < 1e-11, name


def test_dense_M_and_mu_definitions():
    q, k, v, qt, kt, vt, _, _ = _inputs()
    f = dense.forward(*(x.numpy() for x in (q, k, v, qt, kt, vt)))
    s = (q @ k.transpose(-1, -2)) * q.shape[-1] ** -0.5
    assert np.abs(f["M"] - (torch.logsumexp(s, -1) * dense.LOG2E).numpy()).max() < 1e-12
    assert np.abs(f["P"].sum(-1) - 1).max() < 1e-12


@pytest.mark.parametrize("mode", ["none", "causal", "bias"])
def test_tangent_is_directional_derivative_by_finite_difference(mode):
    q, k, v, qt, kt, vt, _, _ = [x.numpy() for x in _inputs(Z=1, H=1, L=32, D=8, seed=3)]
    mask, causal = _masks(1, 1, 32)[mode]
    npm = None if mask is None else mask.numpy()
    eps = 1e-6
    fp = dense.forward(q + eps * qt, k + eps * kt, v + eps * vt, mask=npm, causal=causal)["O"]
    fm = dense.forward(q - eps * qt, k - eps * kt, v - eps * vt, mask=npm, causal=causal)["O"]
    fd = (fp - fm) / (2 * eps)
    ot = dense.forward(q, k, v, qt, kt, vt, mask=npm, causal=causal)["Ot"]
    assert np.abs(fd - ot).max() < 1e-7


@pytest.mark.parametrize("mode", ["none", "causal", "keypad"])
def test_backward_by_brute_force_finite_difference(mode):
    """d/dx [<gO,O> + <gT,O'>] entry by entry on a tiny problem; no autograd, no closed form."""
    Z, H, L, D = 1, 1, 8, 4
    xs = [x.numpy() for x in _inputs(Z, H, L, D, seed=5)]
    q, k, v, qt, kt, vt, go, gt = xs
    mask, causal = _masks(Z, H, L)[mode]
    npm = None if mask is None else mask.numpy()

    def loss(args):
        f = dense.forward(*args, mask=npm, causal=causal)
        return (f["O"] * go).sum() + (f["Ot"] * gt).sum()

    b = dense.backward(q, k, v, qt, kt, vt, go, gt, mask=npm, causal=causal)
    eps = 1e-6
    for idx, name in enumerate(("dq", "dk", "dv", "dqt", "dkt", "dvt")):
        fd = np.zeros_like(xs[idx])
        for pos in np.ndindex(*xs[idx].shape):
            args_p = [a.copy() for a in xs[:6]]
            args_m = [a.copy() for a in xs[:6]]
            args_p[idx][pos] += eps
            args_m[idx][pos] -= eps
            fd[pos] = (loss(args_p) - loss(args_m)) / (2 * eps)
        assert np.abs(fd - b[name]).max() < 1e-7, name


def test_invariants():
    q, k, v, qt, kt, vt, go, gt = [x.numpy() for x in _inputs(seed=7)]
    # rows of P' sum to zero: constant V and V' = 0 give O' = 0
    f = dense.forward(q, k, np.ones_like(v) * 3.0, qt, kt, np.zeros_like(vt))
    assert np.abs(f["Ot"]).max() < 1e-12
    assert np.abs(f["Pp"].sum(-1)).max() < 1e-12
    # O' is linear in the tangents
    f1 = dense.forward(q, k, v, qt, kt, vt)["Ot"]
    f2 = dense.forward(q, k, v, 2 * qt, 2 * kt, 2 * vt)["Ot"]
    assert np.abs(f2 - 2 * f1).max() < 1e-12
    fa = dense.forward(q, k, v, qt, 0 * kt, 0 * vt)["Ot"]
    fb = dense.forward(q, k, v, 0 * qt, kt, 0 * vt)["Ot"]
    fc = dense.forward(q, k, v, 0 * qt, 0 * kt, vt)["Ot"]
    assert np.abs(fa + fb + fc - f1).max() < 1e-12
    # V' only: O' = P V'
    assert np.abs(fc - dense.forward(q, k, vt)["O"]).max() < 1e-12
    # single key attended (L=1 effectively via mask): O = V row, O' = V' row
    L = q.shape[-2]
    only0 = np.zeros((1, 1, L, L), dtype=bool)
    only0[..., 0] = True
    f0 = dense.forward(q, k, v, qt, kt, vt, mask=only0)
    assert np.abs(f0["O"] - v[:, :, :1]).max() < 1e-12
    assert np.abs(f0["Ot"] - vt[:, :, :1]).max() < 1e-12
    # dV' = P^T gT is the transpose-action of O' = ... + P V'
    b = dense.backward(q, k, v, qt, kt, vt, go, gt)
    P = dense.forward(q, k, v)["P"]
    assert np.abs(b["dvt"] - np.swapaxes(P, -1, -2) @ gt).max() < 1e-12


def test_fully_masked_rows_give_zeros():
    q, k, v, qt, kt, vt, go, gt = [x.numpy() for x in _inputs(Z=1, H=1, L=16, D=8, seed=9)]
    mask = np.ones((1, 1, 16, 16), dtype=bool)
    mask[0, 0, 3, :] = False
    f = dense.forward(q, k, v, qt, kt, vt, mask=mask)
    assert np.all(f["O"][0, 0, 3] == 0) and np.all(f["Ot"][0, 0, 3] == 0)
    assert np.isposinf(f["M"][0, 0, 3])
    b = dense.backward(q, k, v, qt, kt, vt, go, gt, mask=mask)
    assert np.all(b["dq"][0, 0, 3] == 0) and np.all(np.isfinite(b["dk"]))
    o, ot, M, mu = tiled.forward(*(torch.from_numpy(x) for x in (q, k, v, qt, kt, vt)),
                                 mask=torch.from_numpy(mask), bm=8, bn=8)
    assert torch.all(o[0, 0, 3] == 0) and torch.all(ot[0, 0, 3] == 0) and math.isinf(M[0, 0, 3])


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("L,bm,bn", [(32, 32, 32), (64, 32, 16), (64, 16, 64), (40, 16, 32), (96, 64, 32)])
def test_tiled_matches_dense(mode, L, bm, bn):
    Z, H, D = 2, 2, 16
    q, k, v, qt, kt, vt, go, gt = _inputs(Z, H, L, D, seed=11)
    mask, causal = _masks(Z, H, L)[mode]
    npm = None if mask is None else mask.numpy()
    f = dense.forward(*(x.numpy() for x in (q, k, v, qt, kt, vt)), mask=npm, causal=causal)
    o, ot, M, mu = tiled.forward(q, k, v, qt, kt, vt, mask=mask, causal=causal, bm=bm, bn=bn)
    assert np.abs(o.numpy() - f["O"]).max() < 1e-12
    assert np.abs(ot.numpy() - f["Ot"]).max() < 1e-11
    assert np.abs(M.numpy() - f["M"]).max() < 1e-12
    assert np.abs(mu.numpy() - f["mu"]).max() < 1e-12
    b = dense.backward(*(x.numpy() for x in (q, k, v, qt, kt, vt, go, gt)), mask=npm, causal=causal)
    g = tiled.backward(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask=mask, causal=causal, bm=bm, bn=bn)
    for name in b:
        assert np.abs(g[name].numpy() - b[name]).max() < 1e-11, name
    # plain forward + first-order backward (tangent-free path)
    o1, none_t, M1, none_mu = tiled.forward(q, k, v, mask=mask, causal=causal, bm=bm, bn=bn)
    assert none_t is None and none_mu is None and torch.equal(o1, o)
    g1 = tiled.backward(q, k, v, None, None, None, o1, None, M1, None, go, None, mask=mask,
                        causal=causal, bm=bm, bn=bn)
    b1 = dense.backward(*(x.numpy() for x in (q, k, v)), None, None, None, go.numpy(), None,
                        mask=npm, causal=causal)
    for name in ("dq", "dk", "dv"):
        assert np.abs(g1[name].numpy() - b1[name]).max() < 1e-11, name


def test_config1_cpu_plumbing_fp32():
    """benchmark configuration 1: fp32 B2 H4 L128 D64, seed 0, N(0,1); SDPA route vs tiled restatement."""
    g = torch.Generator().manual_seed(0)
    q, k, v, qt, kt, vt, go, gt = [torch.randn(2, 4, 128, 64, generator=g) for _ in range(8)]
    o_ref, ot_ref, grads = sdpa_jvp.forward_backward(q, k, v, qt, kt, vt, go, gt)
    o, ot, M, mu = tiled.forward(q, k, v, qt, kt, vt)
    gr = tiled.backward(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt)
    assert (o - o_ref).abs().max() < 1e-5
    assert (ot - ot_ref).abs().max() < 1e-4
    for name, ref in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert (gr[name] - ref).abs().max() < 2e-4 * max(1.0, ref.abs().max().item()), name


def _dropout_route(q, k, v, qt, kt, vt, go, gt, W, mask, causal):
    """O, O' and the six gradients with a fixed dropout matrix W, by torch's softmax under ``torch.func.jvp`` and
    ``autograd.grad``: SDPA's definition of dropout (``softmax(S) * keep / (1 - p) @ V``) written out, since the
    library's own dropout draws a pattern nobody else can see."""
    L, Lk = q.shape[-2], k.shape[-2]

    def attn(a, b, c):
        s = a @ b.transpose(-1, -2) * a.shape[-1] ** -0.5
        if causal:
            s = s.masked_fill(~torch.ones(L, Lk, dtype=torch.bool).tril(), -math.inf)
        if mask is not None:
            s = s.masked_fill(~mask, -math.inf) if mask.dtype == torch.bool else s + mask
        return (torch.softmax(s, -1) * W) @ c

    leaves = [t.detach().clone().requires_grad_(True) for t in (q, k, v, qt, kt, vt)]
    o, ot = torch.func.jvp(attn, tuple(leaves[:3]), tuple(leaves[3:]))
    loss = (o * go).sum() + ((ot * gt).sum() if gt is not None else 0.0)
    grads = torch.autograd.grad(loss, leaves, allow_unused=True)
    return o.detach(), ot.detach(), [torch.zeros_like(x) if g is None else g for g, x in zip(grads, leaves)]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("with_gt", [True, False])
def test_dense_with_dropout_matches_the_library_route(mode, with_gt):
    from oracle import dropout

    Z, H, L = 2, 2, 32
    q, k, v, qt, kt, vt, go, gt = _inputs()
    gt = gt if with_gt else None
    mask, causal = _masks(Z, H, L)[mode]
    W = dropout.keep_scale(Z, H, L, L, 0.3, seed=1234567890123)
    assert 0.55 < (W != 0).mean() < 0.85 and np.allclose(W[W != 0], 1 / (1 - np.float32(0.3)))
    o, ot, grads = _dropout_route(q, k, v, qt, kt, vt, go, gt, torch.from_numpy(W), mask, causal)
    npm = None if mask is None else mask.numpy()
    xs = [x.numpy() for x in (q, k, v, qt, kt, vt)]
    f = dense.forward(*xs, mask=npm, causal=causal, keep_scale=W)
    b = dense.backward(*xs, go.numpy(), None if gt is None else gt.numpy(), mask=npm, causal=causal, keep_scale=W)
    assert np.abs(f["O"] - o.numpy()).max() < 1e-12
    assert np.abs(f["Ot"] - ot.numpy()).max() < 1e-12
    for name, ref in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert np.abs(b[name] - ref.numpy()).max() < 1e-11, name


def test_dropout_pattern_properties():
    """What the mathematics fixes about the pattern: the block mix is a bijection of the low index word for a fixed
    seed and the finishing rounds are a bijection of the 32-bit words (so no value is favoured), the kept fraction is
    1 - p, neighbouring entries along rows, columns and diagonals, and neighbouring seeds, are uncorrelated, p = 0
    keeps all."""
    from oracle import dropout

    idx = np.arange(1 << 16, dtype=np.uint64)
    assert len(np.unique(dropout.mix(idx, 99))) == 1 << 16
    assert len(np.unique(dropout.finish(idx * np.uint64(0x10001)))) == 1 << 16
    for p in (0.1, 0.5, 0.9):
        kp = dropout.keep(2, 3, 64, 128, p, seed=7)
        assert abs(kp.mean() - (1 - p)) < 0.01
        assert abs(kp[0, 0].mean(axis=-1) - (1 - p)).max() < 0.2  # every row has its own draw
    a, b = dropout.keep(1, 1, 64, 64, 0.5, 1), dropout.keep(1, 1, 64, 64, 0.5, 2)
    assert 0.4 < (a != b).mean() < 0.6
    # a 512 x 512 head at p = 1/2: the correlation of entries (i, j) and (i + di, j + dj) is noise (sigma 0.002);
    # rows 31 -> 32 cross a block of the pattern, keys step by the other constant
    k = dropout.keep(1, 2, 512, 512, 0.5, seed=2**40 + 3)[0, 1].astype(np.float64) - 0.5
    for di, dj in ((0, 1), (1, 0), (1, 1), (1, -1), (0, 2), (2, 0), (32, 0), (0, 32), (3, 5)):
        x = k[:512 - di, max(0, -dj):512 - max(0, dj)]
        y = k[di:, max(0, dj):512 - max(0, -dj)]
        assert abs((x * y).mean() / 0.25) < 0.01, (di, dj)
    hi = dropout.mix(np.array([5, 5 + (1 << 32)], dtype=np.uint64), 3)
    assert hi[0] != hi[1]  # the high word of the block index takes part
    # heads differ although their rows and keys have the same numbers
    two = dropout.keep(1, 2, 64, 64, 0.5, 11)
    assert 0.4 < (two[0, 0] != two[0, 1]).mean() < 0.6
    assert dropout.keep(1, 1, 4, 4, 0.0, 5).all() and dropout.keep_scale(1, 1, 4, 4, 0.0, 5) is None
    assert dropout.threshold(0.5) == 1 << 31 and dropout.threshold(1e-12) == 1

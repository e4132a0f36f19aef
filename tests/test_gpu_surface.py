"""GPU tests of the Python surface (``attention``, ``JVPAttn.fwd_dual``) and of the benchmark
configurations at their full sizes.

Small shapes are compared with the fp64 oracle directly.  At full size one (z, h) slab is compared
with the oracle and the rest is covered by properties that do not depend on size: O' is linear in
the tangents, a V'-only tangent gives O' = softmax(S) V', key order does not matter without a
mask, causal rows do not see later keys (bit-exact against a run on the truncated sequence), and
the different backward modes agree where the mathematics says they must.
"""
from functools import partial

import numpy as np
import pytest
import torch
import torch.autograd.forward_ad as fwAD

from oracle import dense

pytestmark = pytest.mark.gpu


def _rel(got, ref):
    got = got.detach().double().cpu().numpy() if isinstance(got, torch.Tensor) else got
    ref = ref.detach().double().cpu().numpy() if isinstance(ref, torch.Tensor) else ref
    assert np.isfinite(got).all()
    return np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30)


def _randn(shape, dtype, seed, std=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * std).to(dtype)


@pytest.mark.parametrize("dt,tol", [(torch.float32, None), (torch.bfloat16, 2e-2), (torch.float16, 2e-2)])
@pytest.mark.parametrize("mode", ["none", "causal", "keypad", "bias"])
def test_surface_three_way_and_gradients(dt, tol, mode):
    """fwAD route, torch.func.jvp route and autograd, all through the public functions."""
    from jvp_flash_attention_amd import JVPAttn

    Z, H, L, D = 2, 2, 128, 64
    q, k, v, qt, kt, vt, go, gt = [_randn((Z, H, L, D), dt, 10 + i) for i in range(8)]
    mask, causal = None, mode == "causal"
    if mode == "keypad":
        lens = torch.tensor([80, 128], device="cuda")
        mask = (torch.arange(L, device="cuda")[None, :] < lens[:, None]).view(Z, 1, 1, L)
    if mode == "bias":
        mask = _randn((Z, H, L, L), dt, 99)
    npm = None if mask is None else (mask.cpu().numpy() if mask.dtype == torch.bool else mask.double().cpu().numpy())
    f64 = [x.double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    ref = dense.forward(*f64[:6], mask=npm, causal=causal)
    rb = dense.backward(*f64, mask=npm, causal=causal)
    fn = partial(JVPAttn.fwd_dual, attn_mask=mask, causal=causal)

    leaves = [x.clone().requires_grad_() for x in (q, k, v, qt, kt, vt)]
    with fwAD.dual_level():
        out = fn(*(fwAD.make_dual(p, t) for p, t in zip(leaves[:3], leaves[3:])))
        o1, ot1 = fwAD.unpack_dual(out)
        loss = (o1.float() * go.float()).sum() + (ot1.float() * gt.float()).sum()
        grads = torch.autograd.grad(loss, leaves)
    o2, ot2 = torch.func.jvp(fn, (q, k, v), (qt, kt, vt))
    assert torch.equal(o1, o2) and torch.equal(ot1, ot2)

    def check(name, got, want):
        if dt == torch.float32:
            err = np.abs(got.detach().double().cpu().numpy() - want).max()
            assert err <= 1e-4, f"{name}: {err:.3e}"
        else:
            assert _rel(got, want) <= tol, f"{name}: {_rel(got, want):.3e}"

    check("O", o1, ref["O"])
    check("O'", ot1, ref["Ot"])
    for n, g in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        check(n, g, rb[n])


def test_surface_block_diagonal_mask_uses_tile_lists():
    """A packed-sequence mask through the public functions: the host scans it into tile lists once, and
    forward and backward reuse them (forward-mode tangent and all six gradients against the oracle)."""
    from jvp_flash_attention_amd import JVPAttn, attention

    Z, H, L, D = 1, 2, 768, 64
    dt = torch.bfloat16
    q, k, v, qt, kt, vt, go, gt = [_randn((Z, H, L, D), dt, 40 + i) for i in range(8)]
    seg = torch.bucketize(torch.arange(L, device="cuda"), torch.tensor([200, 450], device="cuda"), right=True)
    mask = (seg[:, None] == seg[None, :]).view(1, 1, L, L)
    f64 = [x.double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    ref = dense.forward(*f64[:6], mask=mask.cpu().numpy(), causal=False)
    rb = dense.backward(*f64, mask=mask.cpu().numpy(), causal=False)
    leaves = [x.clone().requires_grad_() for x in (q, k, v, qt, kt, vt)]
    with fwAD.dual_level():
        out = JVPAttn.fwd_dual(*(fwAD.make_dual(p, t) for p, t in zip(leaves[:3], leaves[3:])), attn_mask=mask)
        o, ot = fwAD.unpack_dual(out)
        loss = (o.float() * go.float()).sum() + (ot.float() * gt.float()).sum()
        grads = torch.autograd.grad(loss, leaves)
    tiles = mask._jvpfa_tiles
    assert tiles[1] is not None and tiles[2] is not None
    nt = L // 64
    first_block = tiles[1].view(-1, nt + 1)[0].tolist()
    assert first_block[:1 + first_block[0]] == [4, 0, 1, 2, 3]  # rows 0..127 lie in segment 0: keys below 200, tiles 0..3
    assert _rel(o, ref["O"]) <= 2e-2 and _rel(ot, ref["Ot"]) <= 2e-2
    for n, g in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert _rel(g, rb[n]) <= 2e-2, n
    o_plain = attention(q, k, v, attn_mask=mask)
    assert _rel(o_plain, ref["O"]) <= 2e-2


@pytest.mark.parametrize("causal", [False, True])
def test_forward_and_backward_replay_from_a_hip_graph(causal):
    """The entry points allocate nothing and launch on the stream they are given, so a forward +
    backward can be captured once and replayed: three replays with fresh inputs copied into the
    captured buffers, each checked against an eager run on the same inputs."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, L, D = 2, 4, 256, 64
    dt = torch.bfloat16
    scale = D**-0.5
    static = [_randn((Z, H, L, D), dt, 60 + i) for i in range(8)]

    def step(x):
        o, ot, M, mu = be.fwd(*x[:6], None, _lib.MASK_NONE, causal, scale)
        grads = be.bwd(*x[:6], o, ot, M, mu, x[6], x[7], None, _lib.MASK_NONE, causal, scale, want_tangent_grads=True)
        return [o, ot, *grads]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up off the default stream, as graph capture requires
        step(static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(static)
    for rep in range(3):
        fresh = [_randn((Z, H, L, D), dt, 100 + 10 * rep + i) for i in range(8)]
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        eager = step(fresh)
        torch.cuda.synchronize()
        for a, b in zip(captured, eager):
            assert torch.equal(a, b), f"replay {rep}"


def test_surface_head_dim_16_eager_and_compiled():
    """A head dim of 16, which the reference admits, through the public functions: the tangent from
    ``torch.func.jvp``, gradients from autograd, and the same call under ``torch.compile``."""
    from jvp_flash_attention_amd import JVPAttn, attention

    Z, H, L, D = 2, 3, 96, 16
    q, k, v, qt, kt, vt, go, gt = [_randn((Z, H, L, D), torch.bfloat16, 40 + i) for i in range(8)]
    f64 = [x.double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    ref = dense.forward(*f64[:6], mask=None, causal=True)
    rb = dense.backward(*f64, mask=None, causal=True)
    leaves = [x.clone().requires_grad_() for x in (q, k, v, qt, kt, vt)]
    with fwAD.dual_level():
        out = JVPAttn.fwd_dual(*(fwAD.make_dual(p, t) for p, t in zip(leaves[:3], leaves[3:])), causal=True)
        o, ot = fwAD.unpack_dual(out)
        assert o.shape == (Z, H, L, D) and ot.shape == (Z, H, L, D)
        grads = torch.autograd.grad((o.float() * go.float()).sum() + (ot.float() * gt.float()).sum(), leaves)
    assert _rel(o, ref["O"]) <= 2e-2 and _rel(ot, ref["Ot"]) <= 2e-2
    for n, g in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert g.shape == (Z, H, L, D) and _rel(g, rb[n]) <= 2e-2, n

    def f(q, k, v):
        return (attention(q, k, v, causal=True).float() * go.float()).sum()

    pl = [x.clone().requires_grad_() for x in (q, k, v)]
    eager = f(*pl)
    ge = torch.autograd.grad(eager, pl)
    torch._dynamo.reset()
    compiled = torch.compile(f, backend="aot_eager", fullgraph=True)(*pl)
    gc = torch.autograd.grad(compiled, pl)
    assert torch.equal(eager, compiled)
    for a, b in zip(ge, gc):
        assert torch.equal(a, b)


@pytest.mark.parametrize("masked", [False, True])
def test_plain_attention_inside_torch_compile_without_graph_breaks(masked):
    """``torch.compile(fullgraph=True)`` over a function that calls ``attention``: the kernels enter
    the graph as the operators ``jvpfa::fwd`` / ``jvpfa::bwd``; output and gradients equal the eager
    ones bit for bit (the ``aot_eager`` backend runs the traced graph with the same kernels)."""
    from jvp_flash_attention_amd import attention

    Z, H, L, D = 2, 4, 256, 64
    q, k, v = [_randn((Z, H, L, D), torch.bfloat16, 70 + i).requires_grad_() for i in range(3)]
    kw = dict(causal=True)
    if masked:
        keep = torch.rand(Z, 1, L, L, device="cuda", generator=torch.Generator(device="cuda").manual_seed(5)) > 0.3
        keep[..., 0] = True
        kw = dict(attn_mask=keep)

    def f(q, k, v):
        return (attention(q * 1.0, k, v, **kw) * 2.0).float().sum()

    ref = f(q, k, v)
    gref = torch.autograd.grad(ref, (q, k, v))
    torch._dynamo.reset()
    out = torch.compile(f, backend="aot_eager", fullgraph=True)(q, k, v)
    g = torch.autograd.grad(out, (q, k, v))
    assert torch.equal(out, ref)
    for a, b in zip(g, gref):
        assert torch.equal(a, b)


@pytest.mark.parametrize("masked", [False, True])
def test_dropout_inside_torch_compile_without_graph_breaks(masked):
    """``attention`` with dropout under ``torch.compile(fullgraph=True)``: the operators ``jvpfa::fwd_drop`` /
    ``jvpfa::bwd_drop`` draw the seed from torch's CPU generator themselves, as the eager call does, so after the
    same ``torch.manual_seed`` output and gradients equal the eager ones bit for bit; a second compiled call
    draws another pattern."""
    from jvp_flash_attention_amd import attention

    Z, H, L, D = 2, 4, 256, 64
    q, k, v = [_randn((Z, H, L, D), torch.bfloat16, 75 + i).requires_grad_() for i in range(3)]
    kw = dict(causal=True, dropout_p=0.25)
    if masked:
        keep = torch.rand(Z, 1, L, L, device="cuda", generator=torch.Generator(device="cuda").manual_seed(6)) > 0.3
        keep[..., 0] = True
        kw = dict(attn_mask=keep, dropout_p=0.25)

    def f(q, k, v):
        return (attention(q * 1.0, k, v, **kw) * 2.0).float().sum()

    torch.manual_seed(11)
    ref = f(q, k, v)
    gref = torch.autograd.grad(ref, (q, k, v))
    torch._dynamo.reset()
    compiled = torch.compile(f, backend="aot_eager", fullgraph=True)
    torch.manual_seed(11)
    out = compiled(q, k, v)
    g = torch.autograd.grad(out, (q, k, v))
    assert torch.equal(out, ref)
    for a, b in zip(g, gref):
        assert torch.equal(a, b)
    again = compiled(q, k, v)  # the generator has moved on: another pattern
    assert not torch.equal(again, ref)


@pytest.mark.parametrize("dropout_p", [0.0, 0.3])
def test_forward_mode_inside_torch_compile_without_graph_breaks(dropout_p):
    """A forward-mode level opened inside a function compiled with ``fullgraph=True``: ``fwd_dual`` takes the
    tangents off its inputs, runs the dual kernels as ``jvpfa::fwd`` and puts O' back on O; O, O' and the
    gradients of a loss on both (through ``jvpfa::bwd``) equal the eager ones bit for bit."""
    from jvp_flash_attention_amd import JVPAttn

    Z, H, L, D = 2, 2, 192, 64
    q, k, v = [_randn((Z, H, L, D), torch.bfloat16, 85 + i).requires_grad_() for i in range(3)]
    qt, kt, vt = [_randn((Z, H, L, D), torch.bfloat16, 88 + i) for i in range(3)]

    def g(q, k, v, qt, kt, vt):
        with fwAD.dual_level():
            out = JVPAttn.fwd_dual(fwAD.make_dual(q * 1.0, qt), fwAD.make_dual(k, kt), fwAD.make_dual(v, vt), causal=True,
                                   dropout_p=dropout_p)
            o, ot = fwAD.unpack_dual(out * 2.0)
            return o.float().sum() + (ot.float() ** 2).sum(), o.detach().clone(), ot.detach().clone()

    torch.manual_seed(3)
    loss1, o1, ot1 = g(q, k, v, qt, kt, vt)
    g1 = torch.autograd.grad(loss1, (q, k, v))
    torch._dynamo.reset()
    torch.manual_seed(3)
    loss2, o2, ot2 = torch.compile(g, backend="aot_eager", fullgraph=True)(q, k, v, qt, kt, vt)
    g2 = torch.autograd.grad(loss2, (q, k, v))
    assert torch.equal(o1, o2) and torch.equal(ot1, ot2) and torch.equal(loss1, loss2)
    for a, b in zip(g1, g2):
        assert torch.equal(a, b)


def test_dual_tensors_inside_torch_compile_keep_their_tangent():
    """Forward-mode AD inside a compiled function (here with the ``eager`` backend, which runs the traced graph
    as it stands): O' is what the eager call gives, not silently dropped."""
    from jvp_flash_attention_amd import JVPAttn

    Z, H, L, D = 1, 2, 128, 64
    q, k, v, qt, kt, vt = [_randn((Z, H, L, D), torch.bfloat16, 80 + i) for i in range(6)]

    def g(q, k, v, qt, kt, vt):
        with fwAD.dual_level():
            out = JVPAttn.fwd_dual(fwAD.make_dual(q, qt), fwAD.make_dual(k, kt), fwAD.make_dual(v, vt), causal=True)
            o, ot = fwAD.unpack_dual(out)
            return o.clone(), ot.clone()

    o1, ot1 = g(q, k, v, qt, kt, vt)
    torch._dynamo.reset()
    o2, ot2 = torch.compile(g, backend="eager")(q, k, v, qt, kt, vt)
    assert torch.equal(o1, o2) and torch.equal(ot1, ot2)


def test_surface_grouped_heads_and_cross_attention():
    """k, v with fewer heads and another length than q through the public functions: forward-mode
    tangent, and gradients of a loss on O and O' with k's shape for dk, dv (summed over each group)."""
    from jvp_flash_attention_amd import JVPAttn, attention

    Z, H, Hk, Lq, Lk, D = 2, 4, 2, 100, 150, 64
    dt = torch.bfloat16
    q, qt, go, gt = [_randn((Z, H, Lq, D), dt, 90 + i) for i in range(4)]
    k, v, kt, vt = [_randn((Z, Hk, Lk, D), dt, 95 + i) for i in range(4)]
    mask = torch.rand(Z, 1, Lq, Lk, device="cuda", generator=torch.Generator(device="cuda").manual_seed(3)) > 0.4
    mask[..., 0] = True
    f64 = [x.double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    ref = dense.forward(*f64[:6], mask=mask.cpu().numpy())
    rb = dense.backward(*f64, mask=mask.cpu().numpy())
    leaves = [x.clone().requires_grad_() for x in (q, k, v, qt, kt, vt)]
    with fwAD.dual_level():
        out = JVPAttn.fwd_dual(*(fwAD.make_dual(p, t) for p, t in zip(leaves[:3], leaves[3:])), attn_mask=mask)
        o, ot = fwAD.unpack_dual(out)
        loss = (o.float() * go.float()).sum() + (ot.float() * gt.float()).sum()
        grads = torch.autograd.grad(loss, leaves)
    assert _rel(o, ref["O"]) <= 2e-2 and _rel(ot, ref["Ot"]) <= 2e-2
    for n, g in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert tuple(g.shape) == rb[n].shape and _rel(g, rb[n]) <= 2e-2, n
    ql, kl, vl = [x.clone().requires_grad_() for x in (q, k, v)]
    o_plain = attention(ql, kl, vl, causal=True)
    g1 = torch.autograd.grad((o_plain.float() * go.float()).sum(), (ql, kl, vl))
    refc = dense.forward(*f64[:3], causal=True)
    rbc = dense.backward(*f64[:3], None, None, None, f64[6], None, causal=True)
    assert _rel(o_plain, refc["O"]) <= 2e-2
    for n, g in zip(("dq", "dk", "dv"), g1):
        assert _rel(g, rbc[n]) <= 2e-2, n


def test_plain_attention_autograd_and_apply_tuple():
    from jvp_flash_attention_amd import JVPAttn, attention

    Z, H, L, D = 1, 3, 96, 128
    q, k, v, go = [_randn((Z, H, L, D), torch.bfloat16, 20 + i) for i in range(4)]
    f64 = [x.double().cpu().numpy() for x in (q, k, v, go)]
    qq, kk, vv = [x.clone().requires_grad_() for x in (q, k, v)]
    o = attention(qq, kk, vv, causal=True)
    (o.float() * go.float()).sum().backward()
    ref = dense.forward(*f64[:3], causal=True)
    rb = dense.backward(*f64[:3], None, None, None, f64[3], None, causal=True)
    assert _rel(o, ref["O"]) <= 2e-2
    for n, g in (("dq", qq.grad), ("dk", kk.grad), ("dv", vv.grad)):
        assert _rel(g, rb[n]) <= 2e-2, n
    o2, ctx = JVPAttn.apply(q, k, v, None, None, None, None, 0.0, True, None, True, True)
    assert torch.equal(o2, o.detach()) and ctx.o_t is None and ctx.M.shape == (Z, H, L)
    # log2-domain log-sum-exp
    assert np.abs(ctx.M.double().cpu().numpy() - ref["M"]).max() < 2e-2


def test_config2_dense_bf16_full_size_properties():
    """benchmark configuration 2: bf16 B4 H16 L2048 D64, tangents ~ N(0, 0.1^2), no mask."""
    from jvp_flash_attention_amd import _lib, attention

    be = _lib.backend()
    Z, H, L, D = 4, 16, 2048, 64
    dt = torch.bfloat16
    q, k, v = [_randn((Z, H, L, D), dt, 30 + i) for i in range(3)]
    qt, kt, vt = [_randn((Z, H, L, D), dt, 40 + i, std=0.1) for i in range(3)]
    go, gt = [_randn((Z, H, L, D), dt, 50 + i) for i in range(2)]
    scale = D**-0.5
    o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, 0, False, scale)
    # one slab against the oracle
    f64 = [x[1, 5:6][None].double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    ref = dense.forward(*f64[:6])
    assert _rel(o[1, 5], ref["O"][0, 0]) <= 2e-2 and _rel(ot[1, 5], ref["Ot"][0, 0]) <= 2e-2
    dq, dk, dv, dqt, dkt, dvt = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, 0, False, scale,
                                       want_tangent_grads=True)
    rb = dense.backward(*f64)
    for n, g in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), (dq, dk, dv, dqt, dkt, dvt)):
        assert _rel(g[1, 5], rb[n][0, 0]) <= 2e-2, n
    # V'-only tangent: O' = softmax(S) V', the plain attention output with V := V'
    zero = torch.zeros_like(q)
    _, ot_v, _, _ = be.fwd(q, k, v, zero, zero, vt, None, 0, False, scale)
    assert _rel(ot_v, attention(q, k, vt)) <= 1e-2
    # linearity in the tangents
    _, ot_q, _, _ = be.fwd(q, k, v, qt, zero, zero, None, 0, False, scale)
    _, ot_k, _, _ = be.fwd(q, k, v, zero, kt, zero, None, 0, False, scale)
    assert _rel(ot_q.float() + ot_k.float() + ot_v.float(), ot.float()) <= 2e-2
    # without a mask the order of the keys does not matter
    perm = torch.randperm(L, device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    o_p, ot_p, _, _ = be.fwd(q, k[:, :, perm].contiguous(), v[:, :, perm].contiguous(), qt,
                             kt[:, :, perm].contiguous(), vt[:, :, perm].contiguous(), None, 0, False, scale)
    assert _rel(o_p, o) <= 1e-2 and _rel(ot_p, ot) <= 2e-2
    # dV' = P^T gT in tangent mode equals dV = P^T gO of the first-order backward when gO := gT
    g1 = be.bwd(q, k, v, None, None, None, o, None, M, None, gt, None, None, 0, False, scale)
    assert _rel(dvt, g1[2]) <= 1e-2


@pytest.mark.parametrize("D,causal", [(32, False), (32, True), (256, False), (256, True)])
def test_other_head_dims_at_benchmark_size(D, causal):
    """bf16 B4 H16 L2048 with D = 32 and D = 256: a head computed inside the whole batch (more workgroups
    than compute units, heads spread over the dies, for D = 256 two workgroups per query block) equals the
    same head computed alone, bit for bit, forward and backward; one slab is checked against the oracle."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, L = 4, 16, 2048
    dt, scale = torch.bfloat16, D**-0.5
    q, k, v, go, gt = [_randn((Z, H, L, D), dt, 80 + i) for i in range(5)]
    qt, kt, vt = [_randn((Z, H, L, D), dt, 90 + i, std=0.5) for i in range(3)]
    o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, 0, causal, scale)
    grads = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, 0, causal, scale, want_tangent_grads=True)
    for z, h in ((0, 0), (3, 15), (2, 9)):
        one = [x[z:z + 1, h:h + 1].contiguous() for x in (q, k, v, qt, kt, vt, go, gt)]
        o1, ot1, M1, mu1 = be.fwd(*one[:6], None, 0, causal, scale)
        assert torch.equal(o[z, h], o1[0, 0]) and torch.equal(ot[z, h], ot1[0, 0])
        assert torch.equal(M[z, h], M1[0, 0]) and torch.equal(mu[z, h], mu1[0, 0])
        g1 = be.bwd(*one[:6], o1, ot1, M1, mu1, one[6], one[7], None, 0, causal, scale, want_tangent_grads=True)
        for n, a_, b_ in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads, g1):
            assert torch.equal(a_[z, h], b_[0, 0]), n
    z, h = 1, 5
    f64 = [x[z, h:h + 1][None].double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    ref = dense.forward(*f64[:6], causal=causal)
    rb = dense.backward(*f64, causal=causal)
    assert _rel(o[z, h], ref["O"][0, 0]) <= 2e-2 and _rel(ot[z, h], ref["Ot"][0, 0]) <= 2e-2
    for n, g in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert _rel(g[z, h], rb[n][0, 0]) <= 2e-2, n


@pytest.mark.parametrize("D", [32, 64, 256])
def test_long_causal_sequences_prefix_properties(D):
    """bf16 B1 H4 L16384 causal: causal rows never see later keys, so the first half of the outputs equals a
    run on the truncated sequence bit for bit, and with the incoming gradients of the second half set
    to zero the gradients of the first half equal those of the truncated run while dk, dv of the second
    half are exactly zero."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, L = 1, 4, 16384
    dt, scale = torch.bfloat16, D**-0.5
    q, k, v, qt, kt, vt, go, gt = [_randn((Z, H, L, D), dt, 70 + i) for i in range(8)]
    o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, 0, True, scale)
    assert all(torch.isfinite(t).all() for t in (o, ot, M, mu))
    h = L // 2
    cut = [x[:, :, :h].contiguous() for x in (q, k, v, qt, kt, vt)]
    o2, ot2, M2, mu2 = be.fwd(*cut, None, 0, True, scale)
    assert torch.equal(o[:, :, :h], o2) and torch.equal(ot[:, :, :h], ot2) and torch.equal(M[:, :, :h], M2)
    go[:, :, h:] = 0
    gt[:, :, h:] = 0
    full = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, 0, True, scale)
    part = be.bwd(*cut, o2, ot2, M2, mu2, go[:, :, :h].contiguous(), gt[:, :, :h].contiguous(), None, 0, True, scale)
    for n, a_, b_ in zip(("dq", "dk", "dv"), full[:3], part[:3]):
        assert torch.equal(a_[:, :, :h], b_), n
    assert full[1][:, :, h:].abs().max().item() == 0.0 and full[2][:, :, h:].abs().max().item() == 0.0


def test_config3_causal_long_full_size_properties():
    """benchmark configuration 3: fp16 B2 H32 L4096 D128 causal, and the headline bf16 B4 H16 L4096 D128."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    for dt, (Z, H) in ((torch.float16, (2, 32)), (torch.bfloat16, (4, 16))):
        L, D = 4096, 128
        scale = D**-0.5
        q, k, v, qt, kt, vt, go, gt = [_randn((Z, H, L, D), dt, 60 + i) for i in range(8)]
        o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, 0, True, scale)
        assert torch.isfinite(o).all() and torch.isfinite(ot).all()
        # causal rows never see later keys: the first half equals a run on the truncated sequence, bit for bit
        h = L // 2
        cut = [x[:, :, :h].contiguous() for x in (q, k, v, qt, kt, vt)]
        o_h, ot_h, M_h, mu_h = be.fwd(*cut, None, 0, True, scale)
        assert torch.equal(o[:, :, :h], o_h) and torch.equal(ot[:, :, :h], ot_h) and torch.equal(M[:, :, :h], M_h)
        # one slab against the oracle (forward and the tangent-path backward)
        z, hh = Z - 1, 3
        f64 = [x[z, hh:hh + 1][None].double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
        ref = dense.forward(*f64[:6], causal=True)
        assert _rel(o[z, hh], ref["O"][0, 0]) <= 2e-2 and _rel(ot[z, hh], ref["Ot"][0, 0]) <= 2e-2
        dq, dk, dv, *_ = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, 0, True, scale)
        rb = dense.backward(*f64, causal=True)
        for n, g in zip(("dq", "dk", "dv"), (dq, dk, dv)):
            assert _rel(g[z, hh], rb[n][0, 0]) <= 2e-2, n
        # gradients are causal too: dk, dv of the second half do not depend on queries of the first half
        del o_h, ot_h, dq, dk, dv
        torch.cuda.empty_cache()


def test_headline_shape_non_causal_full_size_against_the_oracle():
    """The benchmarked launch itself: bf16 B4 H16 L4096 D128, no mask, not causal (64 interior tiles per
    query block).  Two (z, h) slabs of O, O' and of all six gradients against the oracle, tangents ~ N(0,1)."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, L, D = 4, 16, 4096, 128
    dt, scale = torch.bfloat16, D**-0.5
    q, k, v, qt, kt, vt, go, gt = [_randn((Z, H, L, D), dt, 160 + i) for i in range(8)]
    o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, 0, False, scale)
    grads = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, 0, False, scale, want_tangent_grads=True)
    for z, h in ((0, 0), (3, 13)):
        print(f"case headline slab z{z} h{h}", flush=True)
        f64 = [x[z, h:h + 1][None].double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
        ref = dense.forward(*f64[:6], scale=scale)
        assert _rel(o[z, h], ref["O"][0, 0]) <= 2e-2 and _rel(ot[z, h], ref["Ot"][0, 0]) <= 2e-2
        assert np.abs(M[z, h].double().cpu().numpy() - ref["M"][0, 0]).max() <= 2e-2
        assert np.abs(mu[z, h].double().cpu().numpy() - ref["mu"][0, 0]).max() <= 2e-2
        rb = dense.backward(*f64, scale=scale)
        for n, g in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
            assert _rel(g[z, h], rb[n][0, 0]) <= 2e-2, n
        del ref, rb


@pytest.mark.parametrize("L", [1024, 4096, 16384, 32768])
def test_config5_hvp_sweep_at_every_length(L):
    """benchmark configuration 5: bf16 B1 H16 D128 causal, tangents ~ N(0,1), the gradient of sum(O' * gO')
    with respect to q, k, v (no gO), at each length of the sweep.

    * L <= 4096: one whole head of O, O', dq, dk, dv against the oracle.
    * every L: the tail, where 32-bit offsets would wrap first.  Row i of O, O', dq depends on q[i], q'[i],
      gO'[i] and the keys up to i only, so the last 64 queries of a head over all L keys are an exact
      oracle problem of their own (a boolean mask states the causal limit of each row); dk, dv of the last
      64 keys receive contributions from those 64 queries only, so the same problem gives them too.
    * every L: causal rows never see later keys, so the first half equals a run on the truncated sequence,
      bit for bit, forward and (with the incoming gradient of the second half set to zero) backward."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, D = 1, 16, 128
    dt, scale = torch.bfloat16, D**-0.5
    q, k, v, qt, kt, vt, gt = [_randn((Z, H, L, D), dt, 170 + i) for i in range(7)]
    print(f"case config5 L{L}", flush=True)
    o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, 0, True, scale)
    dq, dk, dv, *_ = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, None, gt, None, 0, True, scale)
    assert all(torch.isfinite(t).all() for t in (o, ot, M, mu, dq, dk, dv))
    np64 = lambda x: x.double().cpu().numpy()  # noqa: E731
    if L <= 4096:
        h = 11
        f64 = [np64(x[:, h:h + 1]) for x in (q, k, v, qt, kt, vt)]
        g64 = np64(gt[:, h:h + 1])
        ref = dense.forward(*f64, causal=True, scale=scale)
        assert _rel(o[0, h], ref["O"][0, 0]) <= 2e-2 and _rel(ot[0, h], ref["Ot"][0, 0]) <= 2e-2
        rb = dense.backward(*f64, np.zeros_like(g64), g64, causal=True, scale=scale)
        for n, g in zip(("dq", "dk", "dv"), (dq, dk, dv)):
            assert _rel(g[0, h], rb[n][0, 0]) <= 2e-2, n
        del ref, rb
    # the tail: last T queries of two heads over all keys
    T = 64
    for h in (0, H - 1):
        rows = slice(L - T, L)
        f64 = [np64(q[:, h:h + 1, rows]), np64(k[:, h:h + 1]), np64(v[:, h:h + 1]),
               np64(qt[:, h:h + 1, rows]), np64(kt[:, h:h + 1]), np64(vt[:, h:h + 1])]
        g64 = np64(gt[:, h:h + 1, rows])
        keep = (np.arange(L)[None, :] <= (L - T + np.arange(T))[:, None])[None, None]
        ref = dense.forward(*f64, mask=keep, scale=scale)
        assert _rel(o[0, h, rows], ref["O"][0, 0]) <= 2e-2 and _rel(ot[0, h, rows], ref["Ot"][0, 0]) <= 2e-2
        assert np.abs(np64(M[0, h, rows]) - ref["M"][0, 0]).max() <= 2e-2
        rb = dense.backward(*f64, np.zeros_like(g64), g64, mask=keep, scale=scale)
        assert _rel(dq[0, h, rows], rb["dq"][0, 0]) <= 2e-2
        assert _rel(dk[0, h, rows], rb["dk"][0, 0, rows]) <= 2e-2 and _rel(dv[0, h, rows], rb["dv"][0, 0, rows]) <= 2e-2
    # the prefix (one workgroup per query block in both runs: a launch this small would otherwise split the key
    # tiles of a block over several workgroups, differently for the two lengths, and agree to rounding only)
    half = L // 2
    cut = [x[:, :, :half].contiguous() for x in (q, k, v, qt, kt, vt)]
    _lib.set_split(False)
    try:
        o1, ot1, M1, mu1 = be.fwd(q, k, v, qt, kt, vt, None, 0, True, scale)
        o2, ot2, M2, mu2 = be.fwd(*cut, None, 0, True, scale)
    finally:
        _lib.set_split(True)
    assert torch.equal(o1[:, :, :half], o2) and torch.equal(ot1[:, :, :half], ot2)
    assert torch.equal(M1[:, :, :half], M2) and torch.equal(mu1[:, :, :half], mu2)
    assert _rel(o, o1) <= 8e-3 and _rel(ot, ot1) <= 8e-3 and (M - M1).abs().max().item() <= 1e-5  # split or not: one ulp
    gt[:, :, half:] = 0
    full = be.bwd(q, k, v, qt, kt, vt, o1, ot1, M1, mu1, None, gt, None, 0, True, scale)
    part = be.bwd(*cut, o2, ot2, M2, mu2, None, gt[:, :, :half].contiguous(), None, 0, True, scale)
    for n, a_, b_ in zip(("dq", "dk", "dv"), full[:3], part[:3]):
        assert torch.equal(a_[:, :, :half], b_), n
    assert full[1][:, :, half:].abs().max().item() == 0.0 and full[2][:, :, half:].abs().max().item() == 0.0


def test_config4_mask_modes_fp32_full_size():
    """benchmark configuration 4: fp32 B4 H8 L1024 D64; (a) key padding [B,1,1,L], (b) additive bias [B,H,L,L]."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, L, D = 4, 8, 1024, 64
    dt = torch.float32
    scale = D**-0.5
    q, k, v, qt, kt, vt, go, gt = [_randn((Z, H, L, D), dt, 70 + i) for i in range(8)]
    g = torch.Generator().manual_seed(7)
    lens = torch.randint(L // 2, L + 1, (Z,), generator=g)
    keypad = (torch.arange(L)[None, :] < lens[:, None]).view(Z, 1, 1, L).cuda()
    bias = _randn((Z, H, L, L), dt, 79)
    for mask, kind in ((keypad, _lib.MASK_BOOL), (bias, _lib.MASK_ADD)):
        o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, mask, kind, False, scale)
        grads = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, kind, False, scale, want_tangent_grads=True)
        for z, h in ((0, 0), (3, 7)):
            f64 = [x[z, h:h + 1][None].double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
            m = mask[z:z + 1, 0:1] if kind == _lib.MASK_BOOL else mask[z:z + 1, h:h + 1]
            npm = m.cpu().numpy() if kind == _lib.MASK_BOOL else m.double().cpu().numpy()
            ref = dense.forward(*f64[:6], mask=npm)
            rb = dense.backward(*f64, mask=npm)
            assert np.abs(o[z, h].double().cpu().numpy() - ref["O"][0, 0]).max() <= 1e-4
            assert np.abs(ot[z, h].double().cpu().numpy() - ref["Ot"][0, 0]).max() <= 1e-4
            for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
                assert np.abs(t[z, h].double().cpu().numpy() - rb[n][0, 0]).max() <= 1e-4, n
        if kind == _lib.MASK_BOOL:
            # masked keys receive no gradient and contribute nothing
            for zz in range(Z):
                n = int(lens[zz])
                if n < L:
                    assert torch.all(grads[1][zz, :, n:] == 0) and torch.all(grads[2][zz, :, n:] == 0)


def test_config5_hvp_memory_is_linear_in_sequence_length():
    """benchmark configuration 5 at two lengths: peak memory of fwd_dual + backward grows like L, not L^2."""
    from jvp_flash_attention_amd import JVPAttn

    def peak(L):
        torch.cuda.empty_cache()
        Z, H, D = 1, 16, 128
        q, k, v, qt, kt, vt, gt = [_randn((Z, H, L, D), torch.bfloat16, 80 + i) for i in range(7)]
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        leaves = [x.requires_grad_() for x in (q, k, v)]
        _, ot = torch.func.jvp(partial(JVPAttn.fwd_dual, causal=True), tuple(leaves), (qt, kt, vt))
        grads = torch.autograd.grad((ot.float() * gt.float()).sum(), leaves)
        assert all(torch.isfinite(g).all() for g in grads)
        return torch.cuda.max_memory_allocated() - base

    p1, p2 = peak(4096), peak(16384)
    assert p2 <= 4.5 * p1, (p1, p2)  # 4x the length: ~4x the memory (16x if anything were O(L^2))


@pytest.mark.parametrize("dtype", ["bfloat16", "float16", "float32"])
def test_validation_report_passes_every_case(dtype, tmp_path, capsys):
    """``python -m jvp_flash_attention_amd.validate`` (the counterpart of the reference's test script): every case of
    sequence length x mask type x causal flag within the reference's own tolerances against math SDPA, in the
    three-way comparison (SDPA / fwAD / torch.func.jvp), with its tables and its JSON file written."""
    import argparse
    import json

    from jvp_flash_attention_amd import validate

    out = tmp_path / "report.json"
    args = argparse.Namespace(dtype=dtype, bsz=2, model_dim=768, head_dim=64, seq_lengths=[32, 128, 512], no_masks=False,
                              no_timing=True, json=str(out))
    rows = validate.run(args)
    assert len(rows) == 12  # 3 lengths x (no mask, causal, boolean mask, additive mask)
    assert all(r["ok"] for r in rows), [(r["L"], r["mask"], r["causal"]) for r in rows if not r["ok"]]
    text = capsys.readouterr().out
    assert "BENCHMARK SUMMARY" in text and "MASK TYPE PERFORMANCE COMPARISON" in text and "accuracy: 12/12 passed" in text
    rep = json.loads(out.read_text())
    assert rep["passed"] == rep["cases"] == 12 and rep["dtype"] == dtype and len(rep["rows"]) == 12
    assert rep["max_tangent_error"] < validate.TOLERANCE[dtype]

"""GPU parity with dropout on the attention probabilities.

The reference has no working dropout (``jvp_flash_attention/jvp_attention.py:2356-2357`` raises for
``dropout_p > 0``; its generator at ``:94-122`` is dead code), so there is no reference output to match: the
semantics are SDPA's (kept probabilities scaled by 1 / (1 - p), the same pattern for O and O').  The pattern is
this library's own, so the tests first read it back from the library (``jvpfa_dropout_keep``), check it bit for bit
against the numpy restatement, and then hold the kernels to the dense fp64 closed form with exactly that pattern,
at the tolerances of the other parity tests (fp32 max-abs 1e-4; bf16 / fp16 relative 2e-2).
"""
import numpy as np
import pytest
import torch

from oracle import dense, dropout
from tests.test_gpu_parity import DTYPES, _make, _mask, _tol_check

pytestmark = pytest.mark.gpu


def _case(Z, H, L, D, dtype, mode, p, seed, Hk=None, Lk=None, plain=False):
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Hk, Lk = Hk or H, Lk or L
    q, k, v, qt, kt, vt, go, gt = _make(Z, H, L, D, dtype, seed=3)
    if (Hk, Lk) != (H, L):
        g = torch.Generator().manual_seed(17)
        k, v, kt, vt = (torch.randn(Z, Hk, Lk, D, generator=g).to(dtype) for _ in range(4))
    mask = _mask(mode, Z, H, L, dtype) if Lk == L else None
    causal = mode == "causal"
    kind = _lib.MASK_NONE if mask is None else (_lib.MASK_BOOL if mask.dtype == torch.bool else _lib.MASK_ADD)
    scale = D**-0.5
    npm = None if mask is None else (mask.numpy() if mask.dtype == torch.bool else mask.double().numpy())
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    dmask = None if mask is None else mask.cuda()
    print(f"dropout case Z{Z} H{H}/{Hk} L{L}/{Lk} D{D} {dtype} {mode} p={p} plain={plain}", flush=True)
    keep = be.dropout_keep(dev[0], Lk, p, seed).cpu().numpy()
    assert np.array_equal(keep, dropout.keep(Z, H, L, Lk, p, seed)), "the exported pattern differs from its restatement"
    W = dropout.keep_scale(Z, H, L, Lk, p, seed)
    names = ("dq", "dk", "dv", "dqt", "dkt", "dvt")
    if plain:
        ref = dense.forward(*f64[:3], mask=npm, causal=causal, scale=scale, keep_scale=W)
        rb = dense.backward(*f64[:3], None, None, None, f64[6], None, mask=npm, causal=causal, scale=scale, keep_scale=W)
        o, ot, M, mu = be.fwd(dev[0], dev[1], dev[2], None, None, None, dmask, kind, causal, scale, p, seed)
        _tol_check("O", o, ref["O"], dtype)
        g = be.bwd(dev[0], dev[1], dev[2], None, None, None, o, None, M, None, dev[6], None, dmask, kind, causal, scale,
                   dropout_p=p, dropout_seed=seed)
        for n, t in zip(names[:3], g[:3]):
            _tol_check(n, t, rb[n], dtype)
        return
    ref = dense.forward(*f64[:6], mask=npm, causal=causal, scale=scale, keep_scale=W)
    o, ot, M, mu = be.fwd(*dev[:6], dmask, kind, causal, scale, p, seed)
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    stat_tol = 1e-4 if dtype == torch.float32 else 2e-2
    # the softmax statistics are those of the undropped probabilities
    assert np.abs(M.double().cpu().numpy() - ref["M"]).max() < stat_tol
    assert np.abs(mu.double().cpu().numpy() - ref["mu"]).max() < stat_tol * max(1.0, np.abs(ref["mu"]).max())
    rb = dense.backward(*f64, mask=npm, causal=causal, scale=scale, keep_scale=W)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, kind, causal, scale, want_tangent_grads=True,
                   dropout_p=p, dropout_seed=seed)
    for n, t in zip(names, grads):
        _tol_check(n, t, rb[n], dtype)
    rb1 = dense.backward(*f64[:7], None, mask=npm, causal=causal, scale=scale, keep_scale=W)
    g1 = be.bwd(dev[0], dev[1], dev[2], None, None, None, o, None, M, None, dev[6], None, dmask, kind, causal, scale,
                dropout_p=p, dropout_seed=seed)
    for n, t in zip(names[:3], g1[:3]):
        _tol_check(n + "(gO only)", t, rb1[n], dtype)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("mode", ["none", "causal"])
def test_dual_with_dropout(dt, D, mode):
    _case(2, 2, 256, D, DTYPES[dt], mode, p=0.2, seed=0x1234_5678_9ABC_DEF0)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("mode", ["keypad", "bias", "bool_full"])
def test_dual_with_dropout_and_masks(dt, D, mode):
    """Every head dim and element type: the masked forward kernels with dropout all carry the in-place rescale of
    their accumulators, and every instantiation of it is run here."""
    _case(2, 2, 192, D, DTYPES[dt], mode, p=0.35, seed=77)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("L,Lk", [(33, 65), (64, 129), (130, 200)])
@pytest.mark.parametrize("causal", [False, True])
def test_keep_decisions_entry_by_entry_through_the_16_bit_kernels(D, L, Lk, causal):
    """q = 0 makes the probabilities uniform over the keys a row sees, and one-hot columns in v, v' make every entry of
    O, O' the sum of at most two entries of P * W: a single wrong keep decision (an off-by-one at a tile or
    32-row-block edge of a kernel's walk through the pattern) then moves an entry by about half its size, where
    the ordinary dropout cases would bury it under the 2e-2 bar.  Lengths straddle 32, 64 and 128; one kernel
    family per head dim (direct-to-LDS, software-pipelined, the D = 256 kernels); gO one-hot exposes the pattern
    in dv the same way."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    dtype, p, seed = torch.bfloat16, 0.3, 0xABCDEF
    Z, H = 1, 2
    g = torch.Generator().manual_seed(9)
    q = torch.zeros(Z, H, L, D)
    k = torch.randn(Z, H, Lk, D, generator=g)
    qt, kt = torch.zeros(Z, H, L, D), torch.zeros(Z, H, Lk, D)
    eye = lambda n, shift: torch.nn.functional.one_hot((torch.arange(n) + shift) % D, D).float().expand(Z, H, n, D)  # noqa: E731
    v, vt, go, gt = eye(Lk, 0), eye(Lk, 1), eye(L, 2), eye(L, 3)
    t = [x.to(dtype).contiguous() for x in (q, k, v, qt, kt, vt, go, gt)]
    f64 = [x.double().numpy() for x in t]
    dev = [x.cuda() for x in t]
    scale = D**-0.5
    W = dropout.keep_scale(Z, H, L, Lk, p, seed)
    ref = dense.forward(*f64[:6], mask=None, causal=causal, scale=scale, keep_scale=W)
    o, ot, M, mu = be.fwd(*dev[:6], None, _lib.MASK_NONE, causal, scale, p, seed)
    # every entry to a fraction of the smallest nonzero one: 1 / ((1 - p) * keys seen) in bf16
    smallest = 1.0 / ((1 - p) * Lk)
    def off(got, want):  # beyond 16-bit rounding of the entry itself
        return (np.abs(got.double().cpu().numpy() - want) - 0.01 * np.abs(want)).max()

    for name, got, want in (("O", o, ref["O"]), ("O'", ot, ref["Ot"])):
        err = off(got, want)
        assert err < 0.05 * smallest, f"{name}: an entry is off by {err:.3e}, entries are multiples of about {smallest:.3e}"
    rb = dense.backward(*f64, mask=None, causal=causal, scale=scale, keep_scale=W)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], None, _lib.MASK_NONE, causal, scale, dropout_p=p, dropout_seed=seed)
    err = off(grads[2], rb["dv"])
    assert err < 0.05 * smallest, f"dv: an entry is off by {err:.3e}"
    for n, got in zip(("dq", "dk", "dv"), grads[:3]):
        _tol_check(n, got, rb[n], dtype)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("mode", ["none", "causal"])
def test_plain_with_dropout(dt, mode):
    _case(1, 3, 200, 64, DTYPES[dt], mode, p=0.5, seed=5, plain=True)


@pytest.mark.parametrize("dt", ["fp16", "fp32"])
def test_dropout_with_grouped_heads_ragged_and_unequal_lengths(dt):
    _case(2, 4, 100, 32, DTYPES[dt], "none", p=0.1, seed=2**40 + 9, Hk=2, Lk=333)
    _case(1, 4, 77, 128, DTYPES[dt], "causal", p=0.1, seed=1, Hk=1)


def test_the_pattern_past_two_to_the_32_entries_and_both_seed_words():
    """The exported pattern is one byte per entry: past 2^32 entries the byte index no longer fits one word; a slab
    across that boundary is read back through a problem whose last rows lie beyond it.  The two seed words both
    change the pattern."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    q = torch.empty(1, 1, 8, 32, device="cuda", dtype=torch.bfloat16)
    a = be.dropout_keep(q, 64, 0.5, 1).cpu().numpy()
    b = be.dropout_keep(q, 64, 0.5, 1 + (1 << 32)).cpu().numpy()
    c = be.dropout_keep(q, 64, 0.5, 2).cpu().numpy()
    assert 0.3 < (a != b).mean() < 0.7 and 0.3 < (a != c).mean() < 0.7
    # Z*H*L*Lk = 2^32 + 2^20 entries of one byte each: a 4 GiB read-back, compared on the slab either side of 2^32
    Z, H, L, Lk = 1, 1, (1 << 16) + 16, 1 << 16
    big = be.dropout_keep(torch.empty(Z, H, L, 32, device="cuda", dtype=torch.bfloat16), Lk, 0.25, 99)
    lo = (1 << 16) - 8
    slab = big[0, 0, lo:lo + 16].cpu().numpy()
    del big
    rows, keys = np.arange(lo, lo + 16, dtype=np.uint64)[:, None], np.arange(Lk, dtype=np.uint64)[None, :]
    assert np.array_equal(slab, dropout.entry_hash(0, rows, keys, L, 99) >= np.uint64(dropout.threshold(0.25)))
    assert abs(slab.mean() - 0.75) < 0.01


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("mode", ["causal", "bool_full"])
def test_dropout_at_head_dim_256(dt, mode):
    _case(1, 2, 200, 256, DTYPES[dt], mode, p=0.25, seed=31337)


def test_dropout_at_head_dim_256_grouped_heads_unequal_lengths_and_longer_rows():
    """The D = 256 kernels walk the pattern three ways (a lane per query in the forward and dq, a lane per key in
    dk/dv with the block of 32 queries mixed once per tile, two waves per row in the dual backward)."""
    _case(2, 4, 100, 256, torch.bfloat16, "none", p=0.1, seed=77, Hk=2, Lk=333)
    _case(1, 1, 600, 256, torch.float16, "causal", p=0.3, seed=78)
    _case(1, 2, 130, 256, torch.bfloat16, "keypad", p=0.3, seed=79, plain=True)


def test_zero_probability_is_the_path_without_dropout_and_bad_arguments_are_refused():
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    q, k, v, qt, kt, vt, go, gt = (x.cuda() for x in _make(1, 2, 256, 128, torch.bfloat16, seed=1))
    a = be.fwd(q, k, v, qt, kt, vt, None, _lib.MASK_NONE, True, 128**-0.5)
    b = be.fwd(q, k, v, qt, kt, vt, None, _lib.MASK_NONE, True, 128**-0.5, 0.0, 123)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    with pytest.raises(RuntimeError, match="libjvpfa"):
        be.fwd(q, k, v, None, None, None, None, _lib.MASK_NONE, False, 1.0, 1.0, 1)
    with pytest.raises(RuntimeError, match="libjvpfa"):
        be.fwd(q, k, v, None, None, None, None, _lib.MASK_NONE, False, 1.0, -0.5, 1)


def test_public_surface_with_dropout_is_repeatable_under_a_seed_and_feeds_forward_and_reverse_mode():
    """``attention(..., dropout_p=p)`` end to end: torch.manual_seed fixes the pattern, the backward regenerates
    it, and the kept probabilities are rescaled so that their expected row sum stays 1."""
    import torch.autograd.forward_ad as fwAD

    from jvp_flash_attention_amd import attention

    q, k, v, qt, kt, vt, go, gt = (x.cuda() for x in _make(2, 2, 512, 64, torch.bfloat16, seed=4))
    torch.manual_seed(5)
    seed = int(torch.randint(0, 2**62, (1,)).item())  # what the call below will draw
    torch.manual_seed(5)
    leaves = [t.clone().requires_grad_() for t in (q, k, v, qt, kt, vt)]
    with fwAD.dual_level():
        duals = [fwAD.make_dual(a, b) for a, b in zip(leaves[:3], leaves[3:])]
        o, ot = fwAD.unpack_dual(attention(*duals, dropout_p=0.3))
        ((o.float() * go.float()).sum() + (ot.float() * gt.float()).sum()).backward()
    W = dropout.keep_scale(2, 2, 512, 512, 0.3, seed)
    f64 = [x.double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    ref = dense.forward(*f64[:6], keep_scale=W)
    rb = dense.backward(*f64, keep_scale=W)
    _tol_check("O", o, ref["O"], torch.bfloat16)
    _tol_check("O'", ot, ref["Ot"], torch.bfloat16)
    for leaf, n in zip(leaves, ("dq", "dk", "dv", "dqt", "dkt", "dvt")):
        _tol_check(n, leaf.grad, rb[n], torch.bfloat16)
    torch.manual_seed(5)
    assert torch.equal(attention(q, k, v, dropout_p=0.3), o.detach())
    other = attention(q, k, v, dropout_p=0.3)
    assert not torch.equal(other, o.detach())
    # unbiased: with V = 1 each output is the sum of a row's kept, rescaled probabilities, 1 in expectation
    ones = torch.ones_like(v)
    assert abs(attention(q, k, ones, dropout_p=0.3).float().mean().item() - 1.0) < 0.01


def test_dropout_inside_torch_compile_runs_between_two_compiled_pieces():
    """The seed is drawn on the host, so a call with dropout is left out of the traced graph; output and gradients
    are those of the eager call made from the same generator state."""
    from jvp_flash_attention_amd import attention

    q, k, v = [x.cuda().requires_grad_() for x in _make(1, 2, 200, 64, torch.bfloat16, seed=6)[:3]]

    def f(q, k, v):
        return (attention(q * 1.0, k, v, dropout_p=0.25, causal=True) * 2.0).float().sum()

    torch.manual_seed(3)
    ref = f(q, k, v)
    gref = torch.autograd.grad(ref, (q, k, v))
    torch._dynamo.reset()
    torch.manual_seed(3)
    out = torch.compile(f, backend="aot_eager")(q, k, v)
    g = torch.autograd.grad(out, (q, k, v))
    assert torch.equal(out, ref)
    for a, b in zip(g, gref):
        assert torch.equal(a, b)
    assert not torch.equal(f(q, k, v), ref)  # the next draw is another pattern


def test_a_recorded_dropout_call_replays_its_pattern():
    """The seed is a kernel argument drawn on the host: a forward with dropout recorded into a HIP graph replays with
    the seed it was recorded with, the same keep pattern every time (callers that want a fresh pattern per step
    record anew).  Pinned here so that the behaviour is a documented one."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, L, D = 1, 2, 256, 64
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v = [torch.randn(Z, H, L, D, generator=g, device="cuda").to(torch.bfloat16) for _ in range(3)]
    scale = D**-0.5
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        be.fwd(q, k, v, None, None, None, None, _lib.MASK_NONE, False, scale, 0.5, 1234)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o = be.fwd(q, k, v, None, None, None, None, _lib.MASK_NONE, False, scale, 0.5, 1234)[0]
    graph.replay()
    torch.cuda.synchronize()
    first = o.clone()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(first, o)
    assert torch.equal(first, be.fwd(q, k, v, None, None, None, None, _lib.MASK_NONE, False, scale, 0.5, 1234)[0])
    assert not torch.equal(first, be.fwd(q, k, v, None, None, None, None, _lib.MASK_NONE, False, scale, 0.5, 1235)[0])

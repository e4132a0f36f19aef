"""Host-side logic on CPU: argument checks, mask classification and the autograd / forward-mode
wiring of ``JVPAttn``, with the device work replaced by the oracle's tile-loop restatement
(``tests/fake_backend.py``).  What is checked here is the plumbing, against the SDPA route."""
from functools import partial

import pytest
import torch
import torch.autograd.forward_ad as fwAD

from jvp_flash_attention_amd import MASK_CONST, JVPAttn, attention
from jvp_flash_attention_amd import _lib
from oracle import sdpa_jvp
from tests.fake_backend import oracle_backend


def _inputs(Z=1, H=2, L=32, D=32, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(Z, H, L, D, generator=g) for _ in range(8)]


def _close(a, b, tol=2e-5):
    assert (a - b).abs().max().item() <= tol * max(1.0, b.abs().max().item())


def test_import_path_alias_matches_reference_import_line():
    from jvp_flash_attention.jvp_attention import JVPAttn as J2, attention as a2, MASK_CONST as m2

    assert J2 is JVPAttn and a2 is attention and m2 == MASK_CONST == -100.0


def test_plain_attention_and_first_order_backward():
    q, k, v, qt, kt, vt, go, _ = _inputs()
    _, _, ref = sdpa_jvp.forward_backward(q, k, v, qt, kt, vt, go, None)
    o_ref, _ = sdpa_jvp.forward(q, k, v, qt, kt, vt)
    with oracle_backend() as be:
        qq, kk, vv = [x.clone().requires_grad_() for x in (q, k, v)]
        o = attention(qq, kk, vv)
        (o * go).sum().backward()
        assert be.calls[0][:2] == ("fwd", False) and be.calls[1][:2] == ("bwd", False)
    _close(o, o_ref)
    for got, want in zip((qq.grad, kk.grad, vv.grad), ref[:3]):
        _close(got, want)


@pytest.mark.parametrize("causal", [False, True])
def test_fwd_dual_three_way_like_reference_tests(causal):
    """SDPA under fwAD vs fwd_dual under fwAD vs torch.func.jvp(fwd_dual): the reference's own
    three-way comparison (tests/test_jvp_attention.py:572-617)."""
    q, k, v, qt, kt, vt, _, _ = _inputs()
    o_ref, ot_ref = sdpa_jvp.forward(q, k, v, qt, kt, vt, causal=causal)
    with oracle_backend():
        with fwAD.dual_level():
            out = JVPAttn.fwd_dual(fwAD.make_dual(q, qt), fwAD.make_dual(k, kt), fwAD.make_dual(v, vt), causal=causal)
            o1, ot1 = fwAD.unpack_dual(out)
            o1, ot1 = o1.clone(), ot1.clone()
        o2, ot2 = torch.func.jvp(partial(JVPAttn.fwd_dual, causal=causal), (q, k, v), (qt, kt, vt))
    for o, ot in ((o1, ot1), (o2, ot2)):
        _close(o, o_ref)
        _close(ot, ot_ref)


def test_attention_notices_dual_inputs():
    """attention() under forward-mode AD returns the tangent too (the reference needs fwd_dual for that)."""
    q, k, v, qt, kt, vt, _, _ = _inputs(seed=3)
    o_ref, ot_ref = sdpa_jvp.forward(q, k, v, qt, kt, vt)
    with oracle_backend() as be:
        o2, ot2 = torch.func.jvp(attention, (q, k, v), (qt, kt, vt))
        assert be.calls[0][:2] == ("fwd", True)
        with fwAD.dual_level():
            o1, ot1 = fwAD.unpack_dual(attention(fwAD.make_dual(q, qt), k, v))  # k, v without tangents
            o1, ot1 = o1.clone(), ot1.clone()
    _close(o2, o_ref)
    _close(ot2, ot_ref)
    _close(o1, o_ref)
    _close(ot1, sdpa_jvp.forward(q, k, v, qt, torch.zeros_like(kt), torch.zeros_like(vt))[1])


def test_gradients_through_the_tangent_reach_all_six_inputs():
    q, k, v, qt, kt, vt, go, gt = _inputs()
    _, _, ref = sdpa_jvp.forward_backward(q, k, v, qt, kt, vt, go, gt)
    with oracle_backend() as be:
        leaves = [x.clone().requires_grad_() for x in (q, k, v, qt, kt, vt)]
        with fwAD.dual_level():
            out = JVPAttn.fwd_dual(*(fwAD.make_dual(p, t) for p, t in zip(leaves[:3], leaves[3:])))
            o, ot = fwAD.unpack_dual(out)
            grads = torch.autograd.grad((o * go).sum() + (ot * gt).sum(), leaves)
        assert ("bwd", True, 0, False, True) in be.calls  # tangent grads requested
    for got, want in zip(grads, ref):
        _close(got, want)


def test_hvp_style_gradient_of_tangent_only_under_func_jvp():
    q, k, v, qt, kt, vt, _, gt = _inputs()
    _, _, ref = sdpa_jvp.forward_backward(q, k, v, qt, kt, vt, torch.zeros_like(q), gt)
    with oracle_backend() as be:
        leaves = [x.clone().requires_grad_() for x in (q, k, v)]
        _, ot = torch.func.jvp(JVPAttn.fwd_dual, tuple(leaves), (qt, kt, vt))
        grads = torch.autograd.grad((ot * gt).sum(), leaves)
        assert be.calls[-1][:2] == ("bwd", True) and be.calls[-1][-1] is False  # primal grads only
    for got, want in zip(grads, ref[:3]):
        _close(got, want)


def test_apply_returns_output_and_context_tuple_and_13_slot_backward():
    q, k, v, qt, kt, vt, go, _ = _inputs()
    _, ot_ref = sdpa_jvp.forward(q, k, v, qt, kt, vt)
    with oracle_backend():
        qq = q.clone().requires_grad_()
        out = JVPAttn.apply(qq, k, v, qt, kt, vt, None, 0.0, False, None, True, True)
        o, ctx = out
        o_t, M, grid, head_dim, sm_scale, mask_tensor, mask_type, dropout_p, seed, drop = ctx
        _close(o_t, ot_ref)
        assert M.shape == q.shape[:3] and M.dtype == torch.float32
        assert tuple(grid) == (1, 2, 1) and head_dim == 32 and mask_type == 0 and dropout_p == 0.0 and not drop
        assert abs(sm_scale - 32**-0.5) < 1e-12 and mask_tensor.numel() == 0
        (o * go).sum().backward()
        assert qq.grad is not None
    assert len(JVPAttn.BwdOut._fields) == 13

    class Ctx:
        pass

    with oracle_backend():
        o, ctx = JVPAttn.forward(q, k, v, None, None, None)
        c = Ctx()
        c.saved_tensors = (q, k, v, o, ctx.M)
        c.mask_tensor, c.MASK_TYPE, c.causal, c.sm_scale = ctx.mask_tensor, 0, False, ctx.sm_scale
        c.dropout_p, c.philox_seed, c.ENABLE_DROPOUT = ctx.dropout_p, ctx.philox_seed, ctx.ENABLE_DROPOUT  # JA:2696-2698
        res = JVPAttn.backward(c, go, None)
    assert isinstance(res, JVPAttn.BwdOut) and all(x is None for x in res[3:]) and all(x is not None for x in res[:3])


def test_argument_errors_match_the_reference():
    q, k, v, *_ = _inputs()
    with oracle_backend():
        with pytest.raises(AssertionError):
            attention(q, k, v, dropout_p=1.0)
        with pytest.raises(AssertionError):
            attention(q, k, v, dropout_p=-0.1)
        with pytest.raises(ValueError):
            attention(q, k, v, attn_mask=torch.ones(1, 2, 32, 32, dtype=torch.bool), causal=True)
        with pytest.raises(AssertionError):
            attention(q, k, v[..., :16])
        with pytest.raises(AssertionError):
            attention(q[..., :24], k[..., :24], v[..., :24])  # head dim not supported
        with pytest.raises(AssertionError):
            attention(q, k, v, attn_mask=torch.ones(1, 2, 32, 16, dtype=torch.bool))
        with pytest.raises(AssertionError):
            attention(q, k, v, attn_mask=torch.zeros(1, 2, 32, 32, dtype=torch.float64))
        bad = torch.ones(1, 2, 32, 32, dtype=torch.bool)
        bad[0, 1] = False
        with pytest.raises(AssertionError):
            attention(q, k, v, attn_mask=bad)  # a head with every key masked
        nanmask = torch.zeros(1, 2, 32, 32)
        nanmask[0, 0, 0, 0] = float("nan")
        with pytest.raises(AssertionError):
            attention(q, k, v, attn_mask=nanmask)
        # a float mask without MASK_CONST is fine here (the reference raises UserWarning)
        attention(q, k, v, attn_mask=torch.zeros(1, 2, 32, 32))


@pytest.mark.parametrize("kind", ["keypad", "bias", "mask_const"])
def test_masks_follow_sdpa_semantics(kind):
    q, k, v, qt, kt, vt, go, gt = _inputs(Z=2)
    if kind == "keypad":
        mask = (torch.arange(32)[None, :] < torch.tensor([20, 32])[:, None]).view(2, 1, 1, 32)
        sdpa_mask = mask
    elif kind == "bias":
        mask = torch.randn(2, 2, 32, 32, generator=torch.Generator().manual_seed(3))
        sdpa_mask = mask
    else:  # the reference's float-mask convention: MASK_CONST marks masked entries
        keep = torch.rand(2, 2, 32, 32, generator=torch.Generator().manual_seed(4)) > 0.5
        keep[..., 0] = True
        mask = torch.where(keep, 0.0, MASK_CONST)
        sdpa_mask = keep
    o_ref, ot_ref, ref = sdpa_jvp.forward_backward(q, k, v, qt, kt, vt, go, gt, attn_mask=sdpa_mask)
    with oracle_backend() as be:
        leaves = [x.clone().requires_grad_() for x in (q, k, v)]
        o, ot = torch.func.jvp(partial(JVPAttn.fwd_dual, attn_mask=mask), tuple(leaves), (qt, kt, vt))
        grads = torch.autograd.grad((o * go).sum() + (ot * gt).sum(), leaves)
        expect = _lib.MASK_BOOL if mask.dtype == torch.bool else _lib.MASK_ADD
        assert be.calls[0][2] == expect
    tol = 2e-5 if kind != "mask_const" else 1e-4  # exp(-100) is not exactly 0
    _close(o, o_ref, tol)
    _close(ot, ot_ref, tol)
    for got, want in zip(grads, ref[:3]):
        _close(got, want, tol)


def test_broadcast_mask_strides_are_zero_on_size_one_axes():
    q = torch.zeros(2, 3, 8, 32)
    mask = torch.ones(2, 1, 1, 8, dtype=torch.bool)
    p = _lib.make_problem(q, mask, _lib.MASK_BOOL, False, 0.5)
    assert list(p.mask_stride) == [8, 0, 0, 1] and p.mask_kind == _lib.MASK_BOOL
    assert (p.Z, p.H, p.L, p.D, p.dtype, p.causal) == (2, 3, 8, 32, 2, 0)


def test_non_contiguous_inputs_are_copied_and_missing_tangents_are_zero():
    q, k, v, qt, kt, vt, _, _ = _inputs()
    qn = q.transpose(1, 2).contiguous().transpose(1, 2)
    assert not qn.is_contiguous()
    o_ref, ot_ref = sdpa_jvp.forward(q, k, v, qt, torch.zeros_like(k), torch.zeros_like(v))
    with oracle_backend():
        with fwAD.dual_level():
            out = JVPAttn.fwd_dual(fwAD.make_dual(qn, qt), k, v)  # only q carries a tangent
            o, ot = fwAD.unpack_dual(out)
            _close(o, o_ref)
            _close(ot, ot_ref)
        # no tangents at all: plain forward
        _close(JVPAttn.fwd_dual(q, k, v), o_ref)


def test_product_has_no_cpu_path():
    q, k, v, *_ = _inputs()
    with pytest.raises(RuntimeError, match="no CPU path|There is no CPU path"):
        attention(q, k, v)


def test_registered_operators_describe_their_outputs_without_running():
    """``jvpfa::fwd`` / ``jvpfa::bwd`` are what ``torch.compile`` records in place of the ctypes calls;
    their shape functions must agree with what the library returns (empty tensors stand for absent
    tangent outputs).  Fake tensors only: nothing is launched."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    from jvp_flash_attention_amd import _lib  # noqa: F401  (registers the operators)

    with FakeTensorMode():
        q = torch.empty(2, 3, 64, 64, device="cuda", dtype=torch.bfloat16)
        o, ot, M, mu = torch.ops.jvpfa.fwd(q, q, q, None, None, None, None, 0, False, 0.125)
        assert o.shape == q.shape and o.dtype == q.dtype and ot.numel() == 0 and mu.numel() == 0
        assert M.shape == (2, 3, 64) and M.dtype == torch.float32
        o, ot, M, mu = torch.ops.jvpfa.fwd(q, q, q, q, q, q, None, 0, True, 0.125)
        assert ot.shape == q.shape and mu.shape == (2, 3, 64) and mu.dtype == torch.float32
        g = torch.ops.jvpfa.bwd(q, q, q, q, q, q, o, ot, M, mu, q, q, None, 0, True, 0.125, True)
        assert [t.shape for t in g] == [q.shape] * 6
        g = torch.ops.jvpfa.bwd(q, q, q, None, None, None, o, None, M, None, q, None, None, 0, True, 0.125, False)
        assert [t.shape for t in g[:3]] == [q.shape] * 3 and all(t.numel() == 0 for t in g[3:])


def test_mask_verification_is_remembered_per_mask_version():
    """``verify_attn_mask`` reads the whole mask; a mask that passed is not read again until it changes."""
    import torch

    from jvp_flash_attention_amd import jvp_attention as ja

    q = torch.zeros(1, 1, 4, 32)
    mask = torch.ones(1, 1, 4, 4, dtype=torch.bool)
    ja._classify_mask(mask, q, True)
    assert ja._already_verified(mask)
    mask[0, 0] = False  # an in-place change bumps the version: the check runs again and fails
    assert not ja._already_verified(mask)
    with pytest.raises(AssertionError, match="all False"):
        ja._classify_mask(mask, q, True)
    bias = torch.zeros(1, 1, 4, 4)
    ja._classify_mask(bias, q, True)
    assert ja._already_verified(bias)
    bias[0, 0, 1, 2] = float("nan")
    with pytest.raises(AssertionError, match="NaN"):
        ja._classify_mask(bias, q, True)
    bias[0, 0, 1, 2] = float("inf")
    with pytest.raises(AssertionError, match=r"\+inf"):
        ja._classify_mask(bias, q, True)
    bias[0, 0, 1, 2] = float("-inf")  # -inf is a legal "masked" value
    ja._classify_mask(bias, q, True)


def test_key_limit_of_a_mask_shared_by_the_batch_follows_the_batch_size_of_each_call():
    """One [1,1,1,L] key-padding mask used with two batch sizes: the kernels index the limits by batch entry,
    so each call must get as many as it has batch entries (the cache keeps one value per row of the mask)."""
    L = _lib.KEY_LIMIT_MIN_L
    mask = torch.ones(1, 1, 1, L, dtype=torch.bool)
    mask[..., 300:] = False
    assert _lib.key_limit_hint(mask, _lib.MASK_BOOL, 2, L).tolist() == [300, 300]
    assert _lib.key_limit_hint(mask, _lib.MASK_BOOL, 8, L).tolist() == [300] * 8
    assert _lib.key_limit_hint(mask, _lib.MASK_BOOL, 1, L).tolist() == [300]
    assert mask._jvpfa_key_limit[1].shape == (1,)


def test_masks_made_in_inference_mode_have_no_version_counter_and_are_not_cached():
    from jvp_flash_attention_amd import jvp_attention as ja

    L = _lib.KEY_LIMIT_MIN_L
    with torch.inference_mode():
        mask = torch.ones(2, 1, 1, L, dtype=torch.bool)
        mask[1, ..., 100:] = False
        bias = torch.zeros(1, 1, 4, 4)
    assert _lib.mask_version(mask) is None
    q = torch.zeros(2, 1, 4, 32)
    assert ja._classify_mask(mask, q, True)[1] == _lib.MASK_BOOL     # verified, every time
    assert not ja._already_verified(mask)
    assert ja._classify_mask(bias, q[:1], True)[1] == _lib.MASK_ADD
    assert _lib.key_limit_hint(mask, _lib.MASK_BOOL, 2, L).tolist() == [L, 100]
    assert not hasattr(mask, "_jvpfa_key_limit")
    with torch.inference_mode(), oracle_backend():
        o = attention(torch.randn(2, 1, L, 32), torch.randn(2, 1, L, 32), torch.randn(2, 1, L, 32), attn_mask=mask)
    assert torch.isfinite(o).all()


def test_forget_mask_drops_what_was_remembered():
    from jvp_flash_attention_amd import jvp_attention as ja

    L = _lib.KEY_LIMIT_MIN_L
    mask = torch.ones(2, 1, 1, L, dtype=torch.bool)
    ja._classify_mask(mask, torch.zeros(2, 1, 4, 32), True)
    _lib.key_limit_hint(mask, _lib.MASK_BOOL, 2, L)
    mask.data[1, ..., 7:] = False  # a write that does not bump the version counter
    assert _lib.key_limit_hint(mask, _lib.MASK_BOOL, 2, L).tolist() == [L, L]  # stale, as documented
    _lib.forget_mask(mask)
    assert not ja._already_verified(mask)
    assert _lib.key_limit_hint(mask, _lib.MASK_BOOL, 2, L).tolist() == [L, 7]


def test_dropout_draws_one_seed_per_call_and_replays_it_in_the_backward():
    """dropout_p > 0 (the reference raises, jvp_attention.py:2356-2357): the forward draws a seed from torch's
    CPU generator, the backward of the same call gets that seed again, and the results are those of SDPA's
    dropout with that pattern, tangent and tangent-path gradients included."""
    from oracle import dense, dropout

    q, k, v, qt, kt, vt, go, gt = _inputs()
    Z, H, L, _ = q.shape
    with oracle_backend() as fake:
        torch.manual_seed(11)
        leaves = [t.clone().requires_grad_() for t in (q, k, v, qt, kt, vt)]
        with fwAD.dual_level():
            duals = [fwAD.make_dual(p, t) for p, t in zip(leaves[:3], leaves[3:])]
            o, ot = fwAD.unpack_dual(attention(*duals, dropout_p=0.25))
            ((o * go).sum() + (ot * gt).sum()).backward()
        fwd_calls = [c for c in fake.calls if c[0] == "fwd"]
        bwd_calls = [c for c in fake.calls if c[0] == "bwd"]
        assert len(fwd_calls) == 1 and len(bwd_calls) == 1
        p, seed = fwd_calls[0][-2:]
        assert p == 0.25 and 0 <= seed < 2**62 and bwd_calls[0][-2:] == (p, seed)
        W = dropout.keep_scale(Z, H, L, L, p, seed)
        xs = [x.numpy() for x in (q, k, v, qt, kt, vt)]
        f = dense.forward(*xs, keep_scale=W)
        b = dense.backward(*xs, go.numpy(), gt.numpy(), keep_scale=W)
        _close(o.detach(), torch.from_numpy(f["O"]))
        _close(ot.detach(), torch.from_numpy(f["Ot"]))
        for leaf, name in zip(leaves, ("dq", "dk", "dv", "dqt", "dkt", "dvt")):
            _close(leaf.grad, torch.from_numpy(b[name]))
        # same generator state, same pattern; another call, another pattern; plain path and apply() carry it too
        torch.manual_seed(11)
        o2 = attention(q, k, v, dropout_p=0.25)
        _close(o2, o.detach())
        o3 = attention(q, k, v, dropout_p=0.25)
        assert (o3 - o2).abs().max() > 1e-3
        out, ctx = JVPAttn.apply(q, k, v, None, None, None, None, 0.25, False, None, True, True)
        assert ctx.dropout_p == 0.25 and ctx.ENABLE_DROPOUT and ctx.philox_seed == fake.calls[-1][-1]
        assert torch.equal(attention(q, k, v, dropout_p=0.0), attention(q, k, v))


def test_bench_measures_one_gpu_and_says_so():
    """`bench.py --gpus N` with N above 1 exits with a message instead of measuring anything."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)


def test_validation_report_figures_from_synthetic_rows(tmp_path):
    """``validate.plot_report`` (the reference's two PNG figures): one panel per (causal, mask) configuration,
    files named as the reference names them; drawn here from made-up rows, no GPU involved."""
    pytest.importorskip("matplotlib")
    from jvp_flash_attention_amd import validate

    rows = [{"L": L, "mask": mask, "causal": causal, "speedup": 3.0 + L / 512, "mem_mb": 1.0 + L / 64,
             "mem_mb_sdpa": 2.0 + (L / 64) ** 2}
            for L in (128, 512, 2048) for mask, causal in (("none", False), ("none", True), ("boolean", False), ("additive", False))]
    paths = validate.plot_report(rows, "bfloat16", str(tmp_path), masks=True)
    assert [p.split("/")[-1] for p in paths] == ["bfloat16_jvp_attention_perf_with_masks.png", "bfloat16_jvp_attention_mem_with_masks.png"]
    for p in paths:
        with open(p, "rb") as f:
            head = f.read(8)
        assert head == b"\x89PNG\r\n\x1a\n"
    assert validate.plot_report(rows[:3], "float32", str(tmp_path), masks=False)[0].endswith("float32_jvp_attention_perf.png")

"""JVP flash attention for MI355X: the Python surface of amorehead/jvp_flash_attention on HIP kernels.

Mirrors ``jvp_flash_attention/jvp_attention.py`` of the reference ("JA" below): the same names
(``JVPAttn``, ``JVPAttn.fwd``, ``JVPAttn.fwd_dual``, ``attention``, ``MASK_CONST``), the same
13-argument ``JVPAttn.forward`` (JA:2311-2325), the same ``(o, ctx_tuple)`` result of
``JVPAttn.apply`` (JA:2633-2647) and 13-slot ``backward`` (JA:2285-2300).  The device work goes
through the C ABI of ``libjvpfa.so`` (hand-written gfx950 kernels); there is no other code path.

Differences from the reference, all deliberate:

* Float masks follow ``scaled_dot_product_attention``: they are added to the *scaled* logits and
  are part of the backward recomputation (the reference scales the mask too, JA:247-251, and
  leaves it out of the backward, JA:1519-1522).  A float mask without any ``MASK_CONST`` entry is
  accepted (the reference raises ``UserWarning``, JA:2459-2462).
* Boolean masks mask exactly: a masked key gets probability 0, and a query row with every key masked gives
  O = O' = 0, M = +inf and zero gradients.  The reference adds ``MASK_CONST`` = -100 to the unscaled logits
  (JA:241-245), so a masked key keeps a weight of about exp(-100 * sm_scale) next to the attended ones (1e-4 at
  D = 128) and a fully masked row comes out as plain unmasked softmax; neither is reproduced, and no fixture of
  the reference pins either, so for those rows the comparison with the reference is unpinned.
* Masks may broadcast: any shape whose axes are 1 or (Z, H, L, L); a key-padding mask
  ``[Z,1,1,L]`` is read in place.  The reference requires the full shape (JA:2383-2388).
* ``fwd_dual`` returns an output whose tangent O' carries an autograd graph, so gradients of
  functions of O' (Hessian-vector products) reach q, k, v and the input tangents.  The
  reference's tangent is a constant (JA:2399, JA:2828) and its backward ignores it (JA:2831).
* Any sequence length L >= 1 (the reference: an even L >= 32, JA:2375-2378, and a multiple of its tile sizes,
  JA:2892).  Head dims as there, {16, 32, 64, 128, 256} (JA:2371-2374); 16 runs on the kernels for 32 with zero
  columns appended.
* k and v may have fewer heads than q (grouped heads: H a multiple of H_kv) and a length of their own
  (cross-attention); causal then means key index <= query index, as in SDPA.  The reference requires
  q, k, v of one shape (JA:2367-2378).
* ``dropout_p`` > 0 works (the reference carries dead code for it and raises ``NotImplementedError``,
  JA:94-122, JA:271-277, JA:2356-2357): dropout on the attention probabilities with SDPA's semantics (kept entries
  scaled by 1/(1-p); the tangent O' sees the same pattern), the pattern a counter-based hash of a seed drawn from
  torch's CPU generator per call (``torch.manual_seed`` makes it repeatable) and of the entry's coordinates, regenerated in
  the backward.  (bf16 / fp16 calls get 6 - 13 % slower at head dim 128, about 30 % at 64, fp32 1 - 6 %.)
* ``attention`` notices dual inputs and then behaves like ``fwd_dual`` (the reference's ``attention``
  is ``JVPAttn.fwd`` and drops the tangent, its README.md:65-67).
* Under ``torch.compile`` every call stays inside the graph (``fullgraph=True``), also with a forward-mode level
  opened inside the compiled function and with dropout; the reference's Function defines ``jvp``, which the tracer
  refuses, so there every call is a graph break.
"""
from __future__ import annotations

from typing import Any, Literal, NamedTuple

import torch
import torch.autograd.forward_ad as fwAD
from torch import Tensor
from torch.autograd import Function
from torch.autograd.function import FunctionCtx, once_differentiable

from . import _lib

MASK_CONST = -100.0  # JA:48-50: value float masks use for "masked"; far below any real logit
MIN_SEQUENCE_LENGTH = 32  # JA:51; kept for importers, not a limit of these kernels
SUPPORTED_HEAD_DIMS = (16, 32, 64, 128, 256)
BLOCK_M = 128  # query rows per workgroup of the forward kernel (only reported through Grid)


def is_hip() -> bool:
    """Platform probes of the reference (JA:54-92), kept for importers: this build is HIP-only."""
    return True


def is_cuda() -> bool:
    return False


def supports_host_descriptor() -> bool:
    return False


def supports_tma() -> bool:
    return False


def is_blackwell() -> bool:
    return False


def _validate(q: Tensor, k: Tensor, v: Tensor, attn_mask: Tensor | None, dropout_p: float, causal: bool):
    """Argument checks of JA:2356-2392, with this build's shape limits."""
    assert 0.0 <= dropout_p < 1.0, f"dropout_p must be in [0, 1), but got {dropout_p}"
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must be (Z, H, N_CTX, HEAD_DIM)"
    Z, H, N_CTX, HEAD_DIM_Q = q.shape
    HEAD_DIM_K, HEAD_DIM_V = k.shape[-1], v.shape[-1]
    assert HEAD_DIM_Q == HEAD_DIM_K and HEAD_DIM_K == HEAD_DIM_V, (
        "JVP attention requires HEAD_DIM_Q == HEAD_DIM_K == HEAD_DIM_V"
        f" but got HEAD_DIM_Q={HEAD_DIM_Q}, HEAD_DIM_K={HEAD_DIM_K}, HEAD_DIM_V={HEAD_DIM_V}"
    )
    assert HEAD_DIM_K in SUPPORTED_HEAD_DIMS, (
        f"JVP attention only supports HEAD_DIM_K in {set(SUPPORTED_HEAD_DIMS)}, but got HEAD_DIM_K={HEAD_DIM_K}"
    )
    assert k.shape == v.shape and k.shape[0] == Z and H % k.shape[1] == 0, (
        "JVP attention requires k and v of one shape (Z, H_kv, N_CTX_kv, HEAD_DIM) with H a multiple of H_kv,"
        f" but got q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}"
    )
    assert N_CTX >= 1, f"JVP attention requires N_CTX >= 1, but got N_CTX={N_CTX}"
    assert q.dtype in _lib.DTYPES and k.dtype == q.dtype and v.dtype == q.dtype, (
        f"q, k, v must share one dtype out of bfloat16/float16/float32, got {q.dtype}, {k.dtype}, {v.dtype}"
    )
    if causal and attn_mask is not None:
        raise ValueError("Causal attention does not support an attention mask.")
    if attn_mask is not None:
        assert attn_mask.dim() == 4 and all(
            m in (1, full) for m, full in zip(attn_mask.shape, (Z, H, N_CTX, k.shape[2]))
        ), "The provided attention mask must have 4 dimensions broadcastable to (Z, H, N_CTX, N_CTX_kv)."
        assert attn_mask.dtype in {torch.bool, q.dtype}, (
            "The attention mask must be of the dtype bool or that of the query tensor."
        )


def _already_verified(mask: Tensor) -> bool:
    """The checks of ``verify_attn_mask`` read the whole mask and wait for the answer; a mask that
    passed them is remembered on the tensor, keyed by its version counter, so that the layers of a
    model and the steps of a loop that share one mask pay once."""
    version = _lib.mask_version(mask)
    return version is not None and getattr(mask, "_jvpfa_verified", None) == version


def _remember_verified(mask: Tensor) -> None:
    version = _lib.mask_version(mask)
    if version is None:
        return
    try:
        mask._jvpfa_verified = version
    except (AttributeError, RuntimeError):
        pass


def _classify_mask(attn_mask: Tensor | None, q: Tensor, verify_attn_mask: bool):
    """Mask kind and the tensor the kernels read (JA:2429-2462)."""
    if attn_mask is None:
        return torch.empty(0, device=q.device, dtype=q.dtype), _lib.MASK_NONE
    if attn_mask.dtype == torch.bool:
        mask_tensor = attn_mask
        if verify_attn_mask and not _already_verified(attn_mask):
            assert mask_tensor.any(dim=-1).any(dim=-1).all(), (
                "The attention mask cannot be all False for any head."
            )
            _remember_verified(attn_mask)
        return mask_tensor, _lib.MASK_BOOL
    mask_tensor = attn_mask.to(q.dtype)
    if verify_attn_mask and not _already_verified(attn_mask):
        # one pass: neither NaN nor +inf compares <= the largest finite value; the reference's two
        # messages (JA:2447-2456) are told apart only when the pass fails
        if not bool((mask_tensor <= torch.finfo(mask_tensor.dtype).max).all()):
            assert not torch.isnan(mask_tensor).any(), "The attention mask cannot contain NaNs."
            assert not torch.isposinf(mask_tensor).any(), "The attention mask cannot contain +inf."
        _remember_verified(attn_mask)
    return mask_tensor, _lib.MASK_ADD


def _unwrap(x):
    """Strip functorch wrappers from a saved tensor (JA:2846-2855)."""
    while isinstance(x, Tensor) and torch._C._functorch.is_functorch_wrapped_tensor(x):
        x = torch._C._functorch.get_unwrapped(x)
    return x


def _new_dropout_seed(dropout_p: float) -> int:
    """A fresh seed for one forward call (0 without dropout), from torch's CPU generator: no device work, and
    ``torch.manual_seed`` makes a run repeatable."""
    return int(torch.randint(0, 2**62, (1,)).item()) if dropout_p > 0.0 else 0


def _dense(t: Tensor | None) -> Tensor | None:
    return None if t is None else (t if t.is_contiguous() else t.contiguous())


class _DualCore(Function):
    """(q, k, v, q', k', v') -> (O, O', M, mu), differentiable in all six tensor inputs.

    The backward is the closed form for ``<gO,O> + <gT,O'>``; with gT = 0 it is the reference's
    backward (JA:1541-1553, JA:1687-1697).
    """

    @staticmethod
    def forward(q, k, v, q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p=0.0, seed=0):
        o, o_t, M, mu = _lib.backend().fwd(q, k, v, q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale,
                                           dropout_p, seed)
        return o, o_t, M, mu

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        q, k, v, q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p, seed = inputs
        o, o_t, M, mu = outputs
        ctx.mark_non_differentiable(M, mu)
        ctx.save_for_backward(q, k, v, q_t, k_t, v_t, o, o_t, M, mu)
        ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale = mask_tensor, MASK_TYPE, causal, sm_scale
        ctx.dropout_p, ctx.philox_seed = dropout_p, seed

    @staticmethod
    @once_differentiable
    def backward(ctx, go, gt, _gM, _gmu):
        q, k, v, q_t, k_t, v_t, o, o_t, M, mu = (_unwrap(t) for t in ctx.saved_tensors)
        want_t = any(ctx.needs_input_grad[3:6])
        dq, dk, dv, dqt, dkt, dvt = _lib.backend().bwd(
            q, k, v, q_t, k_t, v_t, o, o_t, M, mu, _dense(go), _dense(gt),
            ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale, want_tangent_grads=want_t,
            dropout_p=ctx.dropout_p, dropout_seed=ctx.philox_seed,
        )
        return dq, dk, dv, dqt, dkt, dvt, None, None, None, None, None, None


class _PlainCore(Function):
    """(q, k, v) -> (O, M) with the first-order backward: what ``JVPAttn`` computes without tangents,
    as a Function without a custom ``jvp`` (which ``torch.compile`` refuses to trace).  ``JVPAttn.fwd``
    uses it while compiling."""

    @staticmethod
    def forward(q, k, v, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p=0.0, seed=0):
        o, _o_t, M, _mu = _lib.backend().fwd(q, k, v, None, None, None, mask_tensor, MASK_TYPE, causal, sm_scale,
                                             dropout_p, seed)
        return o, M

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        q, k, v, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p, seed = inputs
        o, M = outputs
        ctx.mark_non_differentiable(M)
        ctx.save_for_backward(q, k, v, o, M)
        ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale = mask_tensor, MASK_TYPE, causal, sm_scale
        ctx.dropout_p, ctx.philox_seed = dropout_p, seed

    @staticmethod
    @once_differentiable
    def backward(ctx, go, _gM):
        q, k, v, o, M = ctx.saved_tensors
        dq, dk, dv, _, _, _ = _lib.backend().bwd(
            q, k, v, None, None, None, o, None, M, None, _dense(go), None,
            ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale,
            dropout_p=ctx.dropout_p, dropout_seed=ctx.philox_seed,
        )
        return dq, dk, dv, None, None, None, None, None, None


class _DualCoreTraced(Function):
    """``_DualCore`` for code under ``torch.compile``: the same forward and backward without the look through
    ``torch.func`` wrappers, which the tracer cannot follow (and which do not occur while it traces)."""

    forward = _DualCore.forward
    setup_context = _DualCore.setup_context

    @staticmethod
    @once_differentiable
    def backward(ctx, go, gt, _gM, _gmu):
        q, k, v, q_t, k_t, v_t, o, o_t, M, mu = ctx.saved_tensors
        want_t = any(ctx.needs_input_grad[3:6])
        dq, dk, dv, dqt, dkt, dvt = _lib.backend().bwd(
            q, k, v, q_t, k_t, v_t, o, o_t, M, mu, _dense(go), _dense(gt),
            ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale, want_tangent_grads=want_t,
            dropout_p=ctx.dropout_p, dropout_seed=ctx.philox_seed,
        )
        return dq, dk, dv, dqt, dkt, dvt, None, None, None, None, None, None


class _PlainCoreDrop(Function):
    """``_PlainCore`` with dropout for code under ``torch.compile``: the operators draw and carry the seed
    themselves (see ``_lib.py``), so the call stays inside the graph."""

    @staticmethod
    def forward(q, k, v, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p):
        o, _ot, M, _mu, seed = torch.ops.jvpfa.fwd_drop(q, k, v, None, None, None, mask_tensor, int(MASK_TYPE),
                                                        bool(causal), float(sm_scale), float(dropout_p))
        return o, M, seed

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        q, k, v, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p = inputs
        o, M, seed = outputs
        ctx.mark_non_differentiable(M, seed)
        ctx.save_for_backward(q, k, v, o, M, seed)
        ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale, ctx.dropout_p = mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p

    @staticmethod
    @once_differentiable
    def backward(ctx, go, _gM, _gseed):
        q, k, v, o, M, seed = ctx.saved_tensors
        dq, dk, dv, _, _, _ = torch.ops.jvpfa.bwd_drop(
            q, k, v, None, None, None, o, None, M, None, _dense(go), None, ctx.mask_tensor, int(ctx.MASK_TYPE),
            bool(ctx.causal), float(ctx.sm_scale), False, float(ctx.dropout_p), seed)
        return dq, dk, dv, None, None, None, None, None


class _DualCoreDrop(Function):
    """``_DualCoreTraced`` with dropout, on the operators that draw and carry the seed themselves."""

    @staticmethod
    def forward(q, k, v, q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p):
        return torch.ops.jvpfa.fwd_drop(q, k, v, q_t, k_t, v_t, mask_tensor, int(MASK_TYPE), bool(causal),
                                        float(sm_scale), float(dropout_p))

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        q, k, v, q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p = inputs
        o, o_t, M, mu, seed = outputs
        ctx.mark_non_differentiable(M, mu, seed)
        ctx.save_for_backward(q, k, v, q_t, k_t, v_t, o, o_t, M, mu, seed)
        ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale, ctx.dropout_p = mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p

    @staticmethod
    @once_differentiable
    def backward(ctx, go, gt, _gM, _gmu, _gseed):
        q, k, v, q_t, k_t, v_t, o, o_t, M, mu, seed = ctx.saved_tensors
        want_t = any(ctx.needs_input_grad[3:6])
        out = torch.ops.jvpfa.bwd_drop(
            q, k, v, q_t, k_t, v_t, o, o_t, M, mu, _dense(go), _dense(gt), ctx.mask_tensor, int(ctx.MASK_TYPE),
            bool(ctx.causal), float(ctx.sm_scale), bool(want_t), float(ctx.dropout_p), seed)
        dq, dk, dv = out[:3]
        dqt, dkt, dvt = out[3:] if want_t else (None, None, None)
        return dq, dk, dv, dqt, dkt, dvt, None, None, None, None, None


class _AttachTangent(Function):
    """Identity on O whose forward-mode tangent is the precomputed O' (the reference's trick of
    JA:2688 and JA:2828, with O' an input so that it keeps its autograd graph)."""

    @staticmethod
    def forward(o, o_t, q, k, v):
        return o.view_as(o)

    @staticmethod
    def setup_context(ctx, inputs, output):
        ctx.save_for_forward(inputs[1])

    @staticmethod
    def jvp(ctx, *_tangents):
        return ctx.saved_for_forward[0]

    @staticmethod
    def backward(ctx, g):
        return g, None, None, None, None


# Twins of the three Functions above in the older style (``forward(ctx, ...)``, no ``setup_context``).
# ``Function.apply`` binds the arguments of a ``setup_context`` Function through ``inspect.signature``
# on every call, about 25 us each; that style is only needed under ``torch.func`` transforms and
# while ``torch.compile`` traces, so ordinary eager calls take these.


class _DualCoreEager(Function):
    @staticmethod
    def forward(ctx, q, k, v, q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p=0.0, seed=0):
        o, o_t, M, mu = _lib.backend().fwd(q, k, v, q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale,
                                           dropout_p, seed)
        ctx.mark_non_differentiable(M, mu)
        ctx.save_for_backward(q, k, v, q_t, k_t, v_t, o, o_t, M, mu)
        ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale = mask_tensor, MASK_TYPE, causal, sm_scale
        ctx.dropout_p, ctx.philox_seed = dropout_p, seed
        return o, o_t, M, mu

    backward = _DualCore.backward


class _PlainCoreEager(Function):
    @staticmethod
    def forward(ctx, q, k, v, mask_tensor, MASK_TYPE, causal, sm_scale, dropout_p=0.0, seed=0):
        o, _o_t, M, _mu = _lib.backend().fwd(q, k, v, None, None, None, mask_tensor, MASK_TYPE, causal, sm_scale,
                                             dropout_p, seed)
        ctx.mark_non_differentiable(M)
        ctx.save_for_backward(q, k, v, o, M)
        ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale = mask_tensor, MASK_TYPE, causal, sm_scale
        ctx.dropout_p, ctx.philox_seed = dropout_p, seed
        return o, M

    backward = _PlainCore.backward


class _AttachTangentEager(Function):
    @staticmethod
    def forward(ctx, o, o_t, q, k, v):
        ctx.save_for_forward(o_t)
        return o.view_as(o)

    jvp = _AttachTangent.jvp
    backward = _AttachTangent.backward


def _transforms_active() -> bool:
    """A ``torch.func`` transform (jvp, vmap, grad ...) is running."""
    return torch._C._functorch.peek_interpreter_stack() is not None


class JVPAttn(Function):
    """JVP (Jacobian-Vector Product) for Attention Mechanism."""

    class Grid(NamedTuple):
        """Launch grid of the forward kernel."""

        M_BLOCKS: int
        Z_H: int
        ONE: Literal[1]

    class FnCtx(FunctionCtx):
        """Function context for JVP Attention."""

        sm_scale: float
        HEAD_DIM_K: int
        causal: bool
        grid: "JVPAttn.Grid"
        mask_tensor: Tensor
        MASK_TYPE: int
        dropout_p: float
        philox_seed: int
        ENABLE_DROPOUT: bool

    class FwdOutCtxContrib(NamedTuple):
        """Forward output context contributions for JVP Attention."""

        o_t: Tensor | None
        M: Tensor
        grid: "JVPAttn.Grid"
        HEAD_DIM_K: int
        sm_scale: float
        mask_tensor: Tensor
        MASK_TYPE: int
        dropout_p: float
        philox_seed: int
        ENABLE_DROPOUT: bool

    class FwdOut(NamedTuple):
        """Forward output for JVP Attention."""

        o: Tensor
        ctx: "JVPAttn.FwdOutCtxContrib"

    class JVPOut(NamedTuple):
        """JVP output for JVP Attention."""

        o: Tensor
        ctx: None

    class BwdOut(NamedTuple):
        """Backward output for JVP Attention."""

        q: Tensor
        k: Tensor
        v: Tensor
        q_t: None
        k_t: None
        v_t: None
        attn_mask: None
        dropout_p: None
        causal: None
        sm_scale: None
        warp_specialize: None
        USE_TMA: None
        verify_attn_mask: None

    class Strides(NamedTuple):
        """Strides for JVP Attention."""

        z: int
        h: int
        n_ctx: int
        head_dim: int

    @staticmethod
    def forward(
        q: Tensor,
        k: Tensor,
        v: Tensor,
        q_t: Tensor | None,
        k_t: Tensor | None,
        v_t: Tensor | None,
        attn_mask: Tensor | None = None,
        dropout_p: float = 0.0,
        causal: bool = False,
        sm_scale: float | None = None,
        warp_specialize: bool = True,
        USE_TMA: bool = True,
        verify_attn_mask: bool = True,
    ) -> "JVPAttn.FwdOut":
        """Forward pass (JA:2310-2647): one fused kernel gives ``o`` and, when tangents are
        passed, ``o_t``.  ``warp_specialize`` and ``USE_TMA`` are accepted and ignored (they
        select NVIDIA-specific code in the reference)."""
        _validate(q, k, v, attn_mask, dropout_p, causal)
        Z, H, N_CTX, HEAD_DIM_K = q.shape
        if sm_scale is None:
            sm_scale = HEAD_DIM_K**-0.5
        mask_tensor, MASK_TYPE = _classify_mask(attn_mask, q, verify_attn_mask)
        ENABLE_JVP = q_t is not None
        q, k, v = _dense(_unwrap(q)), _dense(_unwrap(k)), _dense(_unwrap(v))
        if ENABLE_JVP:
            q_t = _dense(_unwrap(q_t))
            k_t = torch.zeros_like(k) if k_t is None else _dense(_unwrap(k_t))
            v_t = torch.zeros_like(v) if v_t is None else _dense(_unwrap(v_t))
        philox_seed = _new_dropout_seed(dropout_p)
        o, o_t, M, _mu = _lib.backend().fwd(q, k, v, q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale,
                                            dropout_p, philox_seed)
        grid = JVPAttn.Grid((N_CTX + BLOCK_M - 1) // BLOCK_M, Z * H, 1)
        return JVPAttn.FwdOut(
            o,
            JVPAttn.FwdOutCtxContrib(o_t, M, grid, HEAD_DIM_K, sm_scale, mask_tensor, MASK_TYPE, dropout_p, philox_seed,
                                     dropout_p > 0.0),
        )

    @staticmethod
    def setup_context(ctx: "JVPAttn.FnCtx", inputs, outputs: "JVPAttn.FwdOut") -> None:
        """JA:2649-2698."""
        q, k, v, _q_t, _k_t, _v_t, _mask, _dropout_p, causal, _scale, _ws, _tma, _verify = inputs
        o, (o_t, M, grid, HEAD_DIM_K, sm_scale, mask_tensor, MASK_TYPE, dropout_p, philox_seed, ENABLE_DROPOUT) = outputs
        ctx.grid = grid
        ctx.save_for_forward(o_t)
        ctx.save_for_backward(q, k, v, o, M)
        ctx.sm_scale = sm_scale
        ctx.HEAD_DIM_K = HEAD_DIM_K
        ctx.causal = causal
        ctx.mask_tensor = mask_tensor
        ctx.MASK_TYPE = MASK_TYPE
        ctx.dropout_p = dropout_p
        ctx.philox_seed = philox_seed
        ctx.ENABLE_DROPOUT = ENABLE_DROPOUT

    @staticmethod
    def fwd(
        q: Tensor,
        k: Tensor,
        v: Tensor,
        attn_mask: Tensor | None = None,
        dropout_p: float = 0.0,
        causal: bool = False,
        sm_scale: float | None = None,
        warp_specialize: bool = True,
        USE_TMA: bool = True,
    ) -> Tensor:
        """Plain attention forward, differentiable in q, k, v (JA:2700-2752)."""
        if not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
            q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        if torch.compiler.is_compiling():
            # the same computation through a Function the tracer can follow (no custom jvp, no
            # data-dependent mask checks); the kernels appear in the graph as jvpfa::fwd / jvpfa::bwd, with
            # dropout as jvpfa::fwd_drop / jvpfa::bwd_drop, which draw and carry the seed themselves
            _validate(q, k, v, attn_mask, dropout_p, causal)
            scale = q.shape[-1] ** -0.5 if sm_scale is None else sm_scale
            mask_tensor, MASK_TYPE = _classify_mask(attn_mask, q, False)
            if dropout_p > 0.0:
                o, _M, _seed = _PlainCoreDrop.apply(q, k, v, mask_tensor, MASK_TYPE, causal, scale, dropout_p)
                return o
            o, _M = _PlainCore.apply(q, k, v, mask_tensor, MASK_TYPE, causal, scale, 0.0, 0)
            return o
        if fwAD._current_level < 0 and not _transforms_active():
            # no forward-mode level anywhere: nothing can ask for a tangent, so the plain Function
            # (same kernels, same backward) stands in for JVPAttn.apply and its per-call set-up
            _validate(q, k, v, attn_mask, dropout_p, causal)
            scale = q.shape[-1] ** -0.5 if sm_scale is None else sm_scale
            mask_tensor, MASK_TYPE = _classify_mask(attn_mask, q, True)
            o, _M = _PlainCoreEager.apply(q, k, v, mask_tensor, MASK_TYPE, causal, scale, dropout_p,
                                          _new_dropout_seed(dropout_p))
            return o
        out: JVPAttn.FwdOut = JVPAttn.apply(
            q, k, v, None, None, None, attn_mask, dropout_p, causal, sm_scale, warp_specialize, USE_TMA
        )
        a, _ = out
        return a

    @staticmethod
    def fwd_dual(
        q: Tensor,
        k: Tensor,
        v: Tensor,
        attn_mask: Tensor | None = None,
        dropout_p: float = 0.0,
        causal: bool = False,
        sm_scale: float | None = None,
        warp_specialize: bool = True,
        USE_TMA: bool = True,
    ) -> Tensor:
        """Attention on dual tensors (JA:2754-2813): inside ``fwAD.dual_level()`` or
        ``torch.func.jvp`` the result is a dual tensor whose tangent is O', computed by the same
        kernel pass as O.  Both O and O' are differentiable (reverse mode) in q, k, v and in the
        input tangents."""
        if torch.compiler.is_compiling():
            # (without a forward-mode level no tangent can exist: the plain path below)
            if fwAD._current_level >= 0:
                # The tracer follows forward-mode levels and dual tensors, but not a Function with a custom jvp:
                # the tangents are taken off the inputs, O and O' come from the Function that is differentiable
                # in all six (the kernels enter the graph as jvpfa::fwd / jvpfa::bwd), and O' is put back on O.
                q_p, q_t = fwAD.unpack_dual(q)
                k_p, k_t = fwAD.unpack_dual(k)
                v_p, v_t = fwAD.unpack_dual(v)
                if q_t is not None or k_t is not None or v_t is not None:
                    q_p, k_p, v_p = _dense(q_p), _dense(k_p), _dense(v_p)
                    _validate(q_p, k_p, v_p, attn_mask, dropout_p, causal)
                    scale = q_p.shape[-1] ** -0.5 if sm_scale is None else sm_scale
                    mask_tensor, MASK_TYPE = _classify_mask(attn_mask, q_p, False)
                    q_t = torch.zeros_like(q_p) if q_t is None else _dense(q_t)
                    k_t = torch.zeros_like(k_p) if k_t is None else _dense(k_t)
                    v_t = torch.zeros_like(v_p) if v_t is None else _dense(v_t)
                    if dropout_p > 0.0:
                        o, o_t, _M, _mu, _seed = _DualCoreDrop.apply(q_p, k_p, v_p, q_t, k_t, v_t, mask_tensor,
                                                                     MASK_TYPE, causal, scale, dropout_p)
                    else:
                        o, o_t, _M, _mu = _DualCoreTraced.apply(q_p, k_p, v_p, q_t, k_t, v_t, mask_tensor, MASK_TYPE,
                                                                causal, scale, 0.0, 0)
                    return fwAD.make_dual(o, o_t)
            return JVPAttn.fwd(q, k, v, attn_mask, dropout_p, causal, sm_scale, warp_specialize, USE_TMA)
        if not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
            q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        q_p, q_t = fwAD.unpack_dual(q)
        k_p, k_t = fwAD.unpack_dual(k)
        v_p, v_t = fwAD.unpack_dual(v)
        if q_t is None and k_t is None and v_t is None:
            return JVPAttn.fwd(q, k, v, attn_mask, dropout_p, causal, sm_scale, warp_specialize, USE_TMA)

        _validate(q_p, k_p, v_p, attn_mask, dropout_p, causal)
        if sm_scale is None:
            sm_scale = q_p.shape[-1] ** -0.5
        mask_tensor, MASK_TYPE = _classify_mask(attn_mask, q_p, True)
        q_t = torch.zeros_like(q_p) if q_t is None else _dense(q_t)
        k_t = torch.zeros_like(k_p) if k_t is None else _dense(k_t)
        v_t = torch.zeros_like(v_p) if v_t is None else _dense(v_t)
        core, attach = (_DualCore, _AttachTangent) if _transforms_active() else (_DualCoreEager, _AttachTangentEager)
        o, o_t, _M, _mu = core.apply(
            _dense(q_p), _dense(k_p), _dense(v_p), q_t, k_t, v_t, mask_tensor, MASK_TYPE, causal, sm_scale,
            dropout_p, _new_dropout_seed(dropout_p),
        )
        # NOTE: q, k, v are passed as dual tensors so that autograd calls jvp(), which hands back O'.
        return attach.apply(o, o_t, q, k, v)

    @staticmethod
    def jvp(ctx: "JVPAttn.FnCtx", gq: Tensor, gk: Tensor, gv: Tensor, *_) -> "JVPAttn.JVPOut":
        """JA:2815-2828: the tangent was computed in forward(); hand it back."""
        return JVPAttn.JVPOut(ctx.saved_for_forward[0], None)

    @staticmethod
    @once_differentiable
    def backward(ctx, do, _) -> "JVPAttn.BwdOut":
        """First-order backward from the gradient of ``o`` (JA:2830-2978)."""
        q, k, v, o, M = (_unwrap(t) for t in ctx.saved_tensors)
        if not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous() and o.is_contiguous()):
            raise ValueError(
                "JVPAttn expected q, k, v, o to be contiguous; got "
                f"q.is_contiguous()={q.is_contiguous()}, k.is_contiguous()={k.is_contiguous()}, "
                f"v.is_contiguous()={v.is_contiguous()}, o.is_contiguous()={o.is_contiguous()}, "
                f"do.is_contiguous()={do.is_contiguous()}"
            )
        do = _dense(_unwrap(do))
        dq, dk, dv, _, _, _ = _lib.backend().bwd(
            q, k, v, None, None, None, o, None, M, None, do, None,
            ctx.mask_tensor, ctx.MASK_TYPE, ctx.causal, ctx.sm_scale,
            dropout_p=ctx.dropout_p, dropout_seed=ctx.philox_seed,
        )
        return JVPAttn.BwdOut(dq, dk, dv, None, None, None, None, None, None, None, None, None, None)


def attention(
    q: Tensor,
    k: Tensor,
    v: Tensor,
    attn_mask: Tensor | None = None,
    dropout_p: float = 0.0,
    causal: bool = False,
    sm_scale: float | None = None,
    warp_specialize: bool = True,
    USE_TMA: bool = True,
) -> Tensor:
    """The reference's ``attention`` (JA:2981, an alias of ``JVPAttn.fwd``), except that dual inputs are
    noticed: inside ``fwAD.dual_level()`` or ``torch.func.jvp`` the tangent O' is propagated, which in
    the reference needs an explicit ``JVPAttn.fwd_dual`` call (its README.md:65-67).  Without tangents
    this is exactly ``JVPAttn.fwd``."""
    return JVPAttn.fwd_dual(q, k, v, attn_mask, dropout_p, causal, sm_scale, warp_specialize, USE_TMA)

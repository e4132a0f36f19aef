"""ctypes binding of ``libjvpfa.so`` (the C ABI declared in ``include/jvpfa.h``).

The library is loaded after ``import torch`` so that the HIP runtime torch already mapped is the
one the kernels launch on.  There is no fallback: if the library is missing, or a tensor is not
on a GPU, the call raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Tuple

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libjvpfa.so")

ABI_VERSION = 8
DTYPES = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
MASK_NONE, MASK_BOOL, MASK_ADD = 0, 1, 2
EXPORTS = ("jvpfa_fwd", "jvpfa_bwd", "jvpfa_fwd_split_workspace_bytes", "jvpfa_dropout_keep", "jvpfa_bwd_workspace_bytes", "jvpfa_bwd_static", "jvpfa_bwd_static_max_rows", "jvpfa_mask_tiles", "jvpfa_mask_tiles_bytes",
           "jvpfa_mask_bits", "jvpfa_mask_bits_bytes",
           "jvpfa_abi_version", "jvpfa_error_string")


class Problem(C.Structure):
    _fields_ = [
        ("Z", C.c_int32), ("H", C.c_int32), ("L", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32), ("causal", C.c_int32), ("mask_kind", C.c_int32),
        ("sm_scale", C.c_float),
        ("mask", C.c_void_p),
        ("mask_stride", C.c_int64 * 4),
        ("dropout_p", C.c_float),
        ("dropout_seed", C.c_uint64),
    ]


class FwdArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("p", Problem),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
        ("qt", C.c_void_p), ("kt", C.c_void_p), ("vt", C.c_void_p),
        ("o", C.c_void_p), ("ot", C.c_void_p),
        ("M", C.c_void_p), ("mu", C.c_void_p),
        ("key_limit", C.c_void_p),
        ("tiles_q", C.c_void_p),
        ("Lk", C.c_int32), ("Hk", C.c_int32),
        ("split_workspace", C.c_void_p), ("split_workspace_bytes", C.c_uint64),
    ]


class BwdArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("p", Problem),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
        ("qt", C.c_void_p), ("kt", C.c_void_p), ("vt", C.c_void_p),
        ("o", C.c_void_p), ("ot", C.c_void_p),
        ("M", C.c_void_p), ("mu", C.c_void_p),
        ("go", C.c_void_p), ("gt", C.c_void_p),
        ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("dqt", C.c_void_p), ("dkt", C.c_void_p), ("dvt", C.c_void_p),
        ("workspace", C.c_void_p),
        ("key_limit", C.c_void_p),
        ("tiles_q", C.c_void_p), ("tiles_k", C.c_void_p),
        ("Lk", C.c_int32), ("Hk", C.c_int32),
        ("mask_bits", C.c_void_p),
    ]


_lib = None


def load() -> C.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m jvp_flash_attention_amd.build` "
                "(there is no non-HIP fallback)"
            )
        lib = C.CDLL(LIB_PATH)
        lib.jvpfa_fwd.argtypes = [C.POINTER(FwdArgs), C.c_void_p]
        lib.jvpfa_fwd.restype = C.c_int
        lib.jvpfa_bwd.argtypes = [C.POINTER(BwdArgs), C.c_void_p]
        lib.jvpfa_bwd.restype = C.c_int
        lib.jvpfa_bwd_workspace_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32]
        lib.jvpfa_bwd_workspace_bytes.restype = C.c_size_t
        lib.jvpfa_bwd_static.argtypes = [C.POINTER(BwdArgs), C.c_void_p]
        lib.jvpfa_bwd_static.restype = C.c_int
        lib.jvpfa_bwd_static_max_rows.argtypes = []
        lib.jvpfa_bwd_static_max_rows.restype = C.c_size_t
        lib.jvpfa_fwd_split_workspace_bytes.argtypes = [C.POINTER(Problem), C.c_int32]
        lib.jvpfa_fwd_split_workspace_bytes.restype = C.c_size_t
        lib.jvpfa_dropout_keep.argtypes = [C.POINTER(Problem), C.c_int32, C.c_void_p, C.c_void_p]
        lib.jvpfa_dropout_keep.restype = C.c_int
        lib.jvpfa_mask_tiles_bytes.argtypes = [C.POINTER(Problem), C.c_int32, C.c_int32]
        lib.jvpfa_mask_tiles_bytes.restype = C.c_size_t
        lib.jvpfa_mask_tiles.argtypes = [C.POINTER(Problem), C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.jvpfa_mask_tiles.restype = C.c_int
        lib.jvpfa_mask_bits_bytes.argtypes = [C.POINTER(Problem), C.c_int32]
        lib.jvpfa_mask_bits_bytes.restype = C.c_size_t
        lib.jvpfa_mask_bits.argtypes = [C.POINTER(Problem), C.c_int32, C.c_void_p, C.c_void_p]
        lib.jvpfa_mask_bits.restype = C.c_int
        lib.jvpfa_abi_version.argtypes = []
        lib.jvpfa_abi_version.restype = C.c_int
        lib.jvpfa_error_string.argtypes = [C.c_int]
        lib.jvpfa_error_string.restype = C.c_char_p
        if lib.jvpfa_abi_version() != ABI_VERSION:
            raise RuntimeError("libjvpfa.so ABI version mismatch; rebuild the library")
        _lib = lib
    return _lib


def check(status: int) -> None:
    if status != 0:
        msg = load().jvpfa_error_string(status).decode()
        raise RuntimeError(f"libjvpfa: {msg} (status {status})")


def _ptr(t):
    return None if t is None else t.data_ptr()


def make_problem(q, mask, mask_kind, causal, sm_scale, dropout_p=0.0, dropout_seed=0) -> Problem:
    Z, H, L, D = q.shape
    p = Problem()
    p.dropout_p, p.dropout_seed = float(dropout_p), int(dropout_seed) & (2**64 - 1)
    p.Z, p.H, p.L, p.D = Z, H, L, D
    p.dtype = DTYPES[q.dtype]
    p.causal = int(bool(causal))
    p.mask_kind = mask_kind
    p.sm_scale = float(sm_scale)
    if mask_kind != MASK_NONE:
        p.mask = mask.data_ptr()
        # a size-1 axis broadcasts, whatever stride torch reports for it
        strides = [0 if mask.shape[i] == 1 else mask.stride(i) for i in range(4)]
        p.mask_stride = (C.c_int64 * 4)(*strides)
    else:
        p.mask = None
        p.mask_stride = (C.c_int64 * 4)(0, 0, 0, 0)
    return p


def mask_version(mask):
    """The version counter of a mask tensor, or None when it has none (tensors created under
    ``torch.inference_mode()`` do not track versions): None means "do not cache, look again"."""
    try:
        return mask._version
    except RuntimeError:
        return None


def forget_mask(mask) -> None:
    """Drop what has been remembered about a mask tensor (verification, key limit, tile lists).  The caches
    are keyed by the tensor's version counter, which ordinary in-place operations bump; writes that bypass it
    (``mask.data``, a custom kernel writing through ``data_ptr()``, a dlpack / numpy alias) do not, and after
    such a write this must be called before the mask is used again."""
    for name in ("_jvpfa_verified", "_jvpfa_key_limit", "_jvpfa_tiles", "_jvpfa_bits"):
        try:
            delattr(mask, name)
        except AttributeError:
            pass


KEY_LIMIT_MIN_L = 512  # below this the two small reductions cost more than the skipped tiles save


def key_limit_hint(mask, mask_kind, Z, L):
    """For a key-padding mask (one row of L keys per batch entry, shared by heads and queries): the
    index after the last key that is not masked, per batch entry, as Z int32 values on the mask's
    device; None for any other mask.  The kernels skip the key tiles past it.  Cached on the mask
    tensor so that the backward reuses what the forward computed."""
    if mask is None or mask_kind == MASK_NONE or L < KEY_LIMIT_MIN_L:
        return None
    if mask.dim() != 4 or mask.shape[1] != 1 or mask.shape[2] != 1 or mask.shape[3] != L:
        return None
    version = mask_version(mask)
    cached = getattr(mask, "_jvpfa_key_limit", None)
    if cached is not None and version is not None and cached[0] == version:
        lim = cached[1]
    else:
        alive = mask if mask.dtype == torch.bool else mask > float("-inf")
        idx = torch.arange(1, L + 1, device=mask.device, dtype=torch.int32)
        lim = (alive.view(mask.shape[0], L) * idx).amax(dim=1).to(torch.int32)  # one value per row of the mask
        if version is not None:
            try:
                mask._jvpfa_key_limit = (version, lim)
            except (AttributeError, RuntimeError):
                pass
    # the kernels index the limits by batch entry: a mask shared by the batch ([1,1,1,L]) is spread over Z
    return lim if lim.shape[0] == Z else lim.expand(Z).contiguous()


_split_enabled = True


def set_split(enabled: bool) -> None:
    """Switch the split of small launches over several workgroups per block on or off (default on): with it a
    launch that would leave most compute units idle (one sequence, few heads) hands the library a workspace for
    partial results, see ``split_workspace`` in ``include/jvpfa.h``."""
    global _split_enabled
    _split_enabled = bool(enabled)


TILE_LISTS_MIN_L = 512  # below this a mask has too few tiles for skipping some to pay for the scan
_tile_lists_enabled = True
_tile_lists_additive = False


def set_tile_lists(enabled: bool, additive: bool | None = None) -> None:
    """Switch the scan of two-dimensional masks for skippable tiles on or off (default: on for
    boolean masks, off for additive ones).  An additive mask only has skippable tiles where it holds
    -inf over a whole tile; a learned bias never does and the scan would read it for nothing, so
    additive masks are scanned only after ``set_tile_lists(True, additive=True)``."""
    global _tile_lists_enabled, _tile_lists_additive
    _tile_lists_enabled = bool(enabled)
    if additive is not None:
        _tile_lists_additive = bool(additive)


def tile_lists(q, mask, mask_kind, want_k, Lk=None):
    """For a mask with a row per query (shape [*, *, L, Lk]): the lists of 64-wide tiles that hold an
    attended entry, made on the device by ``jvpfa_mask_tiles`` -- (tiles_q, tiles_k) int32 tensors,
    tiles_k only if ``want_k`` (the backward).  The kernels visit the listed tiles only, so block
    diagonal, banded or doubly padded masks cost time in proportion to their attended area.
    (None, None) for masks that are not two-dimensional and for short sequences.  Cached on the mask
    tensor, keyed by its version counter, so that layers and the backward reuse one scan."""
    Z, H, L, D = q.shape
    Lk = L if Lk is None else Lk
    if not _tile_lists_enabled or mask is None or mask_kind == MASK_NONE or max(L, Lk) < TILE_LISTS_MIN_L:
        return None, None
    if mask.dim() != 4 or mask.shape[2] != L or mask.shape[3] != Lk:
        return None, None
    if mask_kind == MASK_ADD and not _tile_lists_additive:
        return None, None
    version = mask_version(mask)
    cached = getattr(mask, "_jvpfa_tiles", None)
    if cached is None or version is None or cached[0] != version:
        cached = [version, None, None]
    tq, tk = cached[1], cached[2]
    if tq is None or (want_k and tk is None):
        lib = load()
        prob = make_problem(q, mask, mask_kind, False, 1.0)
        new_q = new_k = None
        if tq is None:
            new_q = torch.empty(lib.jvpfa_mask_tiles_bytes(C.byref(prob), Lk, 0) // 4, device=q.device, dtype=torch.int32)
        if want_k and tk is None:
            new_k = torch.empty(lib.jvpfa_mask_tiles_bytes(C.byref(prob), Lk, 1) // 4, device=q.device, dtype=torch.int32)
        check(lib.jvpfa_mask_tiles(C.byref(prob), Lk, _ptr(new_q), _ptr(new_k), _stream(q)))
        tq = new_q if tq is None else tq
        tk = new_k if new_k is not None else tk
        cached[1], cached[2] = tq, tk
        if version is not None:
            try:
                mask._jvpfa_tiles = cached
            except (AttributeError, RuntimeError):
                pass
    return tq, (tk if want_k else None)


MASK_BITS_MIN_L = 512  # below this the backward is too short for the packed copy to pay for its pass over the mask
_mask_bits_enabled = True


def set_mask_bits(enabled: bool) -> None:
    """Switch the bit-packed copy of boolean masks for the dk/dv kernels on or off (default on)."""
    global _mask_bits_enabled
    _mask_bits_enabled = bool(enabled)


def mask_bits(q, mask, mask_kind, Lk=None):
    """For a boolean mask with a row per query (shape [*, *, L, Lk]) and a 16-bit element type at D <= 128: the
    mask packed along the query axis by ``jvpfa_mask_bits`` (a pair of uint32 per 64 queries and key; an eighth of
    the broadcast mask's bytes), which the dk/dv kernels read instead of one byte per entry.  None otherwise.  Cached
    on the mask tensor, keyed by its version counter, like the tile lists."""
    Z, H, L, D = q.shape
    Lk = L if Lk is None else Lk
    if not _mask_bits_enabled or mask is None or mask_kind != MASK_BOOL or max(L, Lk) < MASK_BITS_MIN_L:
        return None
    if mask.dim() != 4 or mask.shape[2] != L or mask.shape[3] != Lk or q.element_size() != 2 or D > 128:
        return None
    version = mask_version(mask)
    cached = getattr(mask, "_jvpfa_bits", None)
    if cached is not None and version is not None and cached[0] == version:
        return cached[1]
    lib = load()
    prob = make_problem(q, mask, mask_kind, False, 1.0)
    bits = torch.empty(lib.jvpfa_mask_bits_bytes(C.byref(prob), Lk) // 4, device=q.device, dtype=torch.int32)
    check(lib.jvpfa_mask_bits(C.byref(prob), Lk, _ptr(bits), _stream(q)))
    if version is not None:
        try:
            mask._jvpfa_bits = (version, bits)
        except (AttributeError, RuntimeError):
            pass
    return bits


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "jvp_flash_attention_amd runs on an AMD GPU only (HIP kernels); got a tensor on "
                f"{t.device}.  There is no CPU path."
            )


def _stream(t) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


# The reference admits a head dim of 16 (jvp_flash_attention/jvp_attention.py:2371-2374); the matrix instructions
# here contract over 16 and produce 32 columns, so the kernels start at 32 and a head dim of 16 runs on them with
# zero columns appended (one copy of each operand per call).
PADDED_HEAD_DIM = 16


def _pad_head_dim(t):
    return None if t is None else torch.nn.functional.pad(t, (0, 32 - PADDED_HEAD_DIM))


def _cut_head_dim(t):
    return None if t is None else t[..., :PADDED_HEAD_DIM].contiguous()


class HipBackend:
    """Device work of the forward and the backward, through the C ABI.

    ``fwd`` / ``bwd`` call the library directly.  While ``torch.compile`` traces, they go through
    the registered operators ``jvpfa::fwd`` / ``jvpfa::bwd`` instead (same code behind them), which
    the tracer records as opaque nodes with known output shapes rather than following into ctypes."""

    name = "hip"

    def fwd(self, q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p=0.0, dropout_seed=0):
        """Returns (o, ot, M, mu); ot and mu are None for a plain forward."""
        if torch.compiler.is_compiling():
            o, ot, M, mu = torch.ops.jvpfa.fwd(q, k, v, qt, kt, vt, mask, int(mask_kind), bool(causal), float(sm_scale),
                                               float(dropout_p), int(dropout_seed))
            return (o, ot, M, mu) if qt is not None else (o, None, M, None)
        return self._fwd(q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p, dropout_seed)

    def bwd(self, q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale,
            want_tangent_grads=False, dropout_p=0.0, dropout_seed=0):
        """Returns (dq, dk, dv, dqt, dkt, dvt); the last three are None unless requested."""
        if torch.compiler.is_compiling():
            out = torch.ops.jvpfa.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, int(mask_kind), bool(causal),
                                      float(sm_scale), bool(want_tangent_grads), float(dropout_p), int(dropout_seed))
            return tuple(out) if want_tangent_grads else (*out[:3], None, None, None)
        return self._bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale,
                         want_tangent_grads, dropout_p, dropout_seed)

    def _fwd(self, q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p=0.0, dropout_seed=0):
        _require_gpu(q, k, v, qt, kt, vt, mask)
        if q.shape[-1] == PADDED_HEAD_DIM:
            # zero columns change neither Q K^T nor the columns of P V that are kept
            o, ot, M, mu = self._fwd(*map(_pad_head_dim, (q, k, v, qt, kt, vt)), mask, mask_kind, causal, sm_scale,
                                     dropout_p, dropout_seed)
            return _cut_head_dim(o), _cut_head_dim(ot), M, mu
        lib = load()
        dual = qt is not None
        o = torch.empty_like(q)
        ot = torch.empty_like(q) if dual else None
        Z, H, L, _ = q.shape
        M = torch.empty((Z, H, L), device=q.device, dtype=torch.float32)
        mu = torch.empty((Z, H, L), device=q.device, dtype=torch.float32) if dual else None
        a = FwdArgs()
        a.struct_size = C.sizeof(FwdArgs)
        a.p = make_problem(q, mask, mask_kind, causal, sm_scale, dropout_p, dropout_seed)
        a.q, a.k, a.v = _ptr(q), _ptr(k), _ptr(v)
        a.qt, a.kt, a.vt = _ptr(qt), _ptr(kt), _ptr(vt)
        a.o, a.ot, a.M, a.mu = _ptr(o), _ptr(ot), _ptr(M), _ptr(mu)
        a.Hk, a.Lk = k.shape[1], k.shape[2]  # key/value heads and length (may differ from q's)
        with torch.cuda.device(q.device):
            lim = key_limit_hint(mask, mask_kind, Z, k.shape[2])
            a.key_limit = _ptr(lim)
            tq, _ = tile_lists(q, mask, mask_kind, False, k.shape[2])
            a.tiles_q = _ptr(tq)
            nsplit = lib.jvpfa_fwd_split_workspace_bytes(C.byref(a.p), a.Lk) if _split_enabled else 0
            if nsplit:
                split_ws = torch.empty(nsplit, device=q.device, dtype=torch.uint8)
                a.split_workspace, a.split_workspace_bytes = split_ws.data_ptr(), nsplit
            check(lib.jvpfa_fwd(C.byref(a), _stream(q)))
        return o, ot, M, mu

    def _bwd(self, q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale,
             want_tangent_grads=False, dropout_p=0.0, dropout_seed=0):
        _require_gpu(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask)
        if q.shape[-1] == PADDED_HEAD_DIM:
            q, k, v, qt, kt, vt, o, ot, go, gt = map(_pad_head_dim, (q, k, v, qt, kt, vt, o, ot, go, gt))
            grads = self._bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale,
                              want_tangent_grads, dropout_p, dropout_seed)
            return tuple(map(_cut_head_dim, grads))
        lib = load()
        Z, H, L, _ = q.shape
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dqt = dkt = dvt = None
        if want_tangent_grads:
            dqt, dkt, dvt = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        ws = torch.empty(lib.jvpfa_bwd_workspace_bytes(Z, H, L), device=q.device, dtype=torch.uint8)
        a = BwdArgs()
        a.struct_size = C.sizeof(BwdArgs)
        a.p = make_problem(q, mask, mask_kind, causal, sm_scale, dropout_p, dropout_seed)
        a.q, a.k, a.v = _ptr(q), _ptr(k), _ptr(v)
        a.qt, a.kt, a.vt = _ptr(qt), _ptr(kt), _ptr(vt)
        a.o, a.ot, a.M, a.mu = _ptr(o), _ptr(ot), _ptr(M), _ptr(mu)
        a.go, a.gt = _ptr(go), _ptr(gt)
        a.dq, a.dk, a.dv = _ptr(dq), _ptr(dk), _ptr(dv)
        a.dqt, a.dkt, a.dvt = _ptr(dqt), _ptr(dkt), _ptr(dvt)
        a.workspace = _ptr(ws)
        a.Hk, a.Lk = k.shape[1], k.shape[2]
        with torch.cuda.device(q.device):
            lim = key_limit_hint(mask, mask_kind, Z, k.shape[2])
            a.key_limit = _ptr(lim)
            tq, tk = tile_lists(q, mask, mask_kind, True, k.shape[2])
            a.tiles_q, a.tiles_k = _ptr(tq), _ptr(tk)
            bits = mask_bits(q, mask, mask_kind, k.shape[2])
            a.mask_bits = _ptr(bits)
            check(lib.jvpfa_bwd(C.byref(a), _stream(q)))
        return dq, dk, dv, dqt, dkt, dvt


    def dropout_keep(self, q, Lk, dropout_p, dropout_seed):
        """The keep pattern (bool, shape (Z, H, L, Lk)) that a call with this dropout_p and seed applies."""
        _require_gpu(q)
        Z, H, L, _ = q.shape
        keep = torch.empty((Z, H, L, Lk), device=q.device, dtype=torch.uint8)
        prob = make_problem(q, None, MASK_NONE, False, 1.0, dropout_p, dropout_seed)
        with torch.cuda.device(q.device):
            check(load().jvpfa_dropout_keep(C.byref(prob), Lk, keep.data_ptr(), _stream(q)))
        return keep.bool()


_backend = HipBackend()
_hip = _backend  # the operators below always mean the HIP library, whatever backend() has been pointed at

_T, _OT = torch.Tensor, Optional[torch.Tensor]


@torch.library.custom_op("jvpfa::fwd", mutates_args=(), device_types="cuda")
def _op_fwd(q: _T, k: _T, v: _T, qt: _OT, kt: _OT, vt: _OT, mask: _OT, mask_kind: int, causal: bool,
            sm_scale: float, dropout_p: float = 0.0, dropout_seed: int = 0) -> Tuple[_T, _T, _T, _T]:
    o, ot, M, mu = _hip._fwd(q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p, dropout_seed)
    # an operator returns tensors only: empty ones stand for the absent tangent outputs
    return o, (ot if ot is not None else q.new_empty(0)), M, (mu if mu is not None else M.new_empty(0))


@_op_fwd.register_fake
def _(q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p=0.0, dropout_seed=0):
    Z, H, L, _ = q.shape
    stat = q.new_empty((Z, H, L), dtype=torch.float32)
    if qt is None:
        return torch.empty_like(q), q.new_empty(0), stat, stat.new_empty(0)
    return torch.empty_like(q), torch.empty_like(q), stat, torch.empty_like(stat)


@torch.library.custom_op("jvpfa::bwd", mutates_args=(), device_types="cuda")
def _op_bwd(q: _T, k: _T, v: _T, qt: _OT, kt: _OT, vt: _OT, o: _T, ot: _OT, M: _T, mu: _OT, go: _OT, gt: _OT,
            mask: _OT, mask_kind: int, causal: bool, sm_scale: float,
            want_tangent_grads: bool, dropout_p: float = 0.0, dropout_seed: int = 0) -> Tuple[_T, _T, _T, _T, _T, _T]:
    g = _hip._bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale, want_tangent_grads,
                  dropout_p, dropout_seed)
    return tuple(t if t is not None else q.new_empty(0) for t in g)


@_op_bwd.register_fake
def _(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale, want_tangent_grads,
      dropout_p=0.0, dropout_seed=0):
    full = [torch.empty_like(t) for t in (q, k, v)]
    rest = [torch.empty_like(t) if want_tangent_grads else q.new_empty(0) for t in (q, k, v)]
    return (*full, *rest)


# Dropout inside a compiled graph.  The seed of a call is a host integer, and drawing it in traced code would
# end the graph, so these two operators draw it themselves: ``jvpfa::fwd_drop`` takes a fresh seed from torch's
# CPU generator (as the eager path does, so ``torch.manual_seed`` makes either repeatable) and hands it out as a
# one-element int64 CPU tensor, which the Function saves for ``jvpfa::bwd_drop``.  Tagged as seeded random
# operators, so the compiler neither merges two such calls nor drops one.
_RANDOM = (torch.Tag.nondeterministic_seeded,)


@torch.library.custom_op("jvpfa::fwd_drop", mutates_args=(), device_types="cuda", tags=_RANDOM)
def _op_fwd_drop(q: _T, k: _T, v: _T, qt: _OT, kt: _OT, vt: _OT, mask: _OT, mask_kind: int, causal: bool,
                 sm_scale: float, dropout_p: float) -> Tuple[_T, _T, _T, _T, _T]:
    seed = torch.randint(0, 2**62, (1,), dtype=torch.int64)
    o, ot, M, mu = _hip._fwd(q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p, int(seed.item()))
    return o, (ot if ot is not None else q.new_empty(0)), M, (mu if mu is not None else M.new_empty(0)), seed


@_op_fwd_drop.register_fake
def _(q, k, v, qt, kt, vt, mask, mask_kind, causal, sm_scale, dropout_p):
    Z, H, L, _ = q.shape
    stat = q.new_empty((Z, H, L), dtype=torch.float32)
    seed = torch.empty(1, dtype=torch.int64, device="cpu")
    if qt is None:
        return torch.empty_like(q), q.new_empty(0), stat, stat.new_empty(0), seed
    return torch.empty_like(q), torch.empty_like(q), stat, torch.empty_like(stat), seed


@torch.library.custom_op("jvpfa::bwd_drop", mutates_args=(), device_types="cuda")
def _op_bwd_drop(q: _T, k: _T, v: _T, qt: _OT, kt: _OT, vt: _OT, o: _T, ot: _OT, M: _T, mu: _OT, go: _OT, gt: _OT,
                 mask: _OT, mask_kind: int, causal: bool, sm_scale: float, want_tangent_grads: bool,
                 dropout_p: float, seed: _T) -> Tuple[_T, _T, _T, _T, _T, _T]:
    g = _hip._bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale, want_tangent_grads,
                  dropout_p, int(seed.item()))
    return tuple(t if t is not None else q.new_empty(0) for t in g)


@_op_bwd_drop.register_fake
def _(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, mask_kind, causal, sm_scale, want_tangent_grads, dropout_p, seed):
    full = [torch.empty_like(t) for t in (q, k, v)]
    rest = [torch.empty_like(t) if want_tangent_grads else q.new_empty(0) for t in (q, k, v)]
    return (*full, *rest)


def backend():
    return _backend

"""The C ABI without a GPU: the library loads, exports every function ``include/jvpfa.h`` declares,
its structs have the layout the ctypes binding assumes (checked against gcc compiling the header),
and argument validation returns the documented codes before any HIP call is made."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

from jvp_flash_attention_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "jvpfa.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jvpfa_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_function():
    lib = _lib.load()
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS)
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.jvpfa_abi_version() == _lib.ABI_VERSION


def test_struct_layout_matches_the_header(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "jvpfa.h"\n'
        "int main(void){\n"
        'printf("%zu %zu %zu\\n", sizeof(jvpfa_problem), sizeof(jvpfa_fwd_args), sizeof(jvpfa_bwd_args));\n'
        'printf("%zu %zu %zu %zu\\n", offsetof(jvpfa_problem, sm_scale), offsetof(jvpfa_problem, mask), '
        "offsetof(jvpfa_problem, mask_stride), offsetof(jvpfa_fwd_args, q));\n"
        'printf("%zu %zu %zu\\n", offsetof(jvpfa_fwd_args, mu), offsetof(jvpfa_bwd_args, go), offsetof(jvpfa_bwd_args, workspace));\n'
        "return 0;}\n"
    )
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    got = [int(x) for x in out]
    want = [
        C.sizeof(_lib.Problem), C.sizeof(_lib.FwdArgs), C.sizeof(_lib.BwdArgs),
        _lib.Problem.sm_scale.offset, _lib.Problem.mask.offset, _lib.Problem.mask_stride.offset, _lib.FwdArgs.q.offset,
        _lib.FwdArgs.mu.offset, _lib.BwdArgs.go.offset, _lib.BwdArgs.workspace.offset,
    ]
    assert got == want


def _fwd_args(**kw):
    a = _lib.FwdArgs()
    a.struct_size = C.sizeof(_lib.FwdArgs)
    a.p.Z, a.p.H, a.p.L, a.p.D = 1, 1, 32, 64
    a.p.dtype, a.p.causal, a.p.mask_kind, a.p.sm_scale = 0, 0, 0, 0.125
    for name in ("q", "k", "v", "o", "M"):
        setattr(a, name, 0x1000)
    for k, v in kw.items():
        if k.startswith("p_"):
            setattr(a.p, k[2:], v)
        else:
            setattr(a, k, v)
    return a


@pytest.mark.parametrize(
    "kw,code",
    [
        (dict(struct_size=4), -7),
        (dict(q=None), -1),
        (dict(p_D=48), -2),
        (dict(p_dropout_p=1.0), -2),        # dropout_p must be below 1
        (dict(p_L=0), -2),
        (dict(p_dtype=5), -3),
        (dict(p_mask_kind=1), -1),          # mask kind set, mask pointer NULL
        (dict(p_mask_kind=1, p_mask=0x1000, p_causal=1), -5),
        (dict(qt=0x1000), -1),              # tangents must come as a full set
        (dict(qt=0x1000, kt=0x1000, vt=0x1000), -1),  # dual without ot / mu
        (dict(q=0x1004), -4),
    ],
)
def test_forward_argument_validation_codes(kw, code):
    lib = _lib.load()
    assert lib.jvpfa_fwd(C.byref(_fwd_args(**kw)), None) == code
    assert lib.jvpfa_error_string(code).decode() not in ("ok", "unknown status")


def test_key_value_shape_fields_are_checked():
    lib = _lib.load()
    for kw, code in ((dict(Hk=3), -2), (dict(Hk=-1), -2), (dict(Lk=-5), -2), (dict(Hk=8), -2)):
        a = _fwd_args(p_H=4, **kw)
        assert lib.jvpfa_fwd(C.byref(a), None) == code, kw
    a = _fwd_args(p_H=4, Hk=2, Lk=77, q=None)
    assert lib.jvpfa_fwd(C.byref(a), None) == -1  # shape accepted; stops at the NULL pointer


def test_struct_size_must_be_this_library_s():
    """One size per struct: a caller built from another header is told so instead of being guessed at."""
    lib = _lib.load()
    a = _fwd_args(q=None)
    assert lib.jvpfa_fwd(C.byref(a), None) == -1  # got past the size check, to the NULL pointer check
    for size in (_lib.FwdArgs.key_limit.offset, _lib.FwdArgs.Lk.offset, C.sizeof(_lib.FwdArgs) + 8):
        a.struct_size = size
        assert lib.jvpfa_fwd(C.byref(a), None) == -7
    b = _lib.BwdArgs()
    b.p.Z, b.p.H, b.p.L, b.p.D = 1, 1, 32, 64
    b.struct_size = C.sizeof(_lib.BwdArgs)
    assert lib.jvpfa_bwd(C.byref(b), None) == -1
    b.struct_size = _lib.BwdArgs.Lk.offset
    assert lib.jvpfa_bwd(C.byref(b), None) == -7


def test_tile_lists_are_only_made_for_masks_with_a_row_per_query():
    import torch

    q = torch.empty(2, 2, 1024, 64, dtype=torch.bfloat16)
    full = torch.ones(2, 1, 1024, 1024, dtype=torch.bool)
    cases = [
        (q, torch.ones(2, 1, 1, 1024, dtype=torch.bool)),         # key padding: the key limit covers it
        (q[:, :, :256], full[:, :, :256, :256]),                   # too short to pay for the scan
        (q, full[:, :, :, :512]),                                   # not the shape of the scores (Lk = 1024)
        (q, None),
    ]
    for qq, m in cases:
        assert _lib.tile_lists(qq, m, _lib.MASK_BOOL if m is not None else _lib.MASK_NONE, True) == (None, None)
    assert _lib.tile_lists(q, full.to(torch.bfloat16), _lib.MASK_ADD, True) == (None, None)  # additive: on request only
    _lib.set_tile_lists(False)
    try:
        assert _lib.tile_lists(q, full, _lib.MASK_BOOL, True) == (None, None)
    finally:
        _lib.set_tile_lists(True)


def test_the_packed_mask_is_only_made_where_a_kernel_reads_it():
    import torch

    q = torch.empty(2, 2, 1024, 64, dtype=torch.bfloat16)
    full = torch.ones(2, 1, 1024, 1024, dtype=torch.bool)
    cases = [
        (q, torch.ones(2, 1, 1, 1024, dtype=torch.bool), _lib.MASK_BOOL),  # key padding: no row per query
        (q[:, :, :256], full[:, :, :256, :256], _lib.MASK_BOOL),            # too short to pay for the pass
        (q.float(), full, _lib.MASK_BOOL),                                   # fp32 kernels read the mask itself
        (torch.empty(2, 2, 1024, 256, dtype=torch.bfloat16), full, _lib.MASK_BOOL),  # and so do those for D = 256
        (q, full.to(torch.bfloat16), _lib.MASK_ADD),                        # additive masks have no bits
        (q, None, _lib.MASK_NONE),
    ]
    for qq, m, kind in cases:
        assert _lib.mask_bits(qq, m, kind) is None
    _lib.set_mask_bits(False)
    try:
        assert _lib.mask_bits(q, full, _lib.MASK_BOOL) is None
    finally:
        _lib.set_mask_bits(True)


def test_packed_mask_size_and_argument_checks():
    """Host-side part of jvpfa_mask_bits: buffer size and refusals (nothing is launched)."""
    lib = _lib.load()
    p = _lib.Problem()
    p.Z, p.H, p.L, p.D, p.dtype, p.mask_kind = 2, 3, 100, 64, 0, _lib.MASK_BOOL
    p.mask_stride = (C.c_int64 * 4)(0, 100 * 70, 70, 1)  # shared by the batch: 3 planes
    assert lib.jvpfa_mask_bits_bytes(C.byref(p), 70) == 3 * 2 * 70 * 8  # planes * ceil(100/64) * keys * 8 bytes
    assert lib.jvpfa_mask_bits_bytes(C.byref(p), 0) == 3 * 2 * 100 * 8
    assert lib.jvpfa_mask_bits(C.byref(p), 70, None, None) == -1            # no buffer
    assert lib.jvpfa_mask_bits(C.byref(p), 70, C.c_void_p(64), None) == -1  # no mask
    p.mask = 4096
    assert lib.jvpfa_mask_bits(C.byref(p), 70, C.c_void_p(68), None) == -4  # misaligned buffer
    p.mask_kind = _lib.MASK_ADD
    assert lib.jvpfa_mask_bits(C.byref(p), 70, C.c_void_p(64), None) == -3  # additive masks are not packed
    p.mask_kind = _lib.MASK_BOOL
    p.mask_stride = (C.c_int64 * 4)(0, 100 * 70, -70, 1)
    assert lib.jvpfa_mask_bits(C.byref(p), 70, C.c_void_p(64), None) == -2


def test_mask_tile_list_sizes_and_argument_checks():
    """Host-side part of jvpfa_mask_tiles: buffer sizes and refusals (nothing is launched)."""
    lib = _lib.load()
    p = _lib.Problem()
    p.Z, p.H, p.L, p.D = 3, 4, 700, 64
    p.dtype, p.mask_kind = 0, _lib.MASK_BOOL
    nblk, nt = 6, 11  # ceil(700/128) blocks of ceil(700/64) + 1 ints each
    for strides, planes in (((490000 * 4, 490000, 700, 1), 12), ((490000, 0, 700, 1), 3), ((0, 0, 700, 1), 1)):
        p.mask_stride = (C.c_int64 * 4)(*strides)
        assert lib.jvpfa_mask_tiles_bytes(C.byref(p), 0, 0) == planes * nblk * (nt + 1) * 4
        assert lib.jvpfa_mask_tiles_bytes(C.byref(p), 0, 1) == planes * nblk * (nt + 1) * 4
        # 200 keys: 4 key tiles per block of query rows; 2 blocks of keys with 11 query tiles each
        assert lib.jvpfa_mask_tiles_bytes(C.byref(p), 200, 0) == planes * nblk * (4 + 1) * 4
        assert lib.jvpfa_mask_tiles_bytes(C.byref(p), 200, 1) == planes * 2 * (nt + 1) * 4
    buf = (C.c_int32 * 16)()
    assert lib.jvpfa_mask_tiles(C.byref(p), 0, buf, None, None) == -1  # no mask pointer
    p.mask = C.addressof(buf)
    assert lib.jvpfa_mask_tiles(C.byref(p), 0, None, None, None) == -1  # no output at all
    assert lib.jvpfa_mask_tiles(C.byref(p), -5, buf, None, None) == -2
    p.mask_kind = _lib.MASK_NONE
    assert lib.jvpfa_mask_tiles(C.byref(p), 0, buf, None, None) == -3
    p.mask_kind, p.L = _lib.MASK_BOOL, 0
    assert lib.jvpfa_mask_tiles(C.byref(p), 0, buf, None, None) == -2
    assert lib.jvpfa_mask_tiles_bytes(C.byref(p), 0, 0) == 0
    # the backward takes both lists or none
    b = _lib.BwdArgs()
    b.struct_size = C.sizeof(_lib.BwdArgs)
    b.p.Z, b.p.H, b.p.L, b.p.D = 1, 1, 32, 64
    b.tiles_q = C.addressof(buf)
    assert lib.jvpfa_bwd(C.byref(b), None) == -1


def test_key_limit_hint_of_key_padding_masks():
    import torch

    L = _lib.KEY_LIMIT_MIN_L
    m = torch.zeros(3, 1, 1, L, dtype=torch.bool)
    m[0, ..., :100] = True
    m[1, ..., :L] = True
    m[2, ..., 5] = True  # last attended key at index 5; earlier ones masked: still a valid limit
    assert _lib.key_limit_hint(m, _lib.MASK_BOOL, 3, L).tolist() == [100, L, 6]
    assert m._jvpfa_key_limit[1].tolist() == [100, L, 6]  # cached for the backward
    m[0, ..., 200] = True  # an in-place change invalidates the cache
    assert _lib.key_limit_hint(m, _lib.MASK_BOOL, 3, L).tolist() == [201, L, 6]
    one = torch.ones(1, 1, 1, L, dtype=torch.bool)
    one[..., L // 2:] = False
    assert _lib.key_limit_hint(one, _lib.MASK_BOOL, 4, L).tolist() == [L // 2] * 4  # broadcast over the batch
    bias = torch.zeros(2, 1, 1, L)
    bias[0, ..., 300:] = float("-inf")
    assert _lib.key_limit_hint(bias, _lib.MASK_ADD, 2, L).tolist() == [300, L]
    # anything that is not one row of keys per batch entry gives no hint; neither do short sequences
    assert _lib.key_limit_hint(torch.ones(2, 1, L, L, dtype=torch.bool), _lib.MASK_BOOL, 2, L) is None
    assert _lib.key_limit_hint(torch.ones(2, 1, 1, 64, dtype=torch.bool), _lib.MASK_BOOL, 2, 64) is None
    assert _lib.key_limit_hint(None, _lib.MASK_NONE, 2, L) is None


def test_backward_argument_validation_codes():
    lib = _lib.load()
    a = _lib.BwdArgs()
    a.struct_size = C.sizeof(_lib.BwdArgs)
    a.p.Z, a.p.H, a.p.L, a.p.D = 1, 1, 32, 64
    a.p.sm_scale = 0.125
    assert lib.jvpfa_bwd(C.byref(a), None) == -1
    for name in ("q", "k", "v", "o", "M", "dq", "dk", "dv", "workspace"):
        setattr(a, name, 0x1000)
    assert lib.jvpfa_bwd(C.byref(a), None) == -1  # neither go nor gt
    a.gt = 0x1000
    assert lib.jvpfa_bwd(C.byref(a), None) == -1  # gt needs the tangent tensors, ot and mu
    a.gt = None
    a.go = 0x1000
    a.dqt = 0x1000
    assert lib.jvpfa_bwd(C.byref(a), None) == -1  # tangent gradients need gt (and all three)
    a.dqt = None
    a.struct_size = 8
    assert lib.jvpfa_bwd(C.byref(a), None) == -7
    assert lib.jvpfa_bwd(None, None) == -1
    assert lib.jvpfa_bwd_workspace_bytes(2, 3, 5) == 3 * 32 * 4  # 30 rows padded to 32 floats per statistic
    assert lib.jvpfa_bwd_workspace_bytes(0, 3, 5) == 0


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libjvpfa.so")
    with pytest.raises(RuntimeError, match="no non-HIP fallback"):
        _lib.load()


def test_product_does_not_import_the_oracle():
    code = "import sys, jvp_flash_attention_amd; sys.exit(1 if any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules) else 0)"
    assert subprocess.run([sys.executable, "-c", code], cwd=ROOT).returncode == 0
    for dirpath, _, files in os.walk(os.path.join(ROOT, "jvp_flash_attention_amd")):
        for f in files:
            if f.endswith(".py"):
                assert "oracle" not in open(os.path.join(dirpath, f)).read().replace("oracle_backend", "")

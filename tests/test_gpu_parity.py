"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle.

Tolerances (the stated target): fp32 max-abs <= 1e-4; bf16 / fp16 relative error
``max|x - ref| / max|ref| <= 2e-2``.  The oracle is the dense fp64 closed form evaluated on the
same, already rounded, inputs (it is itself pinned against PyTorch's math SDPA under
``torch.func.jvp`` in ``test_oracle.py``).
"""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import dense

pytestmark = pytest.mark.gpu

DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def _tol_check(name, got, ref, dtype, floor=1e-30):
    got = got.detach().double().cpu().numpy()
    assert np.isfinite(got).all(), f"{name}: non-finite values"
    err = np.abs(got - ref).max()
    if dtype == torch.float32:
        assert err <= 1e-4, f"{name}: max-abs {err:.3e} > 1e-4"
    elif np.abs(ref).max() == 0.0:
        # a quantity that is exactly zero (every row attends a single key, so dS cancels): the 16-bit kernels
        # return the rounding residue of the stored O, O', held to the absolute bound of test_single_key
        assert err <= 5e-2, f"{name}: max-abs {err:.3e} > 5e-2 where the exact value is 0"
    else:
        rel = err / max(np.abs(ref).max(), floor)
        assert rel <= 2e-2, f"{name}: relative {rel:.3e} > 2e-2"


def _make(Z, H, L, D, dtype, seed, tangent_std=1.0):
    g = torch.Generator().manual_seed(seed)
    t = [torch.randn(Z, H, L, D, generator=g) for _ in range(8)]
    for i in (3, 4, 5):
        t[i] = t[i] * tangent_std
    return [x.to(dtype) for x in t]


def _mask(mode, Z, H, L, dtype, seed=1):
    g = torch.Generator().manual_seed(seed)
    if mode in ("none", "causal"):
        return None
    if mode == "keypad":  # benchmark configuration 4(a): per-batch valid length uniform in [L/2, L]
        lens = torch.randint(L // 2, L + 1, (Z,), generator=g)
        return (torch.arange(L)[None, :] < lens[:, None]).view(Z, 1, 1, L)
    if mode == "bias":  # benchmark configuration 4(b)
        return torch.randn(Z, H, L, L, generator=g).to(dtype)
    if mode == "bool_full":  # the reference's test masks: random, keep-probability 0.1 (test file :334-363)
        m = torch.rand(Z, H, L, L, generator=g) > 0.9
        m[..., 0] = True
        return m
    if mode == "bias_bcast":
        return torch.randn(1, H, L, L, generator=g).to(dtype)
    raise ValueError(mode)


def _run_case(Z, H, L, D, dtype, mode, seed=0, tangent_std=1.0, plain=False, tangent_grads=True, causal=None):
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    q, k, v, qt, kt, vt, go, gt = _make(Z, H, L, D, dtype, seed, tangent_std)
    mask = _mask(mode, Z, H, L, dtype)
    causal = (mode == "causal") if causal is None else causal
    kind = _lib.MASK_NONE if mask is None else (_lib.MASK_BOOL if mask.dtype == torch.bool else _lib.MASK_ADD)
    scale = D**-0.5
    npm = None if mask is None else (mask.numpy() if mask.dtype == torch.bool else mask.double().numpy())
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    dmask = None if mask is None else mask.cuda()
    print(f"case Z{Z} H{H} L{L} D{D} {dtype} {mode} plain={plain}", flush=True)
    if plain:
        ref = dense.forward(*f64[:3], mask=npm, causal=causal, scale=scale)
        rb = dense.backward(*f64[:3], None, None, None, f64[6], None, mask=npm, causal=causal, scale=scale)
        o, ot, M, mu = be.fwd(dev[0], dev[1], dev[2], None, None, None, dmask, kind, causal, scale)
        assert ot is None and mu is None
        _tol_check("O", o, ref["O"], dtype)
        assert np.abs(M.double().cpu().numpy() - ref["M"]).max() < (1e-4 if dtype == torch.float32 else 2e-2)
        dq, dk, dv, *_ = be.bwd(dev[0], dev[1], dev[2], None, None, None, o, None, M, None, dev[6], None,
                                dmask, kind, causal, scale)
        for n, t in (("dq", dq), ("dk", dk), ("dv", dv)):
            _tol_check(n, t, rb[n], dtype)
        return
    ref = dense.forward(*f64[:6], mask=npm, causal=causal, scale=scale)
    o, ot, M, mu = be.fwd(*dev[:6], dmask, kind, causal, scale)
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    stat_tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert np.abs(M.double().cpu().numpy() - ref["M"]).max() < stat_tol
    assert np.abs(mu.double().cpu().numpy() - ref["mu"]).max() < stat_tol * max(1.0, np.abs(ref["mu"]).max())
    rb = dense.backward(*f64, mask=npm, causal=causal, scale=scale)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, kind, causal, scale,
                   want_tangent_grads=tangent_grads)
    names = ("dq", "dk", "dv", "dqt", "dkt", "dvt")
    for n, t in zip(names, grads):
        if t is not None:
            _tol_check(n, t, rb[n], dtype)
    if tangent_grads:  # the call for dq, dk, dv alone takes other kernels (small grids: both roles in one launch)
        g3 = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, kind, causal, scale)
        assert g3[3] is None and g3[4] is None and g3[5] is None
        for n, t in zip(names[:3], g3[:3]):
            _tol_check(n + "(three gradients)", t, rb[n], dtype)
    # first-order backward from gO only through the same saved state (reference's backward)
    rb1 = dense.backward(*f64[:7], None, mask=npm, causal=causal, scale=scale)
    g1 = be.bwd(dev[0], dev[1], dev[2], None, None, None, o, None, M, None, dev[6], None, dmask, kind, causal, scale)
    for n, t in zip(names[:3], g1[:3]):
        _tol_check(n + "(gO only)", t, rb1[n], dtype)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("mode", ["none", "causal"])
def test_dual_fwd_bwd_dense_and_causal(dt, D, mode):
    _run_case(2, 2, 256, D, DTYPES[dt], mode)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("mode", ["none", "causal", "keypad", "bias", "bool_full"])
def test_head_dim_256(dt, mode):
    # the largest head dim the reference admits (its jvp_attention.py:2371-2374)
    _run_case(1, 2, 200, 256, DTYPES[dt], mode, seed=17)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("mode", ["none", "causal", "keypad", "bias"])
def test_head_dim_16(dt, mode):
    """The smallest head dim the reference admits (its jvp_attention.py:2371-2374): the backend appends zero columns
    and runs the kernels for 32; outputs and all six gradients come back with 16 columns."""
    _run_case(2, 2, 100, 16, DTYPES[dt], mode, seed=31)
    if mode == "none":
        _run_case(1, 2, 70, 16, DTYPES[dt], mode, seed=32, plain=True)


@pytest.mark.parametrize("L", [65, 130, 333])
@pytest.mark.parametrize("mode", ["none", "causal", "keypad", "bool_full"])
def test_head_dim_256_lengths_across_the_64_row_workgroups(L, mode):
    """The dual backward at D = 256 runs workgroups of 64 rows (two pairs of waves that hand each other score
    tiles through LDS), the other D = 256 kernels 128 rows: lengths that end inside either kind of block."""
    _run_case(1, 2, L, 256, torch.bfloat16, mode, seed=23)


def test_head_dim_256_tiles_away_from_every_edge():
    _run_case(1, 1, 1100, 256, torch.bfloat16, "causal", seed=24)
    _run_case(1, 1, 520, 256, torch.float16, "bias", seed=25)
    _run_case(1, 1, 520, 256, torch.float16, "none", seed=26, plain=True)


@pytest.mark.parametrize("dt", ["bf16", "fp16"])
def test_head_dim_256_rows_whose_weight_sits_on_one_key(dt):
    """A batch entry padded down to a single key next to an ordinary one, 24 queries over 183 keys: every row of
    the first has all its weight on key 0, so O' = V'[0] and its gradients through the scores are exactly zero, and
    what the kernels leave there instead is measured against the other entry's gradients (the tensor's maximum).
    The second forward pass measures S' from the row's mean over its first tile for this: with S' as it stands,
    T - mu O is the difference of two sums of size |S'| |V|, one of them through 16-bit operands, and dk of the
    padded entry came out at 3e-2 of the maximum."""
    from jvp_flash_attention_amd import _lib

    Z, H, L, Lk, D = 2, 2, 24, 183, 256
    dtype = DTYPES[dt]
    g = torch.Generator().manual_seed(7098)
    q, qt, go, gt = (torch.randn(Z, H, L, D, generator=g).to(dtype) for _ in range(4))
    k, v, kt, vt = (torch.randn(Z, H, Lk, D, generator=g).to(dtype) for _ in range(4))
    lens = torch.tensor([1, 126])
    mask = (torch.arange(Lk)[None, :] < lens[:, None]).view(Z, 1, 1, Lk)
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    be, scale = _lib.backend(), D**-0.5
    print(f"case one key per row {dt} D{D}", flush=True)
    o, ot, M, mu = be.fwd(*dev[:6], mask.cuda(), _lib.MASK_BOOL, False, scale)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], mask.cuda(), _lib.MASK_BOOL, False, scale, want_tangent_grads=True)
    ref = dense.forward(*f64[:6], mask=mask.numpy(), causal=False, scale=scale)
    rb = dense.backward(*f64, mask=mask.numpy(), causal=False, scale=scale)
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    # the padded entry alone: O' is V'[0] to the rounding of the element type (no cancellation left)
    assert (ot[0].float().cpu() - vt[0, :, :1].float()).abs().max().item() <= 2.0**-7 * vt[0, :, :1].float().abs().max().item()
    assert np.abs(mu.double().cpu().numpy() - ref["mu"]).max() <= 1e-3 * max(1.0, np.abs(ref["mu"]).max())  # (mu = mu_c + c)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        _tol_check(n, t, rb[n], dtype)


def test_head_dim_256_in_fp32_plain_and_at_a_benchmark_length():
    """fp32 at D = 256 reads its own rows' fragments from global memory instead of keeping them in registers:
    the plain path, and a length with many interior tiles (causal, so that both loops' edges are crossed)."""
    _run_case(1, 2, 200, 256, torch.float32, "none", seed=18, plain=True)
    _run_case(1, 1, 1024, 256, torch.float32, "causal", seed=19)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("mode", ["keypad", "bias", "bool_full", "bias_bcast"])
def test_dual_fwd_bwd_masks(dt, mode):
    _run_case(2, 3, 192, 64, DTYPES[dt], mode)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("mode", ["keypad", "bias"])
def test_masks_d128(dt, mode):
    _run_case(2, 2, 128, 128, DTYPES[dt], mode)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("L", [2, 31, 40, 100, 130, 333])
@pytest.mark.parametrize("mode", ["none", "causal", "keypad"])
def test_ragged_lengths(dt, L, mode):
    _run_case(1, 2, L, 64, DTYPES[dt], mode)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("L", [100, 333])
@pytest.mark.parametrize("mode", ["bool_full", "bias"])
def test_dense_masks_with_unaligned_rows(dt, L, mode):
    # a row of the mask starts at a multiple of L elements: not aligned for vector fetches when L is odd-ish
    _run_case(1, 2, L, 64, DTYPES[dt], mode, seed=11)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("mode", ["bool_full", "bias", "keypad"])
def test_masks_over_several_tiles_interior_and_edge(D, mode):
    # L = 328: five key tiles, the last one ragged; aligned rows, so interior tiles take the fetch-ahead path
    _run_case(1, 2, 328, D, torch.bfloat16, mode, seed=12)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("kind", ["bool", "bias"])
def test_key_padding_with_skipped_tiles(D, kind, dt):
    """Long enough for the host to pass the key-limit hint: key tiles past the longest valid length of a
    batch entry are skipped (forward, dq) and fully padded key blocks return zero gradients (dk/dv)."""
    from jvp_flash_attention_amd import _lib

    Z, H, L = 3, 2, 640
    dtype = DTYPES[dt]
    q, k, v, qt, kt, vt, go, gt = _make(Z, H, L, D, dtype, 21)
    lens = [640, 200, 65]
    keep = torch.arange(L)[None, :] < torch.tensor(lens)[:, None]
    mask = keep.view(Z, 1, 1, L) if kind == "bool" else torch.where(keep, 0.0, float("-inf")).view(Z, 1, 1, L).to(dtype)
    mk = _lib.MASK_BOOL if kind == "bool" else _lib.MASK_ADD
    npm = keep.view(Z, 1, 1, L).numpy()
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    dmask = mask.cuda()
    be = _lib.backend()
    scale = D**-0.5
    assert _lib.key_limit_hint(dmask, mk, Z, L).tolist() == lens
    ref = dense.forward(*f64[:6], mask=npm, causal=False, scale=scale)
    o, ot, M, mu = be.fwd(*dev[:6], dmask, mk, False, scale)
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    rb = dense.backward(*f64, mask=npm, causal=False, scale=scale)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, mk, False, scale, want_tangent_grads=True)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        _tol_check(n, t, rb[n], dtype)
    assert grads[1][1, :, 256:].abs().max().item() == 0.0 and grads[2][2, :, 128:].abs().max().item() == 0.0


def _structured_keep(kind, Z, H, L, seed=5):
    """Boolean (Z or 1, H or 1, L, L) masks with whole tiles masked: the shapes that packed sequences,
    local windows and padding on both axes produce."""
    g = torch.Generator().manual_seed(seed)
    i, j = torch.arange(L)[:, None], torch.arange(L)[None, :]
    if kind == "blockdiag":  # packed sequences: segment boundaries at random places, one set per batch entry
        keep = torch.zeros(Z, 1, L, L, dtype=torch.bool)
        for z in range(Z):
            cuts = sorted({0, L, *torch.randint(1, L, (3,), generator=g).tolist()})
            seg = torch.zeros(L, dtype=torch.long)
            for n, (a, b) in enumerate(zip(cuts[:-1], cuts[1:])):
                seg[a:b] = n
            keep[z, 0] = seg[:, None] == seg[None, :]
        return keep
    if kind == "band":  # local window of 100 keys either side, shared by batch and heads
        return ((i - j).abs() <= 100).view(1, 1, L, L)
    if kind == "pad2d":  # outer product of per-batch padding vectors; padded queries attend nothing
        lens = torch.randint(L // 4, L + 1, (Z,), generator=g)
        valid = torch.arange(L)[None, :] < lens[:, None]
        return (valid[:, :, None] & valid[:, None, :]).view(Z, 1, L, L)
    if kind == "lower":  # an explicit lower-triangular mask, per head
        return (j <= i).view(1, 1, L, L).expand(1, H, L, L).contiguous()
    raise ValueError(kind)


def _numpy_tile_lists(keep, L):
    """(tiles_q, tiles_k) as lists of index lists, from a (P, L, L) boolean array."""
    nblk, nt = (L + 127) // 128, (L + 63) // 64
    tq, tk = [], []
    for pl in keep:
        for b in range(nblk):
            rows = pl[128 * b:128 * b + 128]
            tq.append([t for t in range(nt) if rows[:, 64 * t:64 * t + 64].any()] or [0])
            cols = pl[:, 128 * b:128 * b + 128]
            tk.append([t for t in range(nt) if cols[64 * t:64 * t + 64].any()] or [0])
    return tq, tk


@pytest.mark.parametrize("kind", ["blockdiag", "band", "pad2d", "lower"])
@pytest.mark.parametrize("as_bias", [False, True])
@pytest.mark.parametrize("L", [640, 700])
def test_mask_tile_lists_match_a_numpy_scan(kind, as_bias, L):
    from jvp_flash_attention_amd import _lib

    Z, H = 2, 2
    keep = _structured_keep(kind, Z, H, L)
    dtype = torch.bfloat16
    mask = torch.where(keep, 0.5, float("-inf")).to(dtype) if as_bias else keep
    mk = _lib.MASK_ADD if as_bias else _lib.MASK_BOOL
    q = torch.empty(Z, H, L, 64, dtype=dtype, device="cuda")
    _lib.set_tile_lists(True, additive=True)  # additive masks are only scanned on request
    try:
        tq, tk = _lib.tile_lists(q, mask.cuda(), mk, True)
    finally:
        _lib.set_tile_lists(True, additive=False)
    nt = (L + 63) // 64
    rq, rk = _numpy_tile_lists(keep.reshape(-1, L, L).numpy(), L)
    for got, ref in ((tq, rq), (tk, rk)):
        got = got.cpu().view(-1, nt + 1).tolist()
        assert len(got) == len(ref)
        for row, want in zip(got, ref):
            assert row[0] == len(want) and row[1:1 + row[0]] == want


def _numpy_mask_bits(keep):
    """(P, ceil(L/64), Lk, 2) uint32 from a (P, L, Lk) boolean array: bit i of word [p, t, j, hf] =
    keep[p, 64 t + 32 hf + i, j], rows past L counting as masked."""
    P, L, Lk = keep.shape
    nqt = (L + 63) // 64
    padded = np.zeros((P, nqt * 64, Lk), dtype=np.uint32)
    padded[:, :L] = keep
    weights = (np.uint32(1) << np.arange(32, dtype=np.uint32))[None, None, None, :, None]
    words = (padded.reshape(P, nqt, 2, 32, Lk) * weights).sum(axis=3, dtype=np.uint64).astype(np.uint32)
    return words.transpose(0, 1, 3, 2)


@pytest.mark.parametrize("shape", [(2, 2, 700, 700), (2, 1, 333, 515), (1, 3, 640, 1030), (1, 1, 33, 2050)])
@pytest.mark.parametrize("layout", ["dense", "offset", "strided"])
def test_the_packed_mask_matches_a_numpy_packing(shape, layout):
    """jvpfa_mask_bits against numpy: ragged row and key counts, masks shared by heads or batch, and masks whose
    rows do not start on a 4-byte boundary or whose keys are not contiguous (the loop that reads byte by byte)."""
    from jvp_flash_attention_amd import _lib

    Z, H, L, Lk = shape
    g = torch.Generator().manual_seed(L + Lk)
    keep = torch.rand(Z, H, L, Lk, generator=g) > 0.3
    keep[0, 0, 5] = False
    keep[0, 0, :, 7] = False
    if layout == "dense":
        dmask = keep.cuda()
    elif layout == "offset":  # every row starts one byte past a multiple of four
        big = torch.zeros(Z, H, L, Lk + 8 - Lk % 4, dtype=torch.bool, device="cuda")
        dmask = big[..., 1:1 + Lk]
        dmask.copy_(keep)
    else:  # keys two bytes apart
        big = torch.zeros(Z, H, L, 2 * Lk, dtype=torch.bool, device="cuda")
        dmask = big[..., ::2]
        dmask.copy_(keep)
    # a mask axis of size one is shared by the problem's batch entries / heads
    q = torch.empty(Z if Z > 1 else 2, H if H > 1 else 3, L, 64, dtype=torch.bfloat16, device="cuda")
    lib = _lib.load()
    prob = _lib.make_problem(q, dmask, _lib.MASK_BOOL, False, 1.0)
    n = lib.jvpfa_mask_bits_bytes(C.byref(prob), Lk) // 4
    assert n == Z * H * ((L + 63) // 64) * Lk * 2
    bits = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    _lib.check(lib.jvpfa_mask_bits(C.byref(prob), Lk, bits.data_ptr(), torch.cuda.current_stream().cuda_stream))
    got = bits.cpu().numpy().view(np.uint32).reshape(Z * H, -1, Lk, 2)
    assert np.array_equal(got, _numpy_mask_bits(keep.reshape(Z * H, L, Lk).numpy()))


@pytest.mark.parametrize("dt", ["bf16", "fp16"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("Lq,Lk,Hk", [(700, 700, 4), (545, 830, 2)])
def test_the_packed_mask_changes_no_bit_of_the_backward(dt, D, Lq, Lk, Hk):
    """The dk/dv kernels read a boolean mask from its bit-packed copy when they are handed one: every gradient
    of every kind of call (first order, both output gradients, all six gradients, no gO, dropout) must equal,
    bit for bit, what the same kernels give when they read the mask itself."""
    from jvp_flash_attention_amd import _lib

    Z, H = 2, 4
    dtype = DTYPES[dt]
    g = torch.Generator().manual_seed(Lq + D)
    q, qt, go, gt = (torch.randn(Z, H, Lq, D, generator=g).to(dtype).cuda() for _ in range(4))
    k, v, kt, vt = (torch.randn(Z, Hk, Lk, D, generator=g).to(dtype).cuda() for _ in range(4))
    keep = torch.rand(Z, H, Lq, Lk, generator=g) > 0.2
    keep[1, 2, 40:75] = False  # rows that attend nothing
    keep[0, 1, :, 100:300] = False  # keys that nothing attends
    be, scale = _lib.backend(), D**-0.5
    print(f"case packed mask {dt} D{D} Lq{Lq} Lk{Lk} Hk{Hk}", flush=True)

    def run(dmask):
        o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, dmask, _lib.MASK_BOOL, False, scale)
        out = list(be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, dmask, _lib.MASK_BOOL, False, scale, want_tangent_grads=True))
        out += be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, dmask, _lib.MASK_BOOL, False, scale)[:3]
        out += be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, None, gt, dmask, _lib.MASK_BOOL, False, scale)[:3]
        out += be.bwd(q, k, v, None, None, None, o, None, M, None, go, None, dmask, _lib.MASK_BOOL, False, scale)[:3]
        od, otd, Md, mud = be.fwd(q, k, v, qt, kt, vt, dmask, _lib.MASK_BOOL, False, scale, 0.2, 11)
        out += be.bwd(q, k, v, qt, kt, vt, od, otd, Md, mud, go, gt, dmask, _lib.MASK_BOOL, False, scale,
                      dropout_p=0.2, dropout_seed=11)[:3]
        return out

    dmask = keep.cuda()
    packed = run(dmask)
    assert getattr(dmask, "_jvpfa_bits")[1] is not None
    _lib.set_mask_bits(False)
    try:
        other = keep.cuda()
        from_bytes = run(other)
        assert not hasattr(other, "_jvpfa_bits")
    finally:
        _lib.set_mask_bits(True)
    for a, b in zip(packed, from_bytes):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dt", ["bf16", "fp16"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("Lq,Lk,Hk,planes", [(704, 704, 16, "zh"), (545, 832, 4, "z1"), (300, 1160, 16, "11"),
                                             (600, 712, 16, "keys")])
def test_additive_masks_whose_tiles_go_through_lds(dt, D, Lq, Lk, Hk, planes):
    """An additive mask whose rows are contiguous keys starting on 16-byte boundaries reaches the dk/dv kernels as
    tiles in LDS (where they have the room); any other layout is fetched element by element.  Both against the
    oracle, and against each other: the same values one element further on in memory (rows no longer aligned)
    must give the same gradients to rounding of the last bit.  (64 heads: with fewer workgroups than compute
    units the backward runs as one launch of both roles, which reads every mask element by element.)"""
    from jvp_flash_attention_amd import _lib

    Z, H = 4, 16
    dtype = DTYPES[dt]
    g = torch.Generator().manual_seed(Lq + Lk + D)
    q, qt, go, gt = (torch.randn(Z, H, Lq, D, generator=g).to(dtype) for _ in range(4))
    k, v, kt, vt = (torch.randn(Z, Hk, Lk, D, generator=g).to(dtype) for _ in range(4))
    # "keys": one row of keys per batch entry, shared by heads and queries (a mask row of stride 0)
    shape = {"zh": (Z, H, Lq, Lk), "z1": (Z, 1, Lq, Lk), "11": (1, 1, Lq, Lk), "keys": (Z, 1, 1, Lk)}[planes]
    bias = torch.randn(*shape, generator=g).to(dtype)
    bias[..., 17:90] = float("-inf")       # keys nobody attends
    if planes != "keys":
        bias[0, 0, 33:70, :] = float("-inf")   # rows that attend nothing
        bias[0, 0, 200:, 500:] = float("-inf")
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    be, scale = _lib.backend(), D**-0.5
    print(f"case mask tiles {dt} D{D} Lq{Lq} Lk{Lk} Hk{Hk} {planes}", flush=True)

    def run(dmask):
        o, ot, M, mu = be.fwd(*dev[:6], dmask, _lib.MASK_ADD, False, scale)
        out = list(be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, _lib.MASK_ADD, False, scale, want_tangent_grads=True))
        out += be.bwd(*dev[:6], o, ot, M, mu, None, dev[7], dmask, _lib.MASK_ADD, False, scale)[:3]
        out += be.bwd(dev[0], dev[1], dev[2], None, None, None, o, None, M, None, dev[6], None, dmask, _lib.MASK_ADD, False, scale)[:3]
        return o, ot, out

    aligned = bias.cuda()
    assert aligned.data_ptr() % 16 == 0 and (Lk * aligned.element_size()) % 16 == 0
    o, ot, tiled = run(aligned)
    shifted = torch.empty(bias.numel() + 1, dtype=dtype, device="cuda")[1:].view(shape)  # one element off: no tiles
    shifted.copy_(bias)
    _, _, by_element = run(shifted)
    for a, b in zip(tiled, by_element):
        assert torch.allclose(a.float(), b.float(), rtol=0, atol=2e-2 * float(b.float().abs().max()) + 1e-30)
    if planes == "zh":  # with tile lists (tiles that are -inf throughout are not visited): not a bit changes
        _lib.set_tile_lists(True, additive=True)
        try:
            listed_mask = bias.cuda()
            _, _, listed = run(listed_mask)
            assert getattr(listed_mask, "_jvpfa_tiles")[2] is not None
        finally:
            _lib.set_tile_lists(True, additive=False)
        for a, b in zip(listed, tiled):
            assert torch.equal(a, b)
    npm = np.broadcast_to(bias.float().numpy(), (Z, H, Lq, Lk))
    ref = dense.forward(*f64[:6], mask=npm, causal=False, scale=scale)
    rb = dense.backward(*f64, mask=npm, causal=False, scale=scale)
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), tiled[:6]):
        _tol_check(n, t, rb[n], dtype)


@pytest.mark.parametrize("dt,D", [("bf16", 32), ("bf16", 64), ("bf16", 128), ("bf16", 256),
                                  ("fp32", 32), ("fp32", 64), ("fp32", 128), ("fp32", 256)])
@pytest.mark.parametrize("kind", ["blockdiag", "band", "pad2d", "lower"])
@pytest.mark.parametrize("as_bias", [False, True])
def test_structured_masks_with_skipped_tiles(dt, D, kind, as_bias):
    """Masks with whole tiles masked: the host scans them into tile lists and the kernels visit the
    listed tiles only.  Checked against the oracle, and bit for bit against the same kernels made to
    visit every tile (a fully masked tile contributes exact zeros)."""
    from jvp_flash_attention_amd import _lib

    Z, H, L = 2, 2, 700
    dtype = DTYPES[dt]
    q, k, v, qt, kt, vt, go, gt = _make(Z, H, L, D, dtype, 31)
    keep = _structured_keep(kind, Z, H, L)
    mask = torch.where(keep, 0.0, float("-inf")).to(dtype) if as_bias else keep
    mk = _lib.MASK_ADD if as_bias else _lib.MASK_BOOL
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    be = _lib.backend()
    scale = D**-0.5
    print(f"case structured {dt} {kind} D{D} bias={as_bias}", flush=True)

    def run(dmask):
        o, ot, M, mu = be.fwd(*dev[:6], dmask, mk, False, scale)
        grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, mk, False, scale, want_tangent_grads=True)
        g1 = be.bwd(dev[0], dev[1], dev[2], None, None, None, o, None, M, None, dev[6], None, dmask, mk, False, scale)
        return [o, ot, M, mu, *grads, *g1[:3]]

    dmask = mask.cuda()
    _lib.set_tile_lists(True, additive=True)  # additive masks are only scanned on request
    try:
        with_lists = run(dmask)
        assert getattr(dmask, "_jvpfa_tiles")[1] is not None and getattr(dmask, "_jvpfa_tiles")[2] is not None
        _lib.set_tile_lists(False)
        every_tile = run(mask.cuda())
    finally:
        _lib.set_tile_lists(True, additive=False)
    for a, b in zip(with_lists, every_tile):
        assert torch.equal(a, b)

    npm = keep.numpy()
    ref = dense.forward(*f64[:6], mask=npm, causal=False, scale=scale)
    rb = dense.backward(*f64, mask=npm, causal=False, scale=scale)
    _tol_check("O", with_lists[0], ref["O"], dtype)
    _tol_check("O'", with_lists[1], ref["Ot"], dtype)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), with_lists[4:10]):
        _tol_check(n, t, rb[n], dtype)


def _numpy_tile_lists_rect(keep, Lq, Lk):
    """(tiles_q, tiles_k) from a (P, Lq, Lk) boolean array: per block of 128 query rows the 64-key tiles, per
    block of 128 keys the 64-query tiles."""
    tq, tk = [], []
    for pl in keep:
        for b in range((Lq + 127) // 128):
            rows = pl[128 * b:128 * b + 128]
            tq.append([t for t in range((Lk + 63) // 64) if rows[:, 64 * t:64 * t + 64].any()] or [0])
        for b in range((Lk + 127) // 128):
            cols = pl[:, 128 * b:128 * b + 128]
            tk.append([t for t in range((Lq + 63) // 64) if cols[64 * t:64 * t + 64].any()] or [0])
    return tq, tk


@pytest.mark.parametrize("dt,D", [("bf16", 64), ("fp16", 128), ("bf16", 256), ("fp32", 64)])
@pytest.mark.parametrize("Lq,Lk", [(300, 900), (900, 300), (520, 97)])
def test_structured_masks_with_as_many_keys_as_they_like(dt, D, Lq, Lk):
    """Tile lists of a mask whose two axes differ in length (cross attention over packed or windowed memory):
    the lists against a numpy scan, the kernels with lists bit for bit against every tile, and against the
    oracle; 4 query heads over 2 key/value heads."""
    from jvp_flash_attention_amd import _lib

    Z, H, Hk = 2, 4, 2
    dtype = DTYPES[dt]
    g = torch.Generator().manual_seed(Lq + Lk)
    q, qt, go, gt = (torch.randn(Z, H, Lq, D, generator=g).to(dtype) for _ in range(4))
    k, v, kt, vt = (torch.randn(Z, Hk, Lk, D, generator=g).to(dtype) for _ in range(4))
    # a slanted band (each query sees a window of keys around its own relative position), different per batch entry
    i, j = torch.arange(Lq)[:, None].float() / Lq, torch.arange(Lk)[None, :].float() / Lk
    keep = torch.stack([(i - j).abs() <= w for w in (0.08, 0.2)]).view(Z, 1, Lq, Lk)
    keep[1, 0, 10:150] = False  # query rows that attend nothing: zeros
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    be, scale = _lib.backend(), D**-0.5
    print(f"case rectangular lists {dt} D{D} Lq{Lq} Lk{Lk}", flush=True)

    def run(dmask):
        o, ot, M, mu = be.fwd(*dev[:6], dmask, _lib.MASK_BOOL, False, scale)
        grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, _lib.MASK_BOOL, False, scale, want_tangent_grads=True)
        return [o, ot, M, mu, *grads]

    dmask = keep.cuda()
    with_lists = run(dmask)
    tq, tk = getattr(dmask, "_jvpfa_tiles")[1:3]
    rq, rk = _numpy_tile_lists_rect(keep.reshape(-1, Lq, Lk).numpy(), Lq, Lk)
    for got, ref, nt in ((tq, rq, (Lk + 63) // 64), (tk, rk, (Lq + 63) // 64)):
        got = got.cpu().view(-1, nt + 1).tolist()
        assert len(got) == len(ref)
        for row, want in zip(got, ref):
            assert row[0] == len(want) and row[1:1 + row[0]] == want
    _lib.set_tile_lists(False)
    try:
        every_tile = run(keep.cuda())
    finally:
        _lib.set_tile_lists(True)
    for a, b in zip(with_lists, every_tile):
        assert torch.equal(a, b)
    ref = dense.forward(*f64[:6], mask=keep.numpy(), causal=False, scale=scale)
    rb = dense.backward(*f64, mask=keep.numpy(), causal=False, scale=scale)
    _tol_check("O", with_lists[0], ref["O"], dtype)
    _tol_check("O'", with_lists[1], ref["Ot"], dtype)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), with_lists[4:10]):
        _tol_check(n, t, rb[n], dtype)


@pytest.mark.parametrize("seed", range(24))
def test_random_configurations(seed):
    """Element type, head dim, batch, heads, sequence length (ragged ones included, some long enough
    for the tile lists and the key-limit hint) and mask mode drawn from a seeded generator."""
    from jvp_flash_attention_amd import _lib

    rng = np.random.default_rng(1000 + seed)
    dt = ["bf16", "fp16", "fp32"][rng.integers(3)]
    D = [32, 64, 128, 256][rng.integers(4)] if dt != "fp32" else [32, 64, 128, 256][int(rng.integers(3)) + (seed % 5 == 4)]
    Z, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    long_case = seed % 3 == 0
    L = int(rng.integers(513, 900)) if long_case else int(rng.integers(1, 300))
    mode = ["none", "causal", "keypad", "bias", "bool_full", "blockdiag", "band", "pad2d", "lower"][rng.integers(9)]
    dtype = DTYPES[dt]
    if mode in ("none", "causal", "keypad", "bias", "bool_full"):
        _run_case(Z, H, L, D, dtype, mode, seed=seed, tangent_grads=bool(rng.integers(2)))
        return
    keep = _structured_keep(mode, Z, H, L, seed=seed) if L > 100 or mode != "blockdiag" else _structured_keep("band", Z, H, L)
    as_bias = bool(rng.integers(2))
    q, k, v, qt, kt, vt, go, gt = _make(Z, H, L, D, dtype, seed)
    mask = torch.where(keep, 0.0, float("-inf")).to(dtype) if as_bias else keep
    mk = _lib.MASK_ADD if as_bias else _lib.MASK_BOOL
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    print(f"case random {seed}: Z{Z} H{H} L{L} D{D} {dt} {mode} bias={as_bias}", flush=True)
    be, scale, dmask = _lib.backend(), D**-0.5, mask.cuda()
    o, ot, M, mu = be.fwd(*dev[:6], dmask, mk, False, scale)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, mk, False, scale, want_tangent_grads=True)
    ref = dense.forward(*f64[:6], mask=keep.numpy(), causal=False, scale=scale)
    rb = dense.backward(*f64, mask=keep.numpy(), causal=False, scale=scale)
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        _tol_check(n, t, rb[n], dtype)


def test_mask_combined_with_causal_is_refused():
    # as in the reference, causal attention takes no explicit mask: the library reports it instead of guessing
    with pytest.raises(RuntimeError, match="causal"):
        _run_case(1, 2, 128, 64, torch.bfloat16, "keypad", causal=True)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("mode", ["none", "causal", "keypad", "bias"])
def test_plain_forward_and_first_order_backward(dt, mode):
    _run_case(2, 2, 160, 64, DTYPES[dt], mode, plain=True)
    _run_case(1, 2, 128, 128, DTYPES[dt], mode, plain=True)


def test_small_tangents_config2_shape_slice():
    # benchmark configuration 2 statistics (tangents ~ N(0, 0.1^2)) on a slice of its shape
    _run_case(1, 4, 512, 64, torch.bfloat16, "none", tangent_std=0.1)


@pytest.mark.parametrize("dt,D", [("fp32", 64), ("bf16", 32), ("bf16", 64), ("bf16", 128), ("fp16", 256), ("bf16", 256)])
def test_fully_masked_rows_are_zero(dt, D):
    """Rows without any attended key: O = O' = 0, M = +inf, mu = 0 and zero gradients, in every kernel
    family (the reference gives O = 0 there too, its jvp_attention.py:1011-1015)."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, L = 1, 2, 64
    dtype = DTYPES[dt]
    q, k, v, qt, kt, vt, go, gt = [x.cuda() for x in _make(Z, H, L, D, dtype, 3)]
    mask = torch.ones(Z, H, L, L, dtype=torch.bool)
    mask[0, 1, 5, :] = False
    mask[0, 0, 40, :] = False
    mask = mask.cuda()
    o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, mask, _lib.MASK_BOOL, False, D**-0.5)
    for t in (o, ot):
        assert torch.all(t[0, 1, 5] == 0) and torch.all(t[0, 0, 40] == 0) and torch.isfinite(t).all()
    assert torch.isposinf(M[0, 1, 5]) and mu[0, 1, 5] == 0
    grads = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, _lib.MASK_BOOL, False, D**-0.5,
                   want_tangent_grads=True)
    for gname, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert torch.isfinite(t).all(), gname
    assert torch.all(grads[0][0, 1, 5] == 0) and torch.all(grads[3][0, 0, 40] == 0)
    f64 = [x.double().cpu().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    rb = dense.backward(*f64, mask=mask.cpu().numpy(), scale=D**-0.5)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        _tol_check(n, t, rb[n], dtype)


def test_only_tangent_gradient_hvp_style():
    """gO absent (loss is a function of O' only), the Hessian-vector-product use."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    Z, H, L, D = 1, 2, 256, 128
    xs = _make(Z, H, L, D, torch.bfloat16, 5)
    f64 = [x.double().numpy() for x in xs]
    dev = [x.cuda() for x in xs]
    o, ot, M, mu = be.fwd(*dev[:6], None, _lib.MASK_NONE, True, D**-0.5)
    grads = be.bwd(*dev[:6], o, ot, M, mu, None, dev[7], None, _lib.MASK_NONE, True, D**-0.5)
    rb = dense.backward(*f64[:6], np.zeros_like(f64[6]), f64[7], causal=True, scale=D**-0.5)
    for n, t in zip(("dq", "dk", "dv"), grads[:3]):
        _tol_check(n, t, rb[n], torch.bfloat16)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("mode", ["causal", "bool_full"])
def test_all_six_gradients_without_gO(dt, D, mode):
    """gO absent and all six gradients asked for: the dual kernels that also write dq' (and dk', dv' for D = 32)
    in their variant without gO, with grouped heads so that the dk/dv kernel adds up over the heads of a group."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    dtype = DTYPES[dt]
    Z, H, Hk, L = 2, 4, 2, 200
    q, k, v, qt, kt, vt, go, gt = _make(Z, H, L, D, dtype, 9)
    k, v, kt, vt = (x[:, :Hk].contiguous() for x in (k, v, kt, vt))
    mask = _mask(mode, Z, H, L, dtype)
    causal = mode == "causal"
    kind = _lib.MASK_NONE if mask is None else _lib.MASK_BOOL
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt)]
    dmask = None if mask is None else mask.cuda()
    print(f"six gradients without gO {dt} D{D} {mode}", flush=True)
    o, ot, M, mu = be.fwd(*dev, dmask, kind, causal, D**-0.5)
    grads = be.bwd(*dev, o, ot, M, mu, None, gt.cuda(), dmask, kind, causal, D**-0.5, want_tangent_grads=True)
    rb = dense.backward(*f64, np.zeros(q.shape), gt.double().numpy(), mask=None if mask is None else mask.numpy(),
                        causal=causal, scale=D**-0.5)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        _tol_check(n, t, rb[n], dtype)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
def test_single_key(dt):
    """L = 1: softmax is the constant 1, so O = v, O' = v' and dq = dk = dq' = dk' = 0 exactly.
    In 16-bit the zero gradients come out as rounding residue of O and O' (stored rounded), so
    they are held to an absolute bound instead of a relative one."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    dtype = DTYPES[dt]
    q, k, v, qt, kt, vt, go, gt = [x.cuda() for x in _make(2, 2, 1, 64, dtype, 9)]
    o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, _lib.MASK_NONE, False, 0.125)
    assert torch.equal(o, v)
    # O' = (p s') v / l - mu O + v': the first two terms cancel only up to the rounding of p s'
    assert (ot.float() - vt.float()).abs().max().item() <= (1e-5 if dtype == torch.float32 else 5e-2)
    grads = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, _lib.MASK_NONE, False, 0.125,
                   want_tangent_grads=True)
    bound = 1e-5 if dtype == torch.float32 else 5e-2
    for i in (0, 1, 3, 4):
        assert grads[i].float().abs().max().item() <= bound
    assert (grads[2].float() - go.float()).abs().max().item() <= bound
    assert (grads[5].float() - gt.float()).abs().max().item() <= bound


@pytest.mark.parametrize("dt,D", [("bf16", 128), ("fp16", 128), ("fp32", 128), ("bf16", 32), ("bf16", 64), ("bf16", 256)])
@pytest.mark.parametrize("causal", [False, True])
def test_growing_row_maximum_exercises_the_rescale_path(dt, D, causal):
    """Keys whose scores grow along the sequence: the running maximum keeps rising past the lazy
    rescale threshold, so the accumulators are rescaled on many tiles (not only the first)."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    dtype = DTYPES[dt]
    Z, H, L = 1, 2, 512
    q, k, v, qt, kt, vt, go, gt = _make(Z, H, L, D, dtype, 21)
    ramp = torch.linspace(0.2, 6.0, L).view(1, 1, L, 1) * (128 / D) ** 0.5  # the same score range for every D
    k = (k.float() * ramp).to(dtype)
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    scale = D**-0.5
    ref = dense.forward(*f64[:6], causal=causal, scale=scale)
    rb = dense.backward(*f64, causal=causal, scale=scale)
    o, ot, M, mu = be.fwd(*dev[:6], None, _lib.MASK_NONE, causal, scale)
    # fp32 bound relative to the size of the outputs here (scores reach +-60, O' reaches ~1e2)
    for name, got, want in (("O", o, ref["O"]), ("O'", ot, ref["Ot"])):
        got = got.double().cpu().numpy()
        rel = np.abs(got - want).max() / np.abs(want).max()
        assert np.isfinite(got).all() and rel <= (2e-5 if dtype == torch.float32 else 2e-2), (name, rel)
    # M is kept in fp32 from identical inputs in every element type: log2 units at values near 90
    assert np.abs(M.double().cpu().numpy() - ref["M"]).max() < (1e-3 if dtype == torch.float32 else 2e-2)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], None, _lib.MASK_NONE, causal, scale, want_tangent_grads=True)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        got = t.double().cpu().numpy()
        rel = np.abs(got - rb[n]).max() / np.abs(rb[n]).max()
        assert np.isfinite(got).all() and rel <= (5e-5 if dtype == torch.float32 else 2e-2), (n, rel)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("mode", ["none", "causal", "bias"])
@pytest.mark.parametrize("std", [64.0, 256.0])
def test_fp16_tangents_of_large_norm(D, mode, std):
    """An HVP caller passes a vector of whatever norm it has.  The operand P (S' - c) of the tangent accumulation is
    a 16-bit number: with fp16 it overflows once p |S' - c| passes 65504, and the lazy rescale lets p exceed 1, so
    the fp16 kernels keep its slack at 2^4 (|S' - c| reaches about 2000 here, the kernels hold to 4000; the
    reference's p <= 1 holds to 65504).  Every forward kernel family for fp16 (direct-to-LDS, software-pipelined with and without a mask, the
    D = 256 pair of passes) and the backward behind it."""
    _run_case(1, 2, 320, D, torch.float16, mode, seed=71, tangent_std=std)


def test_config1_shape_and_seed_on_the_gpu():
    """Benchmark configuration 1 (fp32, B2 H4 L128 D64, seed 0, every tensor iid N(0,1), no mask) is the
    reference's CPU plumbing case; the same tensors through the HIP kernels, held to max-abs 1e-4."""
    _run_case(2, 4, 128, 64, torch.float32, "none", seed=0)


@pytest.mark.parametrize("dt,D", [("bf16", 64), ("fp32", 64), ("bf16", 32), ("bf16", 128), ("bf16", 256)])
@pytest.mark.parametrize("scale", [0.05, 1.0, -0.3])
def test_custom_softmax_scale_including_negative(dt, D, scale):
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    dtype = DTYPES[dt]
    Z, H, L = 1, 2, 192
    xs = _make(Z, H, L, D, dtype, 33)
    if abs(scale) >= 1.0:
        xs[0] = (xs[0].float() * 0.3 * (64 / D) ** 0.5).to(dtype)  # the same score range for every D
    f64 = [x.double().numpy() for x in xs]
    dev = [x.cuda() for x in xs]
    ref = dense.forward(*f64[:6], scale=scale)
    rb = dense.backward(*f64, scale=scale)
    o, ot, M, mu = be.fwd(*dev[:6], None, _lib.MASK_NONE, False, scale)

    def check(name, got, want):
        # with |scale| = 1 the gradients reach ~50, so the fp32 bound is taken relative to that size
        if dtype == torch.float32:
            err = np.abs(got.double().cpu().numpy() - want).max()
            assert err <= 1e-4 * max(1.0, np.abs(want).max() / 8), f"{name}: {err:.3e}"
        else:
            _tol_check(name, got, want, dtype)

    check("O", o, ref["O"])
    check("O'", ot, ref["Ot"])
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], None, _lib.MASK_NONE, False, scale)
    for n, t in zip(("dq", "dk", "dv"), grads[:3]):
        check(n, t, rb[n])


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
def test_additive_mask_with_minus_infinity_entries(dt):
    """SDPA-style float masks use -inf for masked entries; whole tiles and whole rows of -inf included."""
    from jvp_flash_attention_amd import _lib

    be = _lib.backend()
    dtype = DTYPES[dt]
    Z, H, L, D = 1, 2, 160, 64
    xs = _make(Z, H, L, D, dtype, 35)
    g = torch.Generator().manual_seed(5)
    bias = torch.randn(Z, H, L, L, generator=g)
    bias[torch.rand(Z, H, L, L, generator=g) < 0.5] = -float("inf")
    bias[..., :, 64:128] = -float("inf")   # a whole 64-key tile masked for every row
    bias[..., 0] = 0.0                      # every row keeps key 0 ...
    bias[0, 1, 17, :] = -float("inf")      # ... except one fully masked row
    bias = bias.to(dtype)
    f64 = [x.double().numpy() for x in xs]
    dev = [x.cuda() for x in xs]
    scale = D**-0.5
    ref = dense.forward(*f64[:6], mask=bias.double().numpy(), scale=scale)
    rb = dense.backward(*f64, mask=bias.double().numpy(), scale=scale)
    o, ot, M, mu = be.fwd(*dev[:6], bias.cuda(), _lib.MASK_ADD, False, scale)
    assert torch.all(o[0, 1, 17] == 0) and torch.all(ot[0, 1, 17] == 0) and torch.isposinf(M[0, 1, 17])
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], bias.cuda(), _lib.MASK_ADD, False, scale,
                   want_tangent_grads=True)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        _tol_check(n, t, rb[n], dtype)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("shape", [(4, 2, 96, 96), (4, 1, 70, 200), (2, 2, 200, 70), (6, 3, 130, 33), (2, 1, 3, 5), (2, 2, 5, 2)])
@pytest.mark.parametrize("mode", ["none", "causal", "bool", "bias"])
def test_grouped_heads_and_a_key_length_of_its_own(dt, D, shape, mode):
    """Beyond the reference (q, k, v of one shape there): H query heads over Hk key/value heads, Lq
    queries over Lk keys; dk, dv (and dk', dv') have k's shape and sum over the heads of a group."""
    _run_kv_shape_case(dt, D, shape, mode)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(4, 2, 96, 96), (2, 1, 70, 200), (2, 2, 200, 70), (1, 1, 1, 3), (1, 1, 33, 31), (2, 2, 5, 2)])
@pytest.mark.parametrize("mode", ["none", "causal", "bool", "bias"])
def test_head_dim_256_with_grouped_heads_key_lengths_and_tiny_shapes(dt, shape, mode):
    """The D = 256 kernels (two forward passes over 32-key tiles; a backward whose workgroups are two pairs
    of waves that share 32 rows) on the shapes of the test above, down to a single query."""
    _run_kv_shape_case(dt, 256, shape, mode)


def _run_kv_shape_case(dt, D, shape, mode):
    from jvp_flash_attention_amd import _lib

    H, Hk, Lq, Lk = shape
    Z, dtype = 2, DTYPES[dt]
    g = torch.Generator().manual_seed(sum(map(ord, dt + mode)) + D + sum(shape))
    # tangents ~ N(0,1), as large as the primals (what the benchmark configurations with causal masks use)
    q, go, gt, qt = [torch.randn(Z, H, Lq, D, generator=g).to(dtype) for _ in range(4)]
    k, v, kt, vt = [torch.randn(Z, Hk, Lk, D, generator=g).to(dtype) for _ in range(4)]
    mask, kind, causal = None, _lib.MASK_NONE, mode == "causal"
    if mode == "bool":
        mask, kind = torch.rand(Z, H, Lq, Lk, generator=g) > 0.5, _lib.MASK_BOOL
        mask[..., 0] = True
    if mode == "bias":
        mask, kind = torch.randn(Z, 1, Lq, Lk, generator=g).to(dtype), _lib.MASK_ADD
    print(f"case kv-shape Z{Z} H{H}/{Hk} Lq{Lq} Lk{Lk} D{D} {dt} {mode}", flush=True)
    npm = None if mask is None else (mask.numpy() if mask.dtype == torch.bool else mask.double().numpy())
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    scale = D**-0.5
    ref = dense.forward(*f64[:6], mask=npm, causal=causal, scale=scale)
    rb = dense.backward(*f64, mask=npm, causal=causal, scale=scale)
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    dmask = None if mask is None else mask.cuda()
    be = _lib.backend()
    o, ot, M, mu = be.fwd(*dev[:6], dmask, kind, causal, scale)
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, kind, causal, scale, want_tangent_grads=True)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        assert tuple(t.shape) == rb[n].shape, n
        _tol_check(n, t, rb[n], dtype)
    op, _, Mp, _ = be.fwd(dev[0], dev[1], dev[2], None, None, None, dmask, kind, causal, scale)
    _tol_check("O (plain)", op, ref["O"], dtype)
    rb1 = dense.backward(*f64[:7], None, mask=npm, causal=causal, scale=scale)
    g1 = be.bwd(dev[0], dev[1], dev[2], None, None, None, op, None, Mp, None, dev[6], None, dmask, kind, causal, scale)
    for n, t in zip(("dq", "dk", "dv"), g1[:3]):
        _tol_check(n + " (plain)", t, rb1[n], dtype)


def test_grouped_heads_with_key_padding_and_skipped_tiles():
    """The key-limit hint with 8 query heads over 2 key/value heads and 700 keys for 300 queries."""
    from jvp_flash_attention_amd import _lib

    Z, H, Hk, Lq, Lk, D = 2, 8, 2, 300, 700, 64
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(77)
    q, go, gt = [torch.randn(Z, H, Lq, D, generator=g).to(dtype) for _ in range(3)]
    qt = (0.5 * torch.randn(Z, H, Lq, D, generator=g)).to(dtype)
    k, v = [torch.randn(Z, Hk, Lk, D, generator=g).to(dtype) for _ in range(2)]
    kt, vt = [(0.5 * torch.randn(Z, Hk, Lk, D, generator=g)).to(dtype) for _ in range(2)]
    lens = [700, 130]
    mask = (torch.arange(Lk)[None, :] < torch.tensor(lens)[:, None]).view(Z, 1, 1, Lk)
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    dmask, scale, be = mask.cuda(), D**-0.5, _lib.backend()
    assert _lib.key_limit_hint(dmask, _lib.MASK_BOOL, Z, Lk).tolist() == lens
    ref = dense.forward(*f64[:6], mask=mask.numpy(), scale=scale)
    rb = dense.backward(*f64, mask=mask.numpy(), scale=scale)
    o, ot, M, mu = be.fwd(*dev[:6], dmask, _lib.MASK_BOOL, False, scale)
    grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, _lib.MASK_BOOL, False, scale, want_tangent_grads=True)
    _tol_check("O", o, ref["O"], dtype)
    _tol_check("O'", ot, ref["Ot"], dtype)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), grads):
        _tol_check(n, t, rb[n], dtype)
    assert grads[1][1, :, 256:].abs().max().item() == 0.0  # key blocks past the limit of batch entry 1


@pytest.mark.parametrize("D", [32, 64, 128, 256])
@pytest.mark.parametrize("kind", ["blockdiag", "band", "per_head"])
def test_grouped_heads_with_structured_masks_and_skipped_tiles(D, kind):
    """Tile lists with 4 query heads over 2 key/value heads: the lists belong to the mask planes (one
    per query head when the mask has a head axis), so the dk/dv kernel changes list with every query
    head of a group.  Against the oracle, and bit for bit against visiting every tile."""
    from jvp_flash_attention_amd import _lib

    Z, H, Hk, L = 2, 4, 2, 700
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(91)
    q, go, gt = [torch.randn(Z, H, L, D, generator=g).to(dtype) for _ in range(3)]
    qt = (0.5 * torch.randn(Z, H, L, D, generator=g)).to(dtype)
    k, v = [torch.randn(Z, Hk, L, D, generator=g).to(dtype) for _ in range(2)]
    kt, vt = [(0.5 * torch.randn(Z, Hk, L, D, generator=g)).to(dtype) for _ in range(2)]
    if kind == "per_head":  # a band whose width and offset differ from head to head
        i, j = torch.arange(L)[:, None], torch.arange(L)[None, :]
        keep = torch.stack([((i - j) <= 40 + 90 * h) & ((j - i) <= 200 - 60 * h) for h in range(H)]).view(1, H, L, L)
    else:
        keep = _structured_keep(kind, Z, H, L)
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt, go, gt)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt, go, gt)]
    be, scale = _lib.backend(), D**-0.5
    print(f"case grouped structured {kind} D{D}", flush=True)

    def run(dmask):
        o, ot, M, mu = be.fwd(*dev[:6], dmask, _lib.MASK_BOOL, False, scale)
        grads = be.bwd(*dev[:6], o, ot, M, mu, dev[6], dev[7], dmask, _lib.MASK_BOOL, False, scale, want_tangent_grads=True)
        return [o, ot, M, mu, *grads]

    dmask = keep.cuda()
    try:
        with_lists = run(dmask)
        assert getattr(dmask, "_jvpfa_tiles")[1] is not None and getattr(dmask, "_jvpfa_tiles")[2] is not None
        _lib.set_tile_lists(False)
        every_tile = run(keep.cuda())
    finally:
        _lib.set_tile_lists(True, additive=False)
    for a, b in zip(with_lists, every_tile):
        assert torch.equal(a, b)
    ref = dense.forward(*f64[:6], mask=keep.numpy(), scale=scale)
    rb = dense.backward(*f64, mask=keep.numpy(), scale=scale)
    _tol_check("O", with_lists[0], ref["O"], dtype)
    _tol_check("O'", with_lists[1], ref["Ot"], dtype)
    for n, t in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), with_lists[4:10]):
        _tol_check(n, t, rb[n], dtype)


@pytest.mark.parametrize("D", [32, 64, 128, 256])
@pytest.mark.parametrize("heads", [(4, 4), (4, 2)])
@pytest.mark.parametrize("mode", ["none", "causal", "bool"])
def test_results_are_the_same_from_run_to_run(D, heads, mode):
    """Every kernel is deterministic (no atomics, fixed summation order): three runs of the dual forward
    and backward give bit-identical results.  A missing idle slot in front of an inline-asm matrix
    instruction once showed up exactly here: one wave in a few with a different dK from run to run."""
    from jvp_flash_attention_amd import _lib

    H, Hk = heads
    Z, L, dtype = 2, 200, torch.bfloat16
    g = torch.Generator().manual_seed(5 * D + H + Hk)
    q, qt, go, gt = [torch.randn(Z, H, L, D, generator=g).to(dtype).cuda() for _ in range(4)]
    k, v, kt, vt = [torch.randn(Z, Hk, L, D, generator=g).to(dtype).cuda() for _ in range(4)]
    mask, kind, causal = None, _lib.MASK_NONE, mode == "causal"
    if mode == "bool":
        mask, kind = (torch.rand(Z, H, L, L, generator=g) > 0.5).cuda(), _lib.MASK_BOOL
    be, scale = _lib.backend(), D**-0.5
    print(f"case reproducible D{D} H{H}/{Hk} {mode}", flush=True)
    runs = []
    for _ in range(3):
        o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, mask, kind, causal, scale)
        grads = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, kind, causal, scale, want_tangent_grads=True)
        runs.append([o, ot, M, mu, *grads])
    for other in runs[1:]:
        for a_, b_ in zip(runs[0], other):
            assert torch.equal(a_, b_)


@pytest.mark.parametrize("dt", ["bf16", "fp16"])
@pytest.mark.parametrize("shape", [(1, 2, 1024, 1024, True), (1, 2, 1024, 1024, False), (1, 3, 333, 700, False),
                                   (2, 1, 700, 700, True), (1, 1, 4096, 512, False)])
@pytest.mark.parametrize("dual", [True, False])
def test_small_launches_split_over_key_chunks(dt, shape, dual):
    """Launches with far fewer query blocks than the GPU has compute units (D = 128, no mask): the key tiles of a
    block are split over several workgroups and merged.  Against the oracle, and against the same launch without
    the split (one ulp of the element type apart at most; M and mu, which stay fp32, to 1e-5)."""
    from jvp_flash_attention_amd import _lib

    Z, H, L, Lk, causal = shape
    D, dtype = 128, DTYPES[dt]
    g = torch.Generator().manual_seed(L + Lk)
    q, qt = [torch.randn(Z, H, L, D, generator=g).to(dtype) for _ in range(2)]
    k, v, kt, vt = [torch.randn(Z, H, Lk, D, generator=g).to(dtype) for _ in range(4)]
    dev = [x.cuda() for x in (q, k, v, qt, kt, vt)]
    if not dual:
        dev[3:] = [None, None, None]
    be, scale = _lib.backend(), D**-0.5
    print(f"case split Z{Z} H{H} L{L} Lk{Lk} causal={causal} {dt} dual={dual}", flush=True)
    a = _lib.FwdArgs()
    a.p = _lib.make_problem(dev[0], None, _lib.MASK_NONE, causal, scale)
    assert _lib.load().jvpfa_fwd_split_workspace_bytes(C.byref(a.p), Lk) > 0  # this launch does split
    got = be.fwd(*dev, None, _lib.MASK_NONE, causal, scale)
    _lib.set_split(False)
    try:
        one = be.fwd(*dev, None, _lib.MASK_NONE, causal, scale)
    finally:
        _lib.set_split(True)
    f64 = [x.double().numpy() for x in (q, k, v, qt, kt, vt)]
    ref = dense.forward(*f64, causal=causal, scale=scale) if dual else dense.forward(*f64[:3], causal=causal, scale=scale)
    _tol_check("O", got[0], ref["O"], dtype)
    assert np.abs(got[2].double().cpu().numpy() - ref["M"]).max() < 1e-4
    assert (got[2] - one[2]).abs().max().item() <= 1e-5
    ulp = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10
    assert ((got[0].float() - one[0].float()).abs() <= ulp * one[0].float().abs().clamp_min(1.0)).all()
    if dual:
        _tol_check("O'", got[1], ref["Ot"], dtype)
        assert np.abs(got[3].double().cpu().numpy() - ref["mu"]).max() < 1e-4 * max(1.0, np.abs(ref["mu"]).max())
        assert ((got[1].float() - one[1].float()).abs() <= 2 * ulp * one[1].float().abs().clamp_min(1.0)).all()


def test_c_abi_from_a_plain_cpp_program():
    """``tests/cabi_host/host_check`` (built with the library) calls jvpfa_fwd / jvpfa_bwd from C++ with
    memory it allocated through the HIP runtime, no Python or torch in its process, and compares with
    its own O(L^2) double-precision evaluation: fp32, max-abs <= 1e-4, key-padding mask and causal."""
    import os
    import subprocess

    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cabi_host", "host_check")
    if not os.path.exists(exe):
        pytest.skip("tests/cabi_host/host_check is not built: run `python -m jvp_flash_attention_amd.build`")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0 and "host check ok" in r.stdout

"""``jvpfa_bwd_static``: the backward for callers that cannot allocate a workspace.  Called through the C
ABI and held, bit for bit, to what ``jvpfa_bwd`` gives for the same arguments with a workspace from the
caller (every kernel is deterministic), on two calls in a row, the second with a smaller input, so that
what the first left in the library's array cannot leak into the second."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _args(_lib, t, o, ot, M, mu, outs, causal, scale, ws):
    q, k, v, qt, kt, vt, go, gt = t
    a = _lib.BwdArgs()
    a.struct_size = C.sizeof(_lib.BwdArgs)
    a.p = _lib.make_problem(q, None, _lib.MASK_NONE, causal, scale)
    for name, x in (("q", q), ("k", k), ("v", v), ("qt", qt), ("kt", kt), ("vt", vt), ("o", o), ("ot", ot), ("M", M),
                    ("mu", mu), ("go", go), ("gt", gt), ("dq", outs[0]), ("dk", outs[1]), ("dv", outs[2]),
                    ("dqt", outs[3]), ("dkt", outs[4]), ("dvt", outs[5])):
        setattr(a, name, x.data_ptr())
    a.workspace = None if ws is None else ws.data_ptr()
    a.Hk, a.Lk = k.shape[1], k.shape[2]
    return a


def _both_ways(_lib, Z, H, L, D, dtype, causal, seed):
    lib = _lib.load()
    g = torch.Generator(device="cuda").manual_seed(seed)
    t = [torch.randn(Z, H, L, D, generator=g, device="cuda").to(dtype) for _ in range(8)]
    scale = D**-0.5
    o, ot, M, mu = _lib.backend().fwd(*t[:6], None, _lib.MASK_NONE, causal, scale)
    stream = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(lib.jvpfa_bwd_workspace_bytes(Z, H, L), device="cuda", dtype=torch.uint8)
    want = [torch.empty_like(t[0]) for _ in range(6)]
    _lib.check(lib.jvpfa_bwd(C.byref(_args(_lib, t, o, ot, M, mu, want, causal, scale, ws)), stream))
    got = [torch.full_like(t[0], float("nan")) for _ in range(6)]
    print(f"case static scratch Z{Z} H{H} L{L} D{D} {dtype} causal={causal}", flush=True)
    _lib.check(lib.jvpfa_bwd_static(C.byref(_args(_lib, t, o, ot, M, mu, got, causal, scale, None)), stream))
    torch.cuda.synchronize()
    for name, a_, b_ in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), got, want):
        assert torch.isfinite(a_).all(), name
        assert torch.equal(a_, b_), name


def test_static_scratch_backward_matches_the_workspace_backward_twice_in_a_row():
    from jvp_flash_attention_amd import _lib

    _both_ways(_lib, 2, 4, 700, 128, torch.bfloat16, False, 1)
    _both_ways(_lib, 1, 2, 130, 64, torch.float32, True, 2)  # smaller, other kernels, stale statistics behind it
    _both_ways(_lib, 2, 4, 700, 128, torch.bfloat16, True, 3)


def test_static_scratch_backward_under_graph_capture_allocates_nothing():
    """What the entry point is for: after one eager call on the device (which looks the array's address up), a call
    recorded into a HIP graph; replays with fresh inputs match the workspace backward bit for bit, and the device's
    free memory does not move across the eager calls that follow the first."""
    from jvp_flash_attention_amd import _lib

    lib = _lib.load()
    Z, H, L, D, dtype, causal = 2, 4, 300, 128, torch.bfloat16, True
    scale = D**-0.5
    g = torch.Generator(device="cuda").manual_seed(11)
    t = [torch.randn(Z, H, L, D, generator=g, device="cuda").to(dtype) for _ in range(8)]
    o, ot, M, mu = _lib.backend().fwd(*t[:6], None, _lib.MASK_NONE, causal, scale)
    ws = torch.empty(lib.jvpfa_bwd_workspace_bytes(Z, H, L), device="cuda", dtype=torch.uint8)
    got = [torch.empty_like(t[0]) for _ in range(6)]
    want = [torch.empty_like(t[0]) for _ in range(6)]
    args = _args(_lib, t, o, ot, M, mu, got, causal, scale, None)
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.jvpfa_bwd_static(C.byref(args), stream))  # the first call on this device resolves the array
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        _lib.check(lib.jvpfa_bwd_static(C.byref(args), stream))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "a later call changed the device's free memory"
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    print("case static scratch under capture", flush=True)
    with torch.cuda.graph(graph, stream=side):
        _lib.check(lib.jvpfa_bwd_static(C.byref(args), torch.cuda.current_stream().cuda_stream))
    for rep in range(3):
        g2 = torch.Generator(device="cuda").manual_seed(100 + rep)
        for x in t:
            x.copy_(torch.randn(Z, H, L, D, generator=g2, device="cuda").to(dtype))
        fo, fot, fM, fmu = _lib.backend().fwd(*t[:6], None, _lib.MASK_NONE, causal, scale)
        for dst, src in ((o, fo), (ot, fot), (M, fM), (mu, fmu)):
            dst.copy_(src)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _lib.check(lib.jvpfa_bwd(C.byref(_args(_lib, t, o, ot, M, mu, want, causal, scale, ws)), stream))
        torch.cuda.synchronize()
        for name, a_, b_ in zip(("dq", "dk", "dv", "dqt", "dkt", "dvt"), got, want):
            assert torch.equal(a_, b_), f"replay {rep}: {name}"


def test_static_scratch_backward_refuses_what_does_not_fit():
    from jvp_flash_attention_amd import _lib

    lib = _lib.load()
    rows = lib.jvpfa_bwd_static_max_rows()
    assert rows == 1 << 20
    a = _lib.BwdArgs()
    a.struct_size = C.sizeof(_lib.BwdArgs)
    a.p.Z, a.p.H, a.p.L, a.p.D = 1, 16, rows // 16 + 4, 64
    for name in ("q", "k", "v", "o", "M", "dq", "dk", "dv", "go"):
        setattr(a, name, 0x1000)
    assert lib.jvpfa_bwd_static(C.byref(a), None) == -8
    assert b"static scratch" in lib.jvpfa_error_string(-8)
    a.struct_size = 8
    assert lib.jvpfa_bwd_static(C.byref(a), None) == -7

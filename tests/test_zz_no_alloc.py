"""gg_gmm_no_alloc: the entry point that allocates nothing, with its partial tiles and arrival
counters in a static device array inside the library, against gg_gmm with a caller-provided
workspace of the same size.  Same kernels, same schedule, same order of additions: the outputs
must be equal bit for bit, on two calls in a row (the second smaller, on whatever the first left
in the array), and equal to the CPU oracle within the bf16 tolerance (rtol 1.6e-2, atol 1e-2
scaled to the data).  Collected last: it shares nothing with the other tests, and a failure here
must not hide them.  The property the entry point is named for is checked too: after gg_init the
free device memory does not move across the calls, and a call recorded into a HIP graph (where an
allocation would fail the capture) replays to the same bits."""
import ctypes
import os

import pytest
import torch

from test_gmm_gpu import GmmArgs, _c_abi, _gmm_args, check

pytestmark = pytest.mark.gpu

WORKSPACE_BYTES = 4096 + 256 * 256 * 256 * 4


def _case(seed, sizes, hin, hout, trans_a, trans_b):
    g = torch.Generator().manual_seed(seed)
    bs = torch.tensor(sizes, dtype=torch.int64)
    t = int(bs.sum())
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
    if trans_a:
        b = torch.randn(t, hout, generator=g).to(torch.bfloat16)
        shape = (len(sizes), hin, hout)
    else:
        b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
        shape = (t, hout)
    return bs, t, a, b, shape


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_no_alloc_entry_point_matches_workspace_entry_point(oracle, layout):
    trans_a, trans_b = layout
    lib = _c_abi()
    lib.gg_gmm_no_alloc.argtypes = [ctypes.c_void_p]
    ws = torch.zeros(WORKSPACE_BYTES, dtype=torch.uint8, device="cuda")
    assert lib.gg_init() == 0, lib.gg_last_error()   # per-device set-up happens here, not in a call
    # deep products with few tiles: both calls cut their tiles along the depth (the scratch is
    # in use); the second call is smaller in every dimension; the third has no pieces at all
    calls = [([300, 40, 0, 129], 6400, 264), ([70, 0, 5], 6272, 136), ([64, 64], 128, 128)]
    if trans_a:
        calls = [([14000, 0, 13000], 264, 520), ([6300, 6200], 136, 264), ([64, 64], 128, 128)]
    for n, (sizes, hin, hout) in enumerate(calls):
        print("[case] no alloc", layout, sizes, hin, hout, flush=True)
        bs, t, a, b, shape = _case(100 + n, sizes, hin, hout, trans_a, trans_b)
        da, db, dbs = a.cuda(), b.cuda(), bs.cuda()
        want = oracle.gmm_loop(a, b, bs, trans_a=trans_a, trans_b=trans_b)
        c_ws = torch.full(shape, 7.0, dtype=torch.bfloat16, device="cuda")
        c_static = torch.full(shape, -7.0, dtype=torch.bfloat16, device="cuda")
        args = _gmm_args(lib, da, db, c_ws, dbs, True, t, hin, hout, trans_a, trans_b, workspace=ws)
        assert lib.gg_gmm(ctypes.byref(args)) == 0, lib.gg_last_error()
        args = _gmm_args(lib, da, db, c_static, dbs, True, t, hin, hout, trans_a, trans_b)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        assert lib.gg_gmm_no_alloc(ctypes.byref(args)) == 0, lib.gg_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory moved across gg_gmm_no_alloc"
        assert torch.equal(c_static, c_ws), f"call {n}: static scratch and workspace disagree"
        check(c_static, want, f"call {n} against the oracle")
        # host-resident sizes through the same entry point
        c_host = torch.full(shape, 3.0, dtype=torch.bfloat16, device="cuda")
        args = _gmm_args(lib, da, db, c_host, bs, False, t, hin, hout, trans_a, trans_b)
        assert lib.gg_gmm_no_alloc(ctypes.byref(args)) == 0, lib.gg_last_error()
        torch.cuda.synchronize()
        assert torch.equal(c_host, c_ws)


def test_no_alloc_entry_point_rejects_a_workspace():
    lib = _c_abi()
    lib.gg_gmm_no_alloc.argtypes = [ctypes.c_void_p]
    bs, t, a, b, shape = _case(1, [8, 8], 16, 24, False, False)
    da, db = a.cuda(), b.cuda()
    c = torch.zeros(shape, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(WORKSPACE_BYTES, dtype=torch.uint8, device="cuda")
    args = _gmm_args(lib, da, db, c, bs, False, t, 16, 24, 0, 0, workspace=ws)
    assert lib.gg_gmm_no_alloc(ctypes.byref(args)) == -1 and b"workspace must be NULL" in lib.gg_last_error()


def test_no_alloc_entry_point_under_graph_capture(oracle):
    """Recorded into a HIP graph after gg_init (an allocation or a synchronisation inside the
    call would fail the capture), then replayed with new operand values and new device-resident
    sizes, with eager work between the replays: every replay equals the eager call bit for bit."""
    lib = _c_abi()
    lib.gg_gmm_no_alloc.argtypes = [ctypes.c_void_p]
    assert lib.gg_init() == 0, lib.gg_last_error()
    hin, hout, t = 6400, 264, 512
    g = torch.Generator().manual_seed(7)
    a = torch.empty(t, hin, dtype=torch.bfloat16, device="cuda")
    b = torch.empty(3, hin, hout, dtype=torch.bfloat16, device="cuda")
    dbs = torch.zeros(3, dtype=torch.int64, device="cuda")
    c = torch.zeros(t, hout, dtype=torch.bfloat16, device="cuda")
    c_eager = torch.zeros_like(c)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        args = _gmm_args(lib, a, b, c, dbs, True, t, hin, hout, False, False, stream=stream.cuda_stream)
        graph.capture_begin()
        rc = lib.gg_gmm_no_alloc(ctypes.byref(args))
        graph.capture_end()
    assert rc == 0, lib.gg_last_error()
    for n, sizes in enumerate([[300, 83, 129], [0, 512, 0], [17, 0, 40]]):
        print("[case] no alloc, graph replay", sizes, flush=True)
        a.copy_(torch.randn(t, hin, generator=g).to(torch.bfloat16))
        b.copy_(torch.randn(3, hin, hout, generator=g).to(torch.bfloat16))
        dbs.copy_(torch.tensor(sizes))
        c.fill_(5.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        c_eager.fill_(5.0)
        eager = _gmm_args(lib, a, b, c_eager, dbs, True, t, hin, hout, False, False)
        assert lib.gg_gmm_no_alloc(ctypes.byref(eager)) == 0, lib.gg_last_error()
        torch.cuda.synchronize()
        assert torch.equal(c, c_eager), f"replay {n} differs from the eager call"
        rows = sum(sizes)
        check(c[:rows], oracle.gmm_loop(a.cpu(), b.cpu(), torch.tensor(sizes))[:rows], f"replay {n} against the oracle")
        assert bool((c[rows:] == 5.0).all())

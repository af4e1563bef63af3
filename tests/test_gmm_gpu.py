"""GPU parity tests: the HIP path against the CPU oracle.

Layout of this file follows the reference's own tests (grouped_gemm/ops_test.py):
fixed sizes, variable sizes, the zero-size expert at Mixtral shape, the zero-K known
answer; then the five benchmark configurations, the C ABI called directly, the
on-device schedule bit-exact against the int64 closed forms, and edge cases.

Tolerance (every element): |got - want| <= 1e-2 * min(1, rms(want)) + 1.6e-2 * |want| against
the fp32-accumulated oracle: the absolute term is scaled down to the data, so outputs of small
numbers cannot pass by being small.  Small cases use the oracle on the CPU; full-size cases run
the oracle's per-expert loop with torch on the GPU in fp32 and add CPU fp64 checks on
sampled rows and entries so that no GPU library is trusted alone.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RTOL, ATOL = 1.6e-2, 1e-2


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from grouped_gemm import ops as _ops
    return _ops


def _announce(*what):
    print("[case]", *what, flush=True)


def check(got, want, what):
    got = got.float().cpu() if got.numel() < (1 << 24) else got.float()
    want = want.float().to(got.device)
    assert tuple(got.shape) == tuple(want.shape), (what, got.shape, want.shape)
    if got.numel() == 0:
        return
    atol = ATOL * min(1.0, float(want.double().pow(2).mean().sqrt()))
    viol = float(((got - want).abs() - (atol + RTOL * want.abs())).max())
    assert viol <= 0.0, f"{what}: outside rtol={RTOL} atol={atol} by {viol}"


def _gmm_flags(ops, a, b, bs, flags, trans_a=False, trans_b=False):
    c = ops.backend._allocate_output(a, b, bs, trans_a, trans_b)
    ops.backend.backend.gmm_with_flags(a, b, c, bs, trans_a, trans_b, flags)
    return c


def fp64_rows_check(a, b, sizes, trans_b, out, nrows=24, seed=0):
    """CPU float64 recomputation of a few output rows (first, last and random rows of
    random experts)."""
    g = torch.Generator().manual_seed(seed)
    starts = torch.cumsum(sizes, 0) - sizes
    for _ in range(nrows):
        e = int(torch.randint(len(sizes), (1,), generator=g))
        m = int(sizes[e])
        if m == 0:
            continue
        r = int(starts[e]) + [0, m - 1, int(torch.randint(m, (1,), generator=g))][_ % 3]
        w = b[e].double().cpu()
        want = a[r].double().cpu() @ (w.t() if trans_b else w)
        check(out[r].cpu(), want, f"fp64 row {r} of expert {e}")


def fp64_weight_gradient_check(lhs, rhs, sizes, bgrad, nblocks=12, seed=2):
    """CPU float64 recomputation of 16 x 16 blocks of the weight gradient of sampled experts
    (first, last and random rows and columns): lhs_e^T @ rhs_e, independent of any GPU library."""
    g = torch.Generator().manual_seed(seed)
    starts = torch.cumsum(sizes, 0) - sizes
    hin, hout = lhs.shape[1], rhs.shape[1]
    for n in range(nblocks):
        e = int(torch.randint(len(sizes), (1,), generator=g))
        s, m = int(starts[e]), int(sizes[e])
        i0 = [0, hin - 16, int(torch.randint(hin - 15, (1,), generator=g))][n % 3]
        j0 = [hout - 16, 0, int(torch.randint(hout - 15, (1,), generator=g))][n % 3]
        want = lhs[s:s + m, i0:i0 + 16].double().cpu().t() @ rhs[s:s + m, j0:j0 + 16].double().cpu()
        got = bgrad[e, i0:i0 + 16, j0:j0 + 16].cpu()
        check(got, want, f"fp64 weight gradient block ({i0}, {j0}) of expert {e}")


# ------------------------------------------------ mirrors of the reference's tests

_PROBLEMS = [(z, m, k, n, tb, dev)
             for (z, m, k, n) in [(1, 128, 128, 128), (8, 128, 128, 128), (16, 128, 128, 128),
                                  (1, 128, 256, 512), (8, 128, 256, 512), (16, 128, 256, 512)]
             for tb in (False, True) for dev in (False, True)]          # ops_test.py:20-36


def _run_fwd_bwd(ops, oracle, a, b, sizes, trans_b, on_device, legacy_rule=True):
    bs = sizes.cuda() if on_device else sizes
    a = a.cuda().requires_grad_(True)
    b = b.cuda().requires_grad_(True)
    out = ops.gmm(a, b, bs, trans_b)
    grad = torch.ones_like(out)                                          # out.sum().backward()
    out.backward(grad)
    want, want_ag, want_bg = oracle.gmm_autograd_loop(a.detach().cpu(), b.detach().cpu(), sizes,
                                                      trans_b, grad.cpu())
    check(out.detach(), want, "forward")
    check(a.grad, want_ag, "agrad")
    check(b.grad, want_bg, "bgrad")
    if legacy_rule:   # the reference's own acceptance rule, against its own bf16 oracle shape
        assert oracle.allclose_ops_test(out.detach(), want.to(torch.bfloat16))


@pytest.mark.parametrize("z,m,k,n,trans_b,on_device", _PROBLEMS)
def test_fixed_sizes(ops, oracle, z, m, k, n, trans_b, on_device):       # ops_test.py:59-80
    _announce("fixed", z, m, k, n, trans_b, on_device)
    torch.manual_seed(0)
    a = oracle.ops_test_randn(z, m, k).view(-1, k)
    b = oracle.ops_test_randn(z, n, k) if trans_b else oracle.ops_test_randn(z, k, n)
    _run_fwd_bwd(ops, oracle, a, b, torch.tensor([m] * z), trans_b, on_device)


@pytest.mark.parametrize("z,m,k,n,trans_b,on_device", _PROBLEMS)
def test_variable_sizes(ops, oracle, z, m, k, n, trans_b, on_device):    # ops_test.py:82-109
    _announce("variable", z, m, k, n, trans_b, on_device)
    torch.manual_seed(0)
    a = oracle.ops_test_randn(z, m, k).view(-1, k)
    b = oracle.ops_test_randn(z, n, k) if trans_b else oracle.ops_test_randn(z, k, n)
    dist = torch.rand(z)
    dist /= dist.sum()
    sizes = (dist * m).to(torch.long)
    sizes[-1] += m * z - sizes.sum()
    assert sizes.sum() == m * z
    _run_fwd_bwd(ops, oracle, a, b, sizes, trans_b, on_device)


@pytest.mark.parametrize("scale", [1.0, 37.0])
@pytest.mark.parametrize("trans_b", [False, True])
def test_variable_sizes_randn(ops, oracle, trans_b, scale):
    # same shapes with signed, O(1) data so cancellation and the tolerance are exercised
    _announce("variable randn", trans_b, scale)
    g = torch.Generator().manual_seed(1)
    z, m, k, n = 8, 100, 264, 520
    sizes = torch.tensor([0, 1, 255, 256, 257, 3, 0, 28])
    a = (torch.randn(int(sizes.sum()), k, generator=g) * scale).to(torch.bfloat16)
    b = torch.randn(z, n, k, generator=g).to(torch.bfloat16) if trans_b else \
        torch.randn(z, k, n, generator=g).to(torch.bfloat16)
    # tolerance scales with the data: compare after dividing the scale back out
    bs = sizes
    out = ops.gmm(a.cuda(), b.cuda(), bs, trans_b)
    want = oracle.gmm_c(a, b, sizes, trans_b=trans_b)[0]
    check(out / scale, want / scale, "forward")


@pytest.mark.parametrize("on_device", [False, True])
def test_zero_size_expert_at_mixtral_shape(ops, oracle, on_device):       # ops_test.py:115-141
    _announce("zero size", on_device)
    torch.manual_seed(0)
    m, k, n, e = 16384, 4096, 14336, 8
    a = oracle.ops_test_randn(e, m // e, k).view(-1, k).cuda().requires_grad_(True)
    b = oracle.ops_test_randn(e, k, n).cuda().requires_grad_(True)
    sizes = torch.tensor([219, 2246, 5, 8103, 1, 1117, 4693, 0]).to(torch.long)
    bs = sizes.cuda() if on_device else sizes
    out = ops.gmm(a, b, bs)
    out.sum().backward()
    ones = torch.ones_like(out)
    with torch.no_grad():
        want = oracle.gmm_loop(a.detach(), b.detach(), sizes)                        # fp32, on the GPU
        want_ag = oracle.gmm_loop(ones, b.detach(), sizes, trans_b=True)
        want_bg = oracle.gmm_loop(a.detach(), ones, sizes, trans_a=True)
    check(out.detach(), want, "forward")
    check(a.grad, want_ag, "agrad")
    check(b.grad, want_bg, "bgrad")
    assert (b.grad[7] == 0).all(), "expert without tokens must get a zero weight gradient"
    fp64_rows_check(a.detach(), b.detach(), sizes, False, out.detach())
    assert oracle.allclose_ops_test(out.detach(), want.to(torch.bfloat16))


@pytest.mark.parametrize("on_device", [False, True])
def test_zero_k_known_answer(ops, on_device):                             # ops_test.py:143-158
    _announce("zero k", on_device)
    sz, total = 128, 192
    a = torch.ones(total, sz).cuda().to(torch.bfloat16)
    b = torch.ones(total, sz).cuda().to(torch.bfloat16)
    c = torch.ones(4, sz, sz).cuda().to(torch.bfloat16)
    bs = torch.tensor([0, 128, 0, 64]).to(torch.long)
    if on_device:
        bs = bs.cuda()
    ret = ops.backend.gmm(a, b, bs, trans_a=True, c=c)
    assert ret is c
    assert (c[0] == 0).all() and (c[1] == 128).all() and (c[2] == 0).all() and (c[3] == 64).all()


# ------------------------------------------------------ the benchmark configurations

def test_config1_golden_fixture(ops):
    _announce("config1 fixture")
    import importlib.util
    spec = importlib.util.spec_from_file_location(
        "make_config1", os.path.join(ROOT, "tests", "golden", "make_config1.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    a, b, grad, sizes = mod.inputs()
    gold = np.load(os.path.join(ROOT, "tests", "golden", "config1.npz"))
    a = a.cuda().requires_grad_(True)
    b = b.cuda().requires_grad_(True)
    out = ops.gmm(a, b, sizes)
    out.backward(grad.cuda())
    check(out.detach()[::8], torch.from_numpy(gold["fwd"]), "forward")
    check(a.grad[::8], torch.from_numpy(gold["agrad"]), "agrad")
    check(b.grad[:, ::8], torch.from_numpy(gold["bgrad"]), "bgrad")


@pytest.mark.parametrize("config,shrink", [(2, 16), (3, 8), (4, 16), (5, 16)])
@pytest.mark.parametrize("on_device", [False, True])
def test_configs_shrunk_against_cpu_oracle(ops, oracle, config, shrink, on_device):
    _announce("config", config, "shrink", shrink, on_device)
    from grouped_gemm_amd import workloads
    w = workloads.make(config, device="cuda", shrink=shrink)
    bs = w.batch_sizes.cuda() if on_device else w.batch_sizes
    a_cpu, b_cpu, g_cpu = w.a.cpu(), w.b.cpu(), w.grad.cpu()
    if "fwd" in w.gemms:
        out = ops.backend.gmm(w.a, w.b, bs, trans_b=w.trans_b)
        check(out, oracle.gmm_loop(a_cpu, b_cpu, w.batch_sizes, trans_b=w.trans_b), "forward")
    if "agrad" in w.gemms:
        ag = ops.backend.gmm(w.grad, w.b, bs, trans_b=not w.trans_b)
        check(ag, oracle.gmm_loop(g_cpu, b_cpu, w.batch_sizes, trans_b=not w.trans_b), "agrad")
    if "bgrad" in w.gemms:
        lhs, rhs = (w.grad, w.a) if w.trans_b else (w.a, w.grad)
        bg = ops.backend.gmm(lhs, rhs, bs, trans_a=True)
        want = oracle.gmm_loop(lhs.cpu(), rhs.cpu(), w.batch_sizes, trans_a=True)
        check(bg, want, "bgrad")
        empty = (w.batch_sizes == 0).nonzero().flatten().tolist()
        for e in empty:
            assert (bg[e] == 0).all()


def _full_size_case(ops, oracle, config):
    from grouped_gemm_amd import workloads
    w = workloads.make(config, device="cuda")
    sizes = w.batch_sizes
    bs = sizes.cuda()
    results = {}
    with torch.no_grad():
        if "fwd" in w.gemms:
            out = ops.backend.gmm(w.a, w.b, bs, trans_b=w.trans_b)
            check(out, oracle.gmm_loop(w.a, w.b, sizes, trans_b=w.trans_b), "forward")
            fp64_rows_check(w.a, w.b, sizes, w.trans_b, out)
            results["fwd"] = out
        if "agrad" in w.gemms:
            ag = ops.backend.gmm(w.grad, w.b, bs, trans_b=not w.trans_b)
            check(ag, oracle.gmm_loop(w.grad, w.b, sizes, trans_b=not w.trans_b), "agrad")
            fp64_rows_check(w.grad, w.b, sizes, not w.trans_b, ag, seed=1)
            del ag
        if "bgrad" in w.gemms:
            lhs, rhs = (w.grad, w.a) if w.trans_b else (w.a, w.grad)
            bg = ops.backend.gmm(lhs, rhs, bs, trans_a=True)
            starts = torch.cumsum(sizes, 0) - sizes
            # expert by expert to bound the fp32 copies
            for e in range(len(sizes)):
                s, m = int(starts[e]), int(sizes[e])
                want = lhs[s:s + m].float().t() @ rhs[s:s + m].float()
                check(bg[e], want, f"bgrad expert {e}")
            fp64_weight_gradient_check(lhs, rhs, sizes, bg)
            # host-resident sizes must give the very same bits as device-resident ones
            bg2 = ops.backend.gmm(lhs, rhs, sizes, trans_a=True)
            assert torch.equal(bg, bg2)
    return w, results


def test_config2_mixtral_full_size(ops, oracle):
    _announce("config2 full")
    w, res = _full_size_case(ops, oracle, 2)
    # linearity in a at full size: gmm(2a, b) == 2 gmm(a, b) bit for bit (power of two)
    out2 = ops.backend.gmm(w.a * 2, w.b, w.batch_sizes.cuda())
    assert torch.equal(out2, res["fwd"] * 2)


def test_config3_ragged_full_size(ops, oracle):
    _announce("config3 full")
    w, res = _full_size_case(ops, oracle, 3)
    assert int((w.batch_sizes == 0).sum()) >= 4
    # each expert on its own (one group per call) gives the same bits as the grouped call when
    # both keep their tiles whole (the depth order of every output element is then the same);
    # with the last round cut along the depth the two differ by fp32 summation order only
    starts = torch.cumsum(w.batch_sizes, 0) - w.batch_sizes
    whole_flag = ops.backend.backend.flag_whole_tiles
    grouped_whole = _gmm_flags(ops, w.a, w.b, w.batch_sizes.cuda(), whole_flag)
    check(grouped_whole, res["fwd"].float(), "whole tiles against depth pieces")
    for e in [int(torch.argmax(w.batch_sizes)), int(torch.argmin(w.batch_sizes + (w.batch_sizes == 0) * 10 ** 9))]:
        s, m = int(starts[e]), int(w.batch_sizes[e])
        a_e, b_e = w.a[s:s + m].contiguous(), w.b[e:e + 1].contiguous()
        alone = _gmm_flags(ops, a_e, b_e, torch.tensor([m]), whole_flag)
        assert torch.equal(alone, grouped_whole[s:s + m])
        check(ops.backend.gmm(a_e, b_e, torch.tensor([m])), alone.float(), f"expert {e} alone, depth pieces")


@pytest.mark.parametrize("shrink", [8, 1])
def test_config3_ragged_weight_gradient(ops, oracle, shrink):
    # the weight gradient of the ragged configuration: Zipf depths from 0 to several thousand rows,
    # at least four empty groups, tiles handed out by descending depth.  Shrunk against the CPU
    # oracle; at full size against fp32 per expert on the GPU and CPU float64 blocks.
    _announce("config3 weight gradient, shrink", shrink)
    from grouped_gemm_amd import workloads
    w = workloads.make(3, device="cuda", shrink=shrink)
    sizes = w.batch_sizes
    assert int((sizes == 0).sum()) >= 4
    bg = ops.backend.gmm(w.a, w.grad, sizes.cuda(), trans_a=True)
    assert torch.equal(bg, ops.backend.gmm(w.a, w.grad, sizes, trans_a=True))
    if shrink > 1:
        check(bg, oracle.gmm_loop(w.a.cpu(), w.grad.cpu(), sizes, trans_a=True), "weight gradient")
    else:
        starts = torch.cumsum(sizes, 0) - sizes
        for e in range(len(sizes)):
            s, m = int(starts[e]), int(sizes[e])
            check(bg[e], w.a[s:s + m].float().t() @ w.grad[s:s + m].float(), f"expert {e}")
        fp64_weight_gradient_check(w.a, w.grad, sizes, bg)
    for e in (sizes == 0).nonzero().flatten().tolist():
        assert (bg[e] == 0).all()


def test_config4_weight_gradient_full_size(ops, oracle):
    _announce("config4 full")
    _full_size_case(ops, oracle, 4)


def test_config5_deepseek_share_full_size_autograd(ops, oracle):
    _announce("config5 full")
    from grouped_gemm_amd import workloads
    w = workloads.make(5, device="cuda")
    sizes = w.batch_sizes
    a = w.a.requires_grad_(True)
    b = w.b.requires_grad_(True)
    out = ops.gmm(a, b, sizes.cuda(), True)
    out.backward(w.grad)
    with torch.no_grad():
        check(out.detach(), oracle.gmm_loop(w.a.detach(), w.b.detach(), sizes, trans_b=True), "forward")
        check(a.grad, oracle.gmm_loop(w.grad, w.b.detach(), sizes, trans_b=False), "agrad")
        starts = torch.cumsum(sizes, 0) - sizes
        for e in range(len(sizes)):
            s, m = int(starts[e]), int(sizes[e])
            want = w.grad[s:s + m].float().t() @ w.a.detach()[s:s + m].float()
            check(b.grad[e], want, f"bgrad expert {e}")
        fp64_weight_gradient_check(w.grad, w.a.detach(), sizes, b.grad)
        fp64_rows_check(w.a.detach(), w.b.detach(), sizes, True, out.detach())


def _random_cases(n, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    cases = []
    for _ in range(n):
        e = r(1, 12)
        kind = r(0, 3)
        if kind == 0:      # many tiny groups
            sizes = [r(0, 9) for _ in range(e)]
        elif kind == 1:    # around the tile heights
            sizes = [r(0, 3) * 128 + r(-2, 2) for _ in range(e)]
        elif kind == 2:    # one big group among empties
            sizes = [0] * e
            sizes[r(0, e - 1)] = r(200, 900)
        else:
            sizes = [r(0, 400) for _ in range(e)]
        sizes = [max(0, s) for s in sizes]
        cases.append((sizes, 8 * r(1, 40), 8 * r(1, 70)))
    return cases


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_random_shapes_against_cpu_oracle(ops, oracle, layout):
    # depths that are not multiples of 64, widths that are not multiples of 256, sizes around
    # the tile heights, host- and device-resident sizes alternating
    trans_a, trans_b = layout
    for idx, (sizes, hin, hout) in enumerate(_random_cases(24, seed=17 + int(trans_a) + 2 * int(trans_b))):
        _announce("random", layout, sizes, hin, hout)
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
        if trans_a:
            b = torch.randn(t, hout, generator=g).to(torch.bfloat16)
        else:
            b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
        dev_bs = bs.cuda() if idx % 2 else bs
        out = ops.backend.gmm(a.cuda(), b.cuda(), dev_bs, trans_a=trans_a, trans_b=trans_b)
        want = oracle.gmm_loop(a, b, bs, trans_a=trans_a, trans_b=trans_b)
        check(out, want, f"case {idx}: sizes={sizes} hin={hin} hout={hout}")


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("on_device", [False, True])
def test_every_row_block_count(ops, oracle, trans_b, on_device):
    # One call whose groups cover every count of 32-row blocks a tile can have, on both sides of
    # each boundary, and groups whose rows are split evenly over two, three and five tiles; the
    # value of each output row names its input row, so a row that lands in the wrong place shows.
    sizes = [1, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 159, 160, 161, 191, 192, 193,
             223, 224, 225, 255, 256, 257, 289, 300, 320, 321, 511, 512, 513, 700, 0, 1025, 1281]
    hin, hout = 192, 328
    bs = torch.tensor(sizes, dtype=torch.int64)
    t = int(bs.sum())
    g = torch.Generator().manual_seed(5)
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
    b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
    _announce("row blocks", trans_b, on_device)
    out = ops.backend.gmm(a.cuda(), b.cuda(), bs.cuda() if on_device else bs, trans_b=trans_b)
    check(out, oracle.gmm_loop(a, b, bs, trans_b=trans_b), "every row block count")
    # exact: one-hot rows times an identity-like weight give back the row index pattern
    eye = torch.zeros(len(sizes), hin, hout)
    eye[:, :, :hin] = torch.eye(hin)
    wb = (eye.transpose(1, 2).contiguous() if trans_b else eye).to(torch.bfloat16)
    idx = torch.arange(t) % 251
    rows = torch.zeros(t, hin)
    rows[torch.arange(t), idx % hin] = (idx % 127 + 1).float()
    got = ops.backend.gmm(rows.to(torch.bfloat16).cuda(), wb.cuda(), bs.cuda() if on_device else bs,
                          trans_b=trans_b).float().cpu()
    want = torch.zeros(t, hout)
    want[:, :hin] = rows
    assert torch.equal(got, want)


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_last_round_pieces_against_whole_tiles(ops, oracle, layout):
    # A launch with fewer tiles than workgroups cuts its tiles into pieces for the idle
    # workgroups (along the depth, summed through the workspace in a fixed order); the flag keeps
    # them whole.  The two differ only in the order of fp32 additions: both must match the oracle,
    # agree with each other far inside the tolerance, and each be the same bits on every call.
    trans_a, trans_b = layout
    whole_flag = ops.backend.backend.flag_whole_tiles
    cases = _random_cases(16, seed=91 + int(trans_b) + 2 * int(trans_a))
    if trans_a:   # the depth is the groups' rows: deep groups, so that the cut runs along the depth
        cases += [([13000, 0, 12500], 264, 520), ([6200, 6300], 136, 264), ([30000], 72, 200)]
    for idx, (sizes, hin, hout) in enumerate(cases):
        hin = hin * 8 if idx % 2 and idx < 16 else hin     # deep enough for several depth pieces
        _announce("pieces", layout, sizes, hin, hout)
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(torch.bfloat16).cuda()
        if trans_a:
            b = torch.randn(t, hout, generator=g).to(torch.bfloat16).cuda()
        else:
            b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16).cuda()
        dev_bs = bs.cuda() if idx % 2 else bs
        cut = _gmm_flags(ops, a, b, dev_bs, 0, trans_a, trans_b)
        whole = _gmm_flags(ops, a, b, dev_bs, whole_flag, trans_a, trans_b)
        want = oracle.gmm_loop(a.cpu(), b.cpu(), bs, trans_a=trans_a, trans_b=trans_b)
        check(whole, want, f"whole, case {idx}")
        check(cut, want, f"cut, case {idx}")
        if want.numel():    # one bf16 rounding step apart at most, relative to the largest value
            assert float((cut.float() - whole.float()).abs().max()) <= 2 ** -7 * float(want.abs().max())
        assert torch.equal(cut, _gmm_flags(ops, a, b, dev_bs, 0, trans_a, trans_b))


def test_deep_groups_of_a_weight_gradient_are_cut_first(oracle):
    # Weight gradient with one or two groups much deeper than the rest: their tiles would set the
    # length of the launch, so they are cut along the depth into 2 or 4 pieces that go out first,
    # one per workgroup; whichever piece arrives last adds the partial tiles up, after its
    # workgroup's other tiles.  Through the C ABI with a workspace of the test's own: the cut
    # leaves partial tiles in it (exactly as many as the plan says) and the arrival counters at
    # zero.  Against the oracle, against whole tiles (fp32 summation order apart), the same bits
    # on every call, zero-row groups all zero.
    lib = _c_abi()
    cases = [  # sizes, hidden_in, hidden_out, tiles cut, pieces each
        ([14000, 300, 200, 0, 150, 6500, 100, 120], 264, 520, 6, 4),   # the group of 6500 rows is too shallow for 4 pieces
        ([7000, 100, 6800], 136, 264, 4, 2),                           # two deep groups, 2 pieces
        ([64] * 50 + [20000] + [64] * 50, 256, 256, 1, 4),
        ([13000, 50, 12800], 1024, 2048, 64, 4),                       # more deep tiles than a round has room for
        ([6080, 100, 90], 264, 520, 0, 0),                             # 95 slices: too shallow to pay for a fix-up
        ([7000, 7000, 7000, 7000], 2048, 4096, 0, 0),                  # deep, but no deeper than a workgroup's share
    ]
    slot = 256 * 256
    for idx, (sizes, hin, hout, cut_tiles, pieces) in enumerate(cases):
        _announce("deep groups first", sizes if len(sizes) < 10 else len(sizes), hin, hout)
        g = torch.Generator().manual_seed(300 + idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(torch.bfloat16).cuda()
        b = torch.randn(t, hout, generator=g).to(torch.bfloat16).cuda()
        dbs = bs.cuda() if idx % 2 else bs
        shape = (len(sizes), hin, hout)
        ws = torch.zeros(1024 + 256 * slot, dtype=torch.float32, device="cuda")
        cut = torch.full(shape, 7.0, dtype=torch.bfloat16, device="cuda")
        args = _gmm_args(lib, a, b, cut, dbs, bool(idx % 2), t, hin, hout, True, False, workspace=ws)
        assert lib.gg_gmm(ctypes.byref(args)) == 0, lib.gg_last_error()
        torch.cuda.synchronize()
        assert not bool(ws[:1024].any()), "arrival counters left nonzero"
        # (a launch with fewer tiles than workgroups may also cut its last round: the deep-group
        # cut comes instead of that one, so the count below is either the one or the other)
        used = int((ws[1024:].view(256, slot) != 0).any(dim=1).sum())
        if cut_tiles:
            assert used == cut_tiles * pieces, f"case {idx}: {used} partial tiles in the workspace"
        whole = torch.full(shape, 7.0, dtype=torch.bfloat16, device="cuda")
        args = _gmm_args(lib, a, b, whole, dbs, bool(idx % 2), t, hin, hout, True, False, workspace=ws, flags=1)
        assert lib.gg_gmm(ctypes.byref(args)) == 0, lib.gg_last_error()
        again = torch.full(shape, 7.0, dtype=torch.bfloat16, device="cuda")
        args = _gmm_args(lib, a, b, again, dbs, bool(idx % 2), t, hin, hout, True, False, workspace=ws)
        assert lib.gg_gmm(ctypes.byref(args)) == 0, lib.gg_last_error()
        torch.cuda.synchronize()
        assert torch.equal(cut, again)
        if hin * hout <= 1024 * 2048:
            want = oracle.gmm_loop(a.cpu(), b.cpu(), bs, trans_a=True)
            check(whole, want, f"whole, case {idx}")
            check(cut, want, f"cut, case {idx}")
        else:   # at this size the per-expert fp32 product on the GPU stands in for the CPU loop
            want = torch.stack([a[s:e].float().t() @ b[s:e].float() for s, e in
                                zip((bs.cumsum(0) - bs).tolist(), bs.cumsum(0).tolist())])
            check(cut, want, f"cut, case {idx}")
        assert float((cut.float() - whole.float()).abs().max()) <= 2 ** -7 * float(whole.float().abs().max())
        for e, rows in enumerate(sizes):
            if rows == 0:
                assert not bool(cut[e].any())


def test_c_abi_without_workspace_cuts_rows_bit_exactly(oracle):
    # gg_gmm_bf16 brings no workspace: the tiles of the last round are cut along their rows, which
    # leaves the depth order of every output element alone, so the result equals the whole-tile
    # one bit for bit.
    lib = _c_abi()
    whole_flag = 1
    for idx, (sizes, hin, hout) in enumerate(_random_cases(8, seed=77)):
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(torch.bfloat16).cuda()
        b = torch.randn(len(sizes), hin, hout, generator=g).to(torch.bfloat16).cuda()
        c1 = torch.zeros(t, hout, dtype=torch.bfloat16, device="cuda")
        c2 = torch.zeros_like(c1)
        _announce("row pieces", sizes, hin, hout)
        rc = lib.gg_gmm_bf16(a.data_ptr(), b.data_ptr(), c1.data_ptr(), bs.data_ptr(), 0, len(sizes), t, hin, hout,
                             0, 0, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.gg_last_error()
        args = _gmm_args(lib, a, b, c2, bs, False, t, hin, hout, 0, 0, flags=whole_flag)
        assert lib.gg_gmm(ctypes.byref(args)) == 0, lib.gg_last_error()
        torch.cuda.synchronize()
        assert torch.equal(c1, c2)
        check(c1, oracle.gmm_loop(a.cpu(), b.cpu(), bs), f"case {idx}")


@pytest.mark.parametrize("trans_b", [False, True])
def test_tiles_by_tile_rows_against_group_order(ops, oracle, trans_b):
    # Many short groups of one, two and three tile rows, deep tiles: their tiles are handed out by
    # ascending number of tile rows (see test_schedule_bit_exact for the order itself).  Every
    # tile is computed as it would be in group order (no workspace: no depth pieces), so the
    # outputs are equal bit for bit to those of GG_FLAG_GROUP_ORDER, and right against the oracle
    # (on the first 40 groups: the whole product would keep the CPU busy for a quarter of a minute).
    # With empty groups in the second case; device- and host-resident sizes.
    lib = _c_abi()
    cases = [([200 + (37 * i) % 180 for i in range(256)], 2048, 1024),
             ([0 if i % 7 == 0 else 100 + (53 * i) % 600 for i in range(300)], 2056, 1032)]
    for idx, (sizes, hin, hout) in enumerate(cases):
        _announce("tiles by tile rows", trans_b, len(sizes), hin, hout)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        assert _handed_out_by_tile_rows(sizes, hin, -(-hout // 256), 256)
        g = torch.Generator(device="cuda").manual_seed(40 + idx)   # (operands of a gigabyte: made on the device)
        da = torch.randn(t, hin, generator=g, device="cuda").to(torch.bfloat16)
        db = (torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g, device="cuda")
              * hin ** -0.5).to(torch.bfloat16)
        dbs = bs.cuda() if idx == 0 else bs
        by_tile_rows = torch.full((t + 1, hout), 7.0, dtype=torch.bfloat16, device="cuda")
        args = _gmm_args(lib, da, db, by_tile_rows, dbs, idx == 0, t, hin, hout, False, trans_b)
        assert lib.gg_gmm(ctypes.byref(args)) == 0, lib.gg_last_error()
        in_order = torch.full((t + 1, hout), 7.0, dtype=torch.bfloat16, device="cuda")
        args = _gmm_args(lib, da, db, in_order, dbs, idx == 0, t, hin, hout, False, trans_b, flags=8)
        assert lib.gg_gmm(ctypes.byref(args)) == 0, lib.gg_last_error()
        torch.cuda.synchronize()
        assert torch.equal(by_tile_rows, in_order)
        assert bool((by_tile_rows[t] == 7.0).all())
        head = int(bs[:40].sum())
        check(by_tile_rows[:head], oracle.gmm_loop(da[:head].cpu(), db[:40].cpu(), bs[:40], trans_b=trans_b), f"case {idx}")


# ----------------------------------------------------------------- schedule, bit-exact

SCHED_CASES = [
    ([128] * 8, 128, 128),
    ([219, 2246, 5, 8103, 1, 1117, 4693, 0], 4096, 14336),
    ([0, 0, 0], 64, 64),
    ([256] * 256, 7168, 2048),          # b offsets pass 2**31 elements
    ([1] * 512, 8, 8),
    ([70000, 0, 3, 70000], 2048, 1408),
    # many short groups of one, two and three tile rows and deep tiles: handed out by their
    # number of tile rows (NN and NT); with empty groups; with one group of more than 8 tile rows,
    # which keeps the group order; with shallow tiles, which do too
    ([200 + (37 * i) % 180 for i in range(256)], 7168, 2048),
    ([0 if i % 7 == 0 else 100 + (53 * i) % 600 for i in range(300)], 2048, 1024),
    ([2100 if i == 77 else 200 + (37 * i) % 180 for i in range(256)], 2048, 2048),
    ([200 + (37 * i) % 180 for i in range(256)], 1024, 2048),
]


def _handed_out_by_tile_rows(sizes, hin, tiles_n, bm):
    # the library's rule (gmm_api.hip, order_by_tile_rows): many groups, short on average, deep
    # tiles, and enough of them for several rounds; and the kernel's: no group of more than 8 tile rows
    grid = torch.cuda.get_device_properties(0).multi_processor_count
    num_groups, tokens = len(sizes), sum(sizes)
    return (num_groups >= 32 and tokens < 2048 * num_groups and hin >= 2048 and
            (tokens // bm + num_groups // 2) * tiles_n >= 4 * grid and max(sizes) <= 8 * bm)


@pytest.mark.parametrize("sizes,hin,hout", SCHED_CASES)
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
@pytest.mark.parametrize("on_device", [False, True])
def test_schedule_bit_exact(ops, oracle, sizes, hin, hout, layout, on_device):
    trans_a, trans_b = layout
    _announce("schedule", len(sizes), hin, hout, layout, on_device)
    bs = torch.tensor(sizes, dtype=torch.int64)
    tokens = int(bs.sum())
    got = ops.backend.debug_schedule(bs.cuda() if on_device else bs, tokens, hin, hout, trans_a, trans_b).cpu().numpy()
    want = oracle.table_closed(sizes, hin, hout, trans_a, trans_b)
    np.testing.assert_array_equal(got[:, :9], want)
    assert np.array_equal(want, oracle.table_walk(sizes, hin, hout, trans_a, trans_b)[0])
    # tiles: two classes (all tiles but the runt rows, then the runt rows), each consecutive and
    # non-overlapping, together enough to cover each group's output
    first_class = got[:, 10] - got[:, 13]
    if trans_a:
        # weight gradient: every group has the same number of tiles and they are handed out by
        # descending depth, groups of equal depth in their own order (the reference's stable sort
        # by k, csrc/grouped_gemm.cu:193-207): a permutation, depths non-increasing along it
        position = np.empty(len(sizes), dtype=np.int64)
        position[np.argsort(-np.array(sizes), kind="stable")] = np.arange(len(sizes))
        assert np.array_equal(got[:, 9], position * first_class)
        by_position = np.argsort(got[:, 9], kind="stable")
        assert sorted(by_position.tolist()) == list(range(len(sizes)))
        assert (np.diff(np.array(sizes)[by_position]) <= 0).all()
    lib = ctypes.CDLL(os.path.join(ROOT, "grouped_gemm_amd", "libgrouped_gemm_hip.so"))
    bm, bn, bk = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    lib.gg_tile_shape(ctypes.c_int64(len(sizes)), ctypes.c_int64(tokens), int(trans_a), int(trans_b),
                      ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(bk))
    m, n = got[:, 0], got[:, 1]
    if not trans_a:
        # NN and NT: in group order, or, for many short groups, by ascending number of tile rows,
        # groups of equal number in their own order; both prefix sums count in that order
        order = np.arange(len(sizes))
        if _handed_out_by_tile_rows(sizes, hin, -(-hout // bn.value), bm.value):
            tile_rows = -(-np.array(sizes) // bm.value)
            order = np.argsort(tile_rows, kind="stable")
            if len(set(tile_rows.tolist())) > 2:
                assert not np.array_equal(order, np.arange(len(sizes))), "the case should exercise the order"
        want_first = np.empty(len(sizes), dtype=np.int64)
        want_first[order] = (np.cumsum(first_class[order]) - first_class[order])
        assert np.array_equal(got[:, 9], want_first)
        want_runt = np.empty(len(sizes), dtype=np.int64)
        want_runt[order] = first_class.sum() + np.cumsum(got[order, 13]) - got[order, 13]
        assert np.array_equal(got[:, 12], want_runt)
    else:
        assert np.array_equal(got[:, 12], first_class.sum() + np.cumsum(got[:, 13]) - got[:, 13])
    assert np.array_equal(got[:, 11], np.array(sizes))
    assert np.array_equal(got[:, 10], -(-m // bm.value) * -(-n // bn.value))
    # a runt row is the last tile row of a group of at least two, at most half as many 32-row
    # blocks tall as the others
    if not trans_a:
        tiles_n = -(-n // bn.value)
        tiles_m = -(-m // bm.value)
        height = -(-(-(-m // np.maximum(tiles_m, 1))) // 32) * 32
        last_blocks = -(-(m - (tiles_m - 1) * height) // 32)
        runt = (tiles_m >= 2) & (2 * last_blocks <= height // 32)
        assert np.array_equal(got[:, 13], runt * tiles_n)
    else:
        assert not got[:, 13].any()


def test_schedule_clips_rows_past_tokens(ops):
    # device-resident sizes that claim more rows than `a` has: clipped, never followed
    bs = torch.tensor([100, 100, 100], dtype=torch.int64).cuda()
    got = ops.backend.debug_schedule(bs, 150, 64, 64, False, False).cpu().numpy()
    assert got[:, 11].tolist() == [100, 50, 0]
    assert got[:, 6].tolist() == [0, 100 * 64, 150 * 64]


def test_schedule_saturates_huge_and_negative_sizes(ops):
    # sizes from an uninitialised buffer: each is clamped to [0, tokens] before it enters a sum, so
    # no sum wraps, no group starts before row 0 and none reaches past `tokens`
    big = (1 << 63) - 1
    for sizes, want_rows, want_start in [
        ([big, big, 5], [150, 0, 0], [0, 150, 150]),
        ([-big, 7, big], [0, 7, 143], [0, 0, 7]),
        ([-1, -(1 << 62), 150, 3], [0, 0, 150, 0], [0, 0, 0, 150]),
    ]:
        bs = torch.tensor(sizes, dtype=torch.int64).cuda()
        for trans_a in (False, True):
            got = ops.backend.debug_schedule(bs, 150, 64, 64, trans_a, False).cpu().numpy()
            assert got[:, 11].tolist() == want_rows, (sizes, got[:, 11])
            assert got[:, 6].tolist() == [s * 64 for s in want_start]
            assert (got[:, 6:9] >= 0).all()


# ----------------------------------------------------------------- C ABI, directly

def _c_abi():
    lib = ctypes.CDLL(os.path.join(ROOT, "grouped_gemm_amd", "libgrouped_gemm_hip.so"))
    lib.gg_last_error.restype = ctypes.c_char_p
    lib.gg_gmm_bf16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.gg_gmm.argtypes = [ctypes.c_void_p]
    return lib


class GmmArgs(ctypes.Structure):
    """gg_gmm_args of include/grouped_gemm_hip.h."""
    _fields_ = [("struct_bytes", ctypes.c_uint32), ("dtype", ctypes.c_int32),
                ("a", ctypes.c_void_p), ("b", ctypes.c_void_p), ("c", ctypes.c_void_p),
                ("batch_sizes", ctypes.c_void_p), ("batch_sizes_on_device", ctypes.c_int32),
                ("trans_a", ctypes.c_int32), ("trans_b", ctypes.c_int32), ("accumulate_f32", ctypes.c_int32),
                ("num_groups", ctypes.c_int64), ("tokens", ctypes.c_int64),
                ("hidden_in", ctypes.c_int64), ("hidden_out", ctypes.c_int64),
                ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_uint64),
                ("flags", ctypes.c_int32), ("reserved0", ctypes.c_int32), ("stream", ctypes.c_void_p),
                ("a_row_index", ctypes.c_void_p), ("b_row_index", ctypes.c_void_p), ("c_row_index", ctypes.c_void_p),
                ("a_num_rows", ctypes.c_int64), ("c_num_rows", ctypes.c_int64),
                ("epilogue", ctypes.c_int32), ("b_num_rows", ctypes.c_int32), ("size_status", ctypes.c_void_p)]


def _gmm_args(lib, a, b, c, sizes, on_device, tokens, hin, hout, trans_a, trans_b, flags=0, workspace=None,
              dtype=0, stream=None):
    g = GmmArgs()
    g.struct_bytes = ctypes.sizeof(GmmArgs)
    g.dtype = dtype
    g.a, g.b, g.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
    g.batch_sizes, g.batch_sizes_on_device = sizes.data_ptr(), int(on_device)
    g.trans_a, g.trans_b = int(trans_a), int(trans_b)
    g.num_groups, g.tokens, g.hidden_in, g.hidden_out = sizes.numel(), tokens, hin, hout
    if workspace is not None:
        g.workspace, g.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    g.flags = flags
    g.stream = stream if stream is not None else torch.cuda.current_stream().cuda_stream
    return g


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
@pytest.mark.parametrize("on_device", [False, True])
def test_c_abi_against_c_oracle(oracle, layout, on_device):
    trans_a, trans_b = layout
    _announce("c abi", layout, on_device)
    lib = _c_abi()
    g = torch.Generator().manual_seed(7)
    sizes = torch.tensor([5, 0, 300, 64, 1, 0, 130], dtype=torch.int64)
    t, hin, hout = int(sizes.sum()), 72, 264
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
    if trans_a:
        b = torch.randn(t, hout, generator=g).to(torch.bfloat16)
        c = torch.full((len(sizes), hin, hout), 7.0, dtype=torch.bfloat16)
    else:
        b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
        c = torch.full((t, hout), 7.0, dtype=torch.bfloat16)
    da, db, dc = a.cuda(), b.cuda(), c.cuda()
    dsz = sizes.cuda() if on_device else sizes
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        rc = lib.gg_gmm_bf16(da.data_ptr(), db.data_ptr(), dc.data_ptr(), dsz.data_ptr(), int(on_device),
                             len(sizes), t, hin, hout, int(trans_a), int(trans_b), stream.cuda_stream)
    assert rc == 0, lib.gg_last_error()
    stream.synchronize()
    want32, _ = oracle.gmm_c(a, b, sizes, trans_a=trans_a, trans_b=trans_b)
    check(dc, want32, "c abi")
    if trans_a:
        assert (dc[1] == 0).all() and (dc[5] == 0).all()


def test_c_abi_rejects_bad_host_sizes():
    lib = _c_abi()
    a = torch.zeros(16, 8, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(2, 8, 8, dtype=torch.bfloat16, device="cuda")
    c = torch.zeros(16, 8, dtype=torch.bfloat16, device="cuda")
    for sizes in ([10, 10], [-1, 4]):
        s = torch.tensor(sizes, dtype=torch.int64)
        rc = lib.gg_gmm_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), s.data_ptr(), 0, 2, 16, 8, 8, 0, 0, None)
        assert rc == -1, sizes
    big = (1 << 63) - 1                                        # would wrap a running sum
    s = torch.tensor([10, big], dtype=torch.int64)
    rc = lib.gg_gmm_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), s.data_ptr(), 0, 2, 16, 8, 8, 0, 0, None)
    assert rc == -1 and b"sum past" in lib.gg_last_error()


def test_c_abi_workspace_sizes(oracle):
    # the general entry point with workspaces of several sizes: every one gives the oracle's
    # result; a workspace too small for a single partial tile is rejected
    lib = _c_abi()
    g = torch.Generator().manual_seed(9)
    sizes = torch.tensor([300, 40, 0, 129], dtype=torch.int64)
    t, hin, hout = int(sizes.sum()), 1024, 264
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16).cuda()
    b = torch.randn(4, hin, hout, generator=g).to(torch.bfloat16).cuda()
    want = oracle.gmm_loop(a.cpu(), b.cpu(), sizes)
    slot = 256 * 256 * 4
    for nbytes in (4096 + slot, 4096 + 7 * slot + 100, 4096 + 64 * slot, 4096 + 256 * slot):
        _announce("workspace bytes", nbytes)
        ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        c = torch.full((t, hout), 7.0, dtype=torch.bfloat16, device="cuda")
        args = _gmm_args(lib, a, b, c, sizes.cuda(), True, t, hin, hout, 0, 0, workspace=ws)
        assert lib.gg_gmm(ctypes.byref(args)) == 0, lib.gg_last_error()
        torch.cuda.synchronize()
        check(c, want, f"workspace of {nbytes} bytes")
        assert not ws[:4096].any(), "the arrival counters must be zero again after the call"
    ws = torch.zeros(4096 + slot - 256, dtype=torch.uint8, device="cuda")
    args = _gmm_args(lib, a, b, c, sizes.cuda(), True, t, hin, hout, 0, 0, workspace=ws)
    assert lib.gg_gmm(ctypes.byref(args)) == -2 and b"workspace" in lib.gg_last_error()


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_groups_are_isolated_from_each_other(ops, layout):
    # NaNs in the rows of one group (and in its weights) must show up in that group's output
    # only: tiles are cut at group ends by the buffer descriptors, never by arithmetic on
    # neighbouring rows.  Sizes straddle every tile and block boundary.
    trans_a, trans_b = layout
    sizes = [70, 1, 0, 300, 129, 255]
    poisoned = 3
    bs = torch.tensor(sizes, dtype=torch.int64)
    starts = [0] + list(torch.cumsum(bs, 0))
    t, hin, hout = int(bs.sum()), 136, 264
    g = torch.Generator().manual_seed(3)
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
    a[starts[poisoned]:starts[poisoned + 1]] = float("nan")
    if trans_a:
        b = torch.randn(t, hout, generator=g).to(torch.bfloat16)
    else:
        b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
        b[poisoned] = float("nan")
    _announce("isolation", layout)
    out = ops.backend.gmm(a.cuda(), b.cuda(), bs.cuda(), trans_a=trans_a, trans_b=trans_b).float().cpu()
    for e in range(len(sizes)):
        block = out[e] if trans_a else out[starts[e]:starts[e + 1]]
        if e == poisoned:
            assert torch.isnan(block).all()
        else:
            assert not torch.isnan(block).any(), e


def test_repeated_calls_are_bitwise_identical(ops):
    # no atomics, no split accumulation: the same call gives the same bits every time
    w_sizes = torch.tensor([300, 0, 17, 1000, 256, 129], dtype=torch.int64)
    t = int(w_sizes.sum())
    g = torch.Generator().manual_seed(11)
    a = torch.randn(t, 520, generator=g).to(torch.bfloat16).cuda()
    b = torch.randn(6, 520, 776, generator=g).to(torch.bfloat16).cuda()
    grad = torch.randn(t, 776, generator=g).to(torch.bfloat16).cuda()
    sd = w_sizes.cuda()
    first = [ops.backend.gmm(a, b, sd), ops.backend.gmm(grad, b, sd, trans_b=True),
             ops.backend.gmm(a, grad, sd, trans_a=True)]
    for _ in range(5):
        again = [ops.backend.gmm(a, b, sd), ops.backend.gmm(grad, b, sd, trans_b=True),
                 ops.backend.gmm(a, grad, sd, trans_a=True)]
        for x, y in zip(first, again):
            assert torch.equal(x, y)


def test_hip_graph_replay_with_new_device_sizes(ops, oracle):
    # The call allocates nothing and never reads batch_sizes on the host when they live on the
    # device, so it can be captured in a HIP graph once and replayed with other group sizes:
    # the kernel re-derives its schedule from the size buffer at every replay.  Replays are
    # interleaved with eager work and checked one by one.
    hin, hout, t = 256, 392, 1500
    g = torch.Generator().manual_seed(23)
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16).cuda()
    b = torch.randn(5, hin, hout, generator=g).to(torch.bfloat16).cuda()
    grad = torch.randn(t, hout, generator=g).to(torch.bfloat16).cuda()
    sizes = torch.tensor([300, 300, 300, 300, 300], dtype=torch.int64).cuda()
    out = torch.empty(t, hout, dtype=torch.bfloat16, device="cuda")
    wgrad = torch.empty(5, hin, hout, dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):      # warm-up outside the capture (first-call attribute setting)
        ops.backend.gmm(a, b, sizes, c=out)
        ops.backend.gmm(a, grad, sizes, trans_a=True, c=wgrad)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.backend.gmm(a, b, sizes, c=out)
        ops.backend.gmm(a, grad, sizes, trans_a=True, c=wgrad)
    for new_sizes in ([300] * 5, [1500, 0, 0, 0, 0], [1, 2, 3, 4, 1490], [0, 700, 0, 800, 0], [299, 301, 17, 600, 283]):
        _announce("graph replay", new_sizes)
        sizes.copy_(torch.tensor(new_sizes, dtype=torch.int64))
        out.fill_(7.0)
        wgrad.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        eager = ops.backend.gmm(a, b, sizes)
        eager_w = ops.backend.gmm(a, grad, sizes, trans_a=True)
        assert torch.equal(out, eager), new_sizes
        assert torch.equal(wgrad, eager_w), new_sizes
        check(out, oracle.gmm_loop(a.cpu(), b.cpu(), torch.tensor(new_sizes)), f"replay {new_sizes}")


def test_hip_graph_replay_of_a_weight_gradient_with_deep_groups(ops, oracle):
    # The weight gradient decides inside the kernel, from the sizes it finds, whether the tiles of
    # a much deeper group are cut along the depth and handed out first (through the binding's
    # per-stream workspace): one captured launch replays as a balanced launch, as one with the
    # deep group in the first, the last or a middle place, and as a balanced one again, each equal
    # to the eager call bit for bit and right against the oracle.
    hin, hout, t = 264, 520, 16000
    g = torch.Generator().manual_seed(29)
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16).cuda()
    grad = torch.randn(t, hout, generator=g).to(torch.bfloat16).cuda()
    sizes = torch.tensor([3200] * 5, dtype=torch.int64).cuda()
    wgrad = torch.empty(5, hin, hout, dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):      # warm-up outside the capture (workspace, first-call attribute setting)
        ops.backend.gmm(a, grad, sizes, trans_a=True, c=wgrad)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.backend.gmm(a, grad, sizes, trans_a=True, c=wgrad)
    for new_sizes in ([3200] * 5, [15000, 200, 300, 0, 500], [100, 0, 200, 300, 15400], [0, 500, 14500, 0, 1000],
                      [7000, 8000, 0, 0, 1000], [3200] * 5):
        _announce("graph replay, weight gradient", new_sizes)
        sizes.copy_(torch.tensor(new_sizes, dtype=torch.int64))
        wgrad.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        eager = ops.backend.gmm(a, grad, sizes, trans_a=True)
        assert torch.equal(wgrad, eager), new_sizes
        check(wgrad, oracle.gmm_loop(a.cpu(), grad.cpu(), torch.tensor(new_sizes), trans_a=True), f"replay {new_sizes}")


_COLD_CAPTURE = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
from grouped_gemm import backend
g = torch.Generator().manual_seed(23)
a = torch.randn(1500, 256, generator=g).to(torch.bfloat16).cuda()
b = torch.randn(5, 256, 392, generator=g).to(torch.bfloat16).cuda()
grad = torch.randn(1500, 392, generator=g).to(torch.bfloat16).cuda()
sizes = torch.tensor([300] * 5, dtype=torch.int64).cuda()
out = torch.empty(1500, 392, dtype=torch.bfloat16, device="cuda")
wgrad = torch.empty(5, 256, 392, dtype=torch.bfloat16, device="cuda")
torch.cuda.synchronize()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph):                 # the library's very first calls in this process
    backend.gmm(a, b, sizes, c=out)
    backend.gmm(a, grad, sizes, trans_a=True, c=wgrad)
for new_sizes in ([300] * 5, [1, 2, 3, 4, 1490], [0, 700, 0, 800, 0]):
    sizes.copy_(torch.tensor(new_sizes, dtype=torch.int64))
    out.fill_(7.0); wgrad.fill_(7.0)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, backend.gmm(a, b, sizes)), new_sizes
    assert torch.equal(wgrad, backend.gmm(a, grad, sizes, trans_a=True)), new_sizes
print("cold capture ok")
"""


def test_hip_graph_capture_of_the_first_call_in_a_process():
    # No warm-up: the library's first call on the device (set-up of every kernel variant, the
    # binding's workspace) happens inside the capture; replays with other sizes equal eager calls.
    import subprocess
    import sys
    res = subprocess.run([sys.executable, "-c", _COLD_CAPTURE, ROOT], capture_output=True, text=True, timeout=280)
    assert res.returncode == 0 and "cold capture ok" in res.stdout, res.stdout[-2000:] + res.stderr[-4000:]


@pytest.mark.parametrize("trans_b", [False, True])
def test_traceable_operator_under_torch_compile(ops, trans_b):
    # one graph, no breaks (fullgraph), forward and both gradients bit-equal to the autograd
    # Function of the reference's surface
    sizes = torch.tensor([37, 0, 300, 163], dtype=torch.int64).cuda()
    g = torch.Generator().manual_seed(29)
    a0 = torch.randn(500, 136, generator=g).to(torch.bfloat16).cuda()
    b0 = torch.randn(4, *((200, 136) if trans_b else (136, 200)), generator=g).to(torch.bfloat16).cuda()
    grad = torch.randn(500, 200, generator=g).to(torch.bfloat16).cuda()

    def run(fn):
        a, b = a0.clone().requires_grad_(), b0.clone().requires_grad_()
        out = fn(a, b)
        out.backward(grad)
        return out.detach(), a.grad, b.grad

    eager = run(lambda a, b: ops.gmm(a, b, sizes, trans_b))
    compiled_fn = torch.compile(lambda a, b: ops.gmm_traceable(a, b, sizes, trans_b) * 1.0,
                                backend="aot_eager", fullgraph=True)
    _announce("torch.compile", trans_b)
    compiled = run(compiled_fn)
    for x, y in zip(eager, compiled):
        assert torch.equal(x, y)


# ------------------------------------------------------------------- float16 operands

@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_float16_random_shapes(ops, oracle, layout):
    # same kernels with the fp16 matrix instruction and an fp16 rounding on store; the oracle is
    # the per-expert loop on fp32-upcast slices (the reference takes bf16 only,
    # csrc/grouped_gemm.cu:492, 505-506).  fp16 keeps 3 more mantissa bits than bf16, so the bf16
    # tolerance holds with room to spare; values are kept inside the fp16 range.
    trans_a, trans_b = layout
    for idx, (sizes, hin, hout) in enumerate(_random_cases(12, seed=41 + int(trans_a) + 2 * int(trans_b))):
        _announce("fp16", layout, sizes, hin, hout)
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(torch.float16)
        if trans_a:
            b = torch.randn(t, hout, generator=g).to(torch.float16)
        else:
            b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.float16)
        dev_bs = bs.cuda() if idx % 2 else bs
        out = ops.backend.gmm(a.cuda(), b.cuda(), dev_bs, trans_a=trans_a, trans_b=trans_b)
        assert out.dtype == torch.float16
        want = oracle.gmm_loop(a, b, bs, trans_a=trans_a, trans_b=trans_b)
        check(out, want, f"case {idx}: sizes={sizes} hin={hin} hout={hout}")
        # tighter: one fp16 rounding of the fp32-accumulated value
        assert float((out.float().cpu() - want).abs().max()) <= 2 ** -10 * float(want.abs().max()) + 1e-6


@pytest.mark.parametrize("trans_b", [False, True])
def test_float16_autograd_and_mixed_dtypes(ops, oracle, trans_b):
    g = torch.Generator().manual_seed(43)
    sizes = torch.tensor([300, 0, 17, 195])
    a = torch.randn(512, 256, generator=g).to(torch.float16)
    b = torch.randn(4, *((384, 256) if trans_b else (256, 384)), generator=g).to(torch.float16)
    grad = torch.randn(512, 384, generator=g).to(torch.float16)
    da, db = a.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    out = ops.gmm(da, db, sizes.cuda(), trans_b)
    out.backward(grad.cuda())
    want, want_ag, want_bg = oracle.gmm_autograd_loop(a, b, sizes, trans_b, grad)
    check(out.detach(), want, "forward")
    check(da.grad, want_ag, "agrad")
    check(db.grad, want_bg, "bgrad")
    assert (db.grad[1] == 0).all()
    with pytest.raises(RuntimeError, match="element type"):
        ops.backend.gmm(a.cuda(), b.cuda().to(torch.bfloat16), sizes)
    # fp16 operands, fp32 accumulated weight gradient
    c0 = torch.randn(4, 256, 384, generator=g)
    c = c0.clone().cuda()
    ops.backend.accumulate_weight_gradient(a.cuda(), grad.cuda(), sizes.cuda(), c)
    want_c = oracle.accumulate_weight_gradient_loop(a, grad, sizes, c0)
    assert float((c.double().cpu() - want_c).abs().max()) <= 1e-4 * float(want_c.abs().max())


# ---- any hidden size, any alignment (the general kernels, and gmm's zero-padded copies instead)

@pytest.fixture(params=[False, True], ids=["general-kernels", "padded-copies"])
def odd_size_path(request, ops):
    """Both ways operands the streaming kernels do not take are served: the extension called
    directly runs them copy-free on the general kernels, backend.gmm through zero-padded copies
    on the streaming ones.  Returns gmm(a, b, batch_sizes, trans_a, trans_b, c=None)."""
    if request.param:
        return lambda a, b, bs, trans_a=False, trans_b=False, c=None: ops.backend.gmm(
            a, b, bs, trans_a=trans_a, trans_b=trans_b, c=c)

    def direct(a, b, bs, trans_a=False, trans_b=False, c=None):
        if c is None:
            c = ops.backend._allocate_output(a, b, bs, trans_a, trans_b)
        ops.backend.backend.gmm(a, b, c, bs, trans_a, trans_b)
        return c
    return direct


def _odd_cases(n, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    pool = [1, 2, 3, 5, 7, 12, 20, 33, 100, 130, 250, 1001]
    cases = []
    for _ in range(n):
        e = r(1, 6)
        sizes = [r(0, 3) * 64 + r(-3, 70) for _ in range(e)]
        sizes = [max(0, x) for x in sizes]
        cases.append((sizes, pool[r(0, len(pool) - 1)], pool[r(0, len(pool) - 1)]))
    cases += [([130, 0, 7], 12, 100), ([300], 1001, 1001), ([5, 129], 100, 12), ([64, 64], 1, 1)]
    return cases


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_hidden_sizes_that_are_not_multiples_of_8(ops, oracle, layout, dtype, odd_size_path):
    # the reference's default build takes any hidden size (csrc/grouped_gemm.cu:373-394); sizes
    # that are multiples of 4, of 2, and odd ones, each through its own vector width
    trans_a, trans_b = layout
    for idx, (sizes, hin, hout) in enumerate(_odd_cases(10, seed=51 + int(trans_a) + 2 * int(trans_b))):
        _announce("any size", layout, dtype, sizes, hin, hout)
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype)
        if trans_a:
            b = torch.randn(t, hout, generator=g).to(dtype)
        else:
            b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(dtype)
        dev_bs = bs.cuda() if idx % 2 else bs
        out = odd_size_path(a.cuda(), b.cuda(), dev_bs, trans_a=trans_a, trans_b=trans_b)
        want = oracle.gmm_loop(a, b, bs, trans_a=trans_a, trans_b=trans_b)
        check(out, want, f"case {idx}: sizes={sizes} hin={hin} hout={hout}")


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_operands_off_the_16_byte_boundary(ops, oracle, layout, odd_size_path):
    # views that start one, two or four elements into a buffer: same results as the aligned call
    trans_a, trans_b = layout
    g = torch.Generator().manual_seed(61)
    sizes = torch.tensor([70, 0, 300, 41])
    t, hin, hout = int(sizes.sum()), 136, 264
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
    b = torch.randn(t, hout, generator=g).to(torch.bfloat16) if trans_a else \
        torch.randn(4, *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
    want = oracle.gmm_loop(a, b, sizes, trans_a=trans_a, trans_b=trans_b)

    def shifted(x, by):
        buf = torch.empty(x.numel() + by, dtype=x.dtype, device="cuda")
        view = buf[by:].view(x.shape)
        view.copy_(x)
        assert view.data_ptr() % 16 == (2 * by) % 16
        return view

    for by_a, by_b, by_c in [(1, 0, 0), (0, 2, 0), (0, 0, 4), (1, 3, 5)]:
        _announce("off boundary", layout, by_a, by_b, by_c)
        c = shifted(torch.zeros(want.shape, dtype=torch.bfloat16), by_c)
        odd_size_path(shifted(a, by_a), shifted(b, by_b), sizes.cuda(), trans_a=trans_a, trans_b=trans_b, c=c)
        check(c, want, f"shifted by {by_a}, {by_b}, {by_c} elements")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_even_sizes_on_4_byte_boundaries_stream(ops, oracle, layout, dtype):
    # Two-byte operands on 4-byte boundaries stream as they are (no copies) when both hidden sizes
    # are even; here no 16-byte chunk mixes elements along the depth (hidden_in a multiple of 8, or
    # trans_a; the other depths have the test below).  Rows of c start on 4-byte boundaries and the last 16-byte chunk of
    # a row holds 2, 4 or 6 columns; chunks of b (and of a with trans_a) run past their rows' ends.
    # Exact placement is checked with sentinels around c; a, b and c sit 4 bytes off the 16-byte
    # boundary; through the extension, through backend.gmm and with fused row indices.
    trans_a, trans_b = layout
    cases = [([300, 0, 17, 195], 264, 250), ([1, 255, 257, 64], 136, 262), ([1000], 72, 518), ([5] * 40, 64, 6),
             ([33, 90], 6400, 1030), ([40] * 30, 128, 772)]
    if trans_a:
        cases = [([300, 0, 17, 195], 262, 250), ([1, 255, 257, 64], 130, 266), ([1000], 70, 518), ([5] * 40, 6, 10),
                 ([7000, 0, 6500], 258, 522), ([40] * 30, 772, 126)]

    def off_boundary(x, fill=None):
        # a view 4 bytes past a 16-byte boundary, with 2 sentinel elements in front and behind
        buf = torch.full((x.numel() + 4,), 7.0 if fill is None else fill, dtype=x.dtype, device="cuda")
        view = buf[2:2 + x.numel()].view(x.shape)
        view.copy_(x)
        assert view.data_ptr() % 16 == 4
        return buf, view

    for idx, (sizes, hin, hout) in enumerate(cases):
        _announce("even sizes, 4-byte boundaries", layout, dtype, sizes, hin, hout)
        g = torch.Generator().manual_seed(70 + idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype)
        if trans_a:
            b = torch.randn(t, hout, generator=g).to(dtype)
        else:
            b = (torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g) * hin ** -0.5).to(dtype)
        want = oracle.gmm_loop(a, b, bs, trans_a=trans_a, trans_b=trans_b)
        _, da = off_boundary(a)
        _, db = off_boundary(b)
        cbuf, c = off_boundary(torch.zeros(want.shape, dtype=dtype))
        cbuf.fill_(7.0)
        ops.backend.backend.gmm(da, db, c, bs.cuda() if idx % 2 else bs, trans_a, trans_b)
        scale = max(1.0, float(want.double().pow(2).mean().sqrt()))
        check(c.float() / scale, want / scale, f"case {idx}")
        assert bool((cbuf[:2] == 7.0).all()) and bool((cbuf[-2:] == 7.0).all())
        out = ops.backend.gmm(da, db, bs.cuda(), trans_a=trans_a, trans_b=trans_b)
        assert torch.equal(out, c)
        if not trans_a:
            perm = torch.randperm(t, generator=g).to(torch.int32).cuda()
            c2 = torch.zeros(t, hout, dtype=dtype, device="cuda")
            ops.backend.gmm_indexed(da, db, bs.cuda(), trans_b=trans_b, c=c2, a_rows=perm, c_rows=perm)
            want2 = torch.zeros_like(want)
            want2[perm.long().cpu()] = oracle.gmm_loop(a[perm.long().cpu()], b, bs, trans_b=trans_b)
            check(c2, want2, f"case {idx}, gathered and scattered")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("trans_b", [False, True])
def test_even_depths_that_are_no_multiple_of_8_stream(ops, oracle, trans_b, dtype):
    # hidden_in even but no multiple of 8, in the layouts whose rows run along the depth: the
    # 16-byte chunk with a row's last 2, 4 or 6 depth values also holds the first values of the next
    # row in memory, which the kernel clears in LDS.  Those first values are poisoned here: one row
    # of a (and, stored transposed, one row of b per group) starts with NaNs, so its own outputs are
    # NaN and every other output must be finite and right.  Depths below one slice, ragged in the
    # first, a middle and the last chunk of a slice, and deep enough for depth pieces otherwise.
    cases = [([300, 0, 17, 195], 262, 250), ([1, 255, 257, 64], 130, 264), ([1000], 70, 518), ([5] * 40, 6, 16),
             ([33, 90], 6404, 1032), ([40] * 30, 66, 772), ([70, 300], 1022, 130), ([129], 58, 72)]
    for idx, (sizes, hin, hout) in enumerate(cases):
        _announce("even depth, no multiple of 8", trans_b, dtype, sizes, hin, hout)
        g = torch.Generator().manual_seed(90 + idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype)
        b = (torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g) * hin ** -0.5).to(dtype)
        bad_row = t // 2
        a[bad_row, :min(6, hin)] = float("nan")
        bad_col = hout // 3
        if trans_b:
            b[:, bad_col, :min(6, hin)] = float("nan")
        want = oracle.gmm_loop(a, b, bs, trans_b=trans_b)
        finite = torch.ones_like(want, dtype=torch.bool)
        finite[bad_row] = False
        if trans_b:
            finite[:, bad_col] = False
        assert bool(torch.isnan(want[~finite]).all()) and bool(torch.isfinite(want[finite]).all())
        da, db = a.cuda(), b.cuda()
        c = torch.full((t + 1, hout), 7.0, dtype=dtype, device="cuda")
        ops.backend.backend.gmm(da, db, c[:t], bs.cuda() if idx % 2 else bs, False, trans_b)
        got = c[:t].cpu()
        assert bool(torch.isnan(got[~finite]).all()), f"case {idx}: poisoned outputs"
        assert bool(torch.isfinite(got[finite]).all()), f"case {idx}: a NaN of a neighbouring row reached a sum"
        clean = lambda x: torch.where(finite, x.float(), torch.zeros((), dtype=torch.float32))
        check(clean(got), clean(want), f"case {idx}")
        assert bool((c[t] == 7.0).all())
        out = ops.backend.gmm(da, db, bs.cuda(), trans_b=trans_b)
        assert torch.equal(clean(out.cpu()), clean(got))
        # rows through indices, and the workspace the binding would fetch: none for these sizes
        perm = torch.randperm(t, generator=g).to(torch.int32).cuda()
        c2 = torch.zeros(t, hout, dtype=dtype, device="cuda")
        ops.backend.gmm_indexed(da, db, bs.cuda(), trans_b=trans_b, c=c2, a_rows=perm, c_rows=perm)
        rows = perm.long().cpu()
        want2 = torch.zeros_like(want)
        want2[rows] = oracle.gmm_loop(a[rows], b, bs, trans_b=trans_b)
        finite2 = torch.isfinite(want2)
        got2 = c2.cpu()
        assert bool((torch.isfinite(got2) == finite2).all()), f"case {idx}, gathered and scattered: NaN placement"
        zero = torch.zeros((), dtype=torch.float32)
        check(torch.where(finite2, got2.float(), zero), torch.where(finite2, want2.float(), zero),
              f"case {idx}, gathered and scattered")


def test_padded_copies_leave_tail_rows_alone(ops, oracle):
    # sum(batch_sizes) < rows of a: the rows of c past the sum keep their contents on this path too
    g = torch.Generator().manual_seed(64)
    sizes = torch.tensor([40, 0, 25])
    a = torch.randn(100, 33, generator=g).to(torch.bfloat16)
    b = torch.randn(3, 33, 50, generator=g).to(torch.bfloat16)
    c = torch.full((100, 50), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.backend.gmm(a.cuda(), b.cuda(), sizes.cuda(), c=c)
    check(c[:65], oracle.gmm_loop(a, b, sizes)[:65], "rows in use")
    assert bool((c[65:] == 7.0).all())
    # malformed calls raise what the plain path raises
    with pytest.raises(RuntimeError):
        ops.backend.gmm(a.cuda(), b.cuda()[:, :32], sizes.cuda())
    with pytest.raises(RuntimeError):
        ops.backend.gmm(a.cuda().t().contiguous().t(), b.cuda(), sizes.cuda())   # a not contiguous


def test_accumulated_weight_gradient_any_size(ops, oracle):
    g = torch.Generator().manual_seed(63)
    sizes = torch.tensor([300, 0, 17, 129])
    t = int(sizes.sum())
    for hin, hout in [(100, 12), (33, 1001), (7, 7)]:
        a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
        b = torch.randn(t, hout, generator=g).to(torch.bfloat16)
        c0 = torch.randn(4, hin, hout, generator=g)
        c = c0.clone().cuda()
        ops.backend.accumulate_weight_gradient(a.cuda(), b.cuda(), sizes.cuda(), c)
        want = oracle.accumulate_weight_gradient_loop(a, b, sizes, c0)
        assert float((c.double().cpu() - want).abs().max()) <= 1e-4 * float(want.abs().max())
        assert torch.equal(c[1].cpu(), c0[1])


# ----------------------------------------------------------------------- fp8 operands

@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_float8_operands(ops, oracle, layout, dtype, odd_size_path):
    # fp8 in a and b (OCP formats), fp32 accumulation of the exact products, one bf16 rounding on
    # store; the oracle is the per-expert loop on the fp32 decode of the same bytes
    trans_a, trans_b = layout
    cases = _random_cases(6, seed=71 + int(trans_a) + 2 * int(trans_b)) + [([130, 0, 7], 100, 12), ([300], 1001, 33)]
    for idx, (sizes, hin, hout) in enumerate(cases):
        _announce("fp8", layout, dtype, sizes, hin, hout)
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype)
        if trans_a:
            b = torch.randn(t, hout, generator=g).to(dtype)
        else:
            b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(dtype)
        out = ops.backend.gmm(a.cuda(), b.cuda(), bs.cuda() if idx % 2 else bs, trans_a=trans_a, trans_b=trans_b)
        assert out.dtype == torch.bfloat16
        want = oracle.gmm_loop(a, b, bs, trans_a=trans_a, trans_b=trans_b)
        check(out, want, f"case {idx}: sizes={sizes} hin={hin} hout={hout}")


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_float8_streaming_kernel(ops, oracle, layout, dtype):
    # hidden sizes that are multiples of 16 run on the streaming kernel with the 32x32x64 fp8 matrix
    # instruction (width-major operands through the byte-wise transposing LDS read): every count
    # of row blocks, ragged depth and width, the DeepSeek-style shape shrunk, device- and
    # host-resident sizes
    trans_a, trans_b = layout
    cases = [([1, 31, 33, 64, 97, 128, 160, 200, 255, 256, 257, 300, 0, 513], 192, 336),
             ([300, 0, 17, 1000], 528, 784), ([5] * 70, 272, 144), ([4000], 1024, 512), ([256] * 16, 448, 128),
             # few tiles and a deep product: the last round is cut along the depth (100 slices of
             # 128 in the NN and NT layouts, 102 in the weight-gradient layout)
             ([300, 200], 12800, 256), ([13000], 256, 256)]
    for idx, (sizes, hin, hout) in enumerate(cases):
        _announce("fp8 streaming", layout, dtype, sizes, hin, hout)
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype)
        if trans_a:
            b = torch.randn(t, hout, generator=g).to(dtype)
        else:
            b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(dtype)
        out = ops.backend.gmm(a.cuda(), b.cuda(), bs.cuda() if idx % 2 else bs, trans_a=trans_a, trans_b=trans_b)
        assert out.dtype == torch.bfloat16
        check(out, oracle.gmm_loop(a, b, bs, trans_a=trans_a, trans_b=trans_b), f"case {idx}")
    # exact: one-hot rows against an identity-like weight give the row's value back in its place
    sizes = [1, 31, 33, 97, 160, 255, 257, 300]
    bs = torch.tensor(sizes, dtype=torch.int64)
    t, hin, hout = int(bs.sum()), 256, 384
    idx = torch.arange(t) % 251
    rows = torch.zeros(t, hin)
    rows[torch.arange(t), idx % hin] = (idx % 7 + 1).float()
    if trans_a:
        # c[e] = rows_e^T @ marks_e with marks one-hot too: c[e][i][j] counts value * 1 over the
        # rows of group e that have their value in column i and their mark in column j
        marks = torch.zeros(t, hout)
        marks[torch.arange(t), (idx * 5) % hout] = 1.0
        got = ops.backend.gmm(rows.to(dtype).cuda(), marks.to(dtype).cuda(), bs.cuda(), trans_a=True).float().cpu()
        want = torch.zeros(len(sizes), hin, hout)
        start = 0
        for e, m in enumerate(sizes):
            want[e] = rows[start:start + m].t() @ marks[start:start + m]
            start += m
        assert float(want.max()) <= 256.0          # sums of small integers: exact in bf16
        assert torch.equal(got, want)
        return
    eye = torch.zeros(len(sizes), hout, hin)
    eye[:, :hin, :] = torch.eye(hin)
    weight = eye if trans_b else eye.transpose(1, 2).contiguous()
    got = ops.backend.gmm(rows.to(dtype).cuda(), weight.to(dtype).cuda(), bs.cuda(), trans_b=trans_b).float().cpu()
    want = torch.zeros(t, hout)
    want[:, :hin] = rows
    assert torch.equal(got, want)


@pytest.mark.parametrize("config", [2, 5])
def test_float8_full_size(ops, oracle, config):
    """fp8 e4m3 at the Mixtral and the DeepSeek-style shape, all three launches of forward +
    backward: against the fp32 loop on the decoded bytes (on the GPU) and CPU float64 spot checks."""
    from grouped_gemm_amd import workloads
    _announce("fp8 full size", config)
    w = workloads.make(config, device="cuda")
    dt = torch.float8_e4m3fn
    sizes, bs = w.batch_sizes, w.batch_sizes.cuda()
    # (scaled up so that the values use the format's normal range, as a scaled fp8 tensor would)
    a8, b8, g8 = (w.a.float() * 32).to(dt), (w.b.float() * 32).to(dt), (w.grad.float() * 32).to(dt)
    with torch.no_grad():
        out = ops.backend.gmm(a8, b8, bs, trans_b=w.trans_b)
        check(out, oracle.gmm_loop(a8, b8, sizes, trans_b=w.trans_b), "fp8 forward")
        fp64_rows_check(a8, b8, sizes, w.trans_b, out)
        del out
        ag = ops.backend.gmm(g8, b8, bs, trans_b=not w.trans_b)
        check(ag, oracle.gmm_loop(g8, b8, sizes, trans_b=not w.trans_b), "fp8 agrad")
        fp64_rows_check(g8, b8, sizes, not w.trans_b, ag, seed=1)
        del ag
        lhs, rhs = (g8, a8) if w.trans_b else (a8, g8)
        bg = ops.backend.gmm(lhs, rhs, bs, trans_a=True)
        starts = torch.cumsum(sizes, 0) - sizes
        for e in range(0, len(sizes), max(1, len(sizes) // 8)):
            s0, m = int(starts[e]), int(sizes[e])
            check(bg[e], lhs[s0:s0 + m].float().t() @ rhs[s0:s0 + m].float(), f"fp8 bgrad expert {e}")
        fp64_weight_gradient_check(lhs, rhs, sizes, bg)
        assert torch.equal(bg, ops.backend.gmm(lhs, rhs, sizes, trans_a=True))


# ------------------------------------------------------------- fused gather / scatter

def _routing(tokens, experts, top_k, seed):
    """Top-k routing of `tokens` rows: the sorted order (row_index[r] = source row of sorted row r),
    the group sizes, and the position of each (token, k) pair in the sorted order."""
    g = torch.Generator().manual_seed(seed)
    expert = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(tokens)])   # (tokens, k)
    flat = expert.flatten()
    order = torch.argsort(flat, stable=True)
    sizes = torch.bincount(flat, minlength=experts).to(torch.int64)
    return (order // top_k).to(torch.int32), sizes, order.to(torch.int32)


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("hidden", [(136, 264), (100, 12)])
def test_gather_and_scatter_against_indexed_oracle(ops, oracle, trans_b, hidden):
    # gmm_indexed(a, ..., a_rows=idx) == gmm(a[idx], ...) and c[c_rows] = gmm(...), the oracle being
    # the index applied by torch and then the pinned per-expert loop
    hin, hout = hidden
    row_index, sizes, order = _routing(400, 6, 2, seed=81)
    g = torch.Generator().manual_seed(82)
    x = torch.randn(400, hin, generator=g).to(torch.bfloat16)
    w = torch.randn(6, *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
    _announce("gather", trans_b, hidden)
    got = ops.backend.gmm_indexed(x.cuda(), w.cuda(), sizes.cuda(), trans_b=trans_b, a_rows=row_index.cuda())
    want = oracle.gmm_loop(x[row_index.long()], w, sizes, trans_b=trans_b)
    check(got, want, "gathered rows")
    # scatter: the sorted product goes back to (token, k) order; rows no index names stay as they were
    a_sorted = x[row_index.long()].contiguous()
    c = torch.full((800 + 3, hout), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.backend.gmm_indexed(a_sorted.cuda(), w.cuda(), sizes, trans_b=trans_b, c=c, c_rows=order.cuda())
    want_c = torch.full((803, hout), 7.0)
    want_c[order.long()] = want
    check(c, want_c, "scattered rows")
    assert (c[800:] == 7.0).all()
    # both at once
    c2 = torch.zeros(800, hout, dtype=torch.bfloat16, device="cuda")
    ops.backend.gmm_indexed(x.cuda(), w.cuda(), sizes.cuda(), trans_b=trans_b, c=c2, a_rows=row_index.cuda(),
                            c_rows=order.cuda())
    check(c2, want_c[:800], "gathered and scattered")


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("trans_b", [False, True])
def test_gather_and_scatter_float8(ops, oracle, trans_b, dtype):
    # fp8 operands with the permutation fused in, on the streaming kernels (hidden sizes multiples of
    # 16) and on the general ones; row counts that leave ragged tiles
    for hin, hout, tokens, experts in [(144, 272, 400, 6), (100, 24, 300, 5), (256, 512, 3000, 3)]:
        row_index, sizes, order = _routing(tokens, experts, 2, seed=85)
        g = torch.Generator().manual_seed(86)
        x = torch.randn(tokens, hin, generator=g).to(dtype)
        w = torch.randn(experts, *((hout, hin) if trans_b else (hin, hout)), generator=g).to(dtype)
        _announce("gather fp8", dtype, trans_b, hin, hout, tokens)
        want = oracle.gmm_loop(x[row_index.long()], w, sizes, trans_b=trans_b)
        got = ops.backend.gmm_indexed(x.cuda(), w.cuda(), sizes.cuda(), trans_b=trans_b, a_rows=row_index.cuda())
        assert got.dtype == torch.bfloat16
        check(got, want, "gathered rows")
        rows = 2 * tokens
        c = torch.full((rows + 3, hout), 7.0, dtype=torch.bfloat16, device="cuda")
        ops.backend.gmm_indexed(x.cuda(), w.cuda(), sizes.cuda(), trans_b=trans_b, c=c, a_rows=row_index.cuda(),
                                c_rows=order.cuda())
        want_c = torch.full((rows + 3, hout), 7.0)
        want_c[order.long()] = want
        check(c, want_c, "gathered and scattered")
        assert (c[rows:] == 7.0).all()


@pytest.mark.parametrize("hidden", [(136, 264), (33, 20)])
def test_weight_gradient_with_gathered_rows(ops, oracle, hidden):
    hin, hout = hidden
    row_index, sizes, order = _routing(300, 5, 2, seed=83)
    g = torch.Generator().manual_seed(84)
    x = torch.randn(300, hin, generator=g).to(torch.bfloat16)
    grad_sorted = torch.randn(600, hout, generator=g).to(torch.bfloat16)
    _announce("gathered weight gradient", hidden)
    got = ops.backend.gmm_indexed(x.cuda(), grad_sorted.cuda(), sizes.cuda(), trans_a=True, a_rows=row_index.cuda())
    want = oracle.gmm_loop(x[row_index.long()], grad_sorted, sizes, trans_a=True)
    check(got, want, "a rows gathered")
    # b gathered: the gradient in (token, k) order, the activations sorted
    grad_unsorted = torch.zeros_like(grad_sorted)
    grad_unsorted[order.long()] = grad_sorted
    a_sorted = x[row_index.long()].contiguous()
    got = ops.backend.gmm_indexed(a_sorted.cuda(), grad_unsorted.cuda(), sizes, trans_a=True, b_rows=order.cuda())
    check(got, want, "b rows gathered")


@pytest.mark.parametrize("trans_b", [False, True])
def test_fused_permutation_autograd(ops, oracle, trans_b):
    # a whole expert layer: gather-fused first GEMM, scatter-fused second GEMM, against the same
    # layer written with index operations and the oracle's loops, forward and all gradients
    hin, hmid = 136, 264
    row_index, sizes, order = _routing(256, 4, 2, seed=85)
    g = torch.Generator().manual_seed(86)
    x0 = torch.randn(256, hin, generator=g).to(torch.bfloat16)
    w1_0 = (torch.randn(4, *((hmid, hin) if trans_b else (hin, hmid)), generator=g) * 0.1).to(torch.bfloat16)
    w2_0 = (torch.randn(4, *((hin, hmid) if trans_b else (hmid, hin)), generator=g) * 0.1).to(torch.bfloat16)
    gout = torch.randn(512, hin, generator=g).to(torch.bfloat16)
    x, w1, w2 = (t.cuda().requires_grad_(True) for t in (x0, w1_0, w2_0))
    _announce("fused layer", trans_b)
    h = ops.gmm_gather(x, w1, sizes.cuda(), row_index.cuda(), trans_b)
    y = ops.gmm_scatter(h, w2, sizes.cuda(), order.cuda(), trans_b)       # (token, k) order
    y.backward(gout.cuda())
    # Reference: the same layer from index operations and the oracle's loop, stage by stage, with a
    # bf16 rounding wherever the fused path stores a bf16 tensor (h, its gradient, the sorted
    # input gradient), so that only fp32 summation order separates the two.
    bf = lambda t: t.to(torch.bfloat16)
    idx, ordr = row_index.long(), order.long()
    h_ref = oracle.gmm_loop(x0[idx], w1_0, sizes, trans_b=trans_b)
    y_sorted = oracle.gmm_loop(bf(h_ref), w2_0, sizes, trans_b=trans_b)
    y_ref = torch.zeros(512, hin).index_put((ordr,), y_sorted)
    dy_sorted = gout[ordr]
    lhs, rhs = (dy_sorted, bf(h_ref)) if trans_b else (bf(h_ref), dy_sorted)
    w2g_ref = oracle.gmm_loop(lhs, rhs, sizes, trans_a=True)
    dh = bf(oracle.gmm_loop(dy_sorted, w2_0, sizes, trans_b=not trans_b))
    lhs, rhs = (dh, x0[idx]) if trans_b else (x0[idx], dh)
    w1g_ref = oracle.gmm_loop(lhs, rhs, sizes, trans_a=True)
    dx_sorted = bf(oracle.gmm_loop(dh, w1_0, sizes, trans_b=not trans_b))
    xg_ref = torch.zeros(256, hin).index_add_(0, idx, dx_sorted.float())

    # outputs well above unit scale are compared in units of their root-mean-square
    def check_scaled(got, want, what):
        scale = max(1.0, float(want.double().pow(2).mean().sqrt()))
        check(got.float().cpu() / scale, want / scale, what)

    check_scaled(h.detach(), h_ref, "first GEMM")
    check_scaled(y.detach(), y_ref, "second GEMM")
    check_scaled(w2.grad, w2g_ref, "w2 gradient")
    check_scaled(w1.grad, w1g_ref, "w1 gradient")
    check_scaled(x.grad, xg_ref, "x gradient")


# ------------------------------------------------------------------ SwiGLU epilogue

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("trans_b", [False, True])
def test_swiglu_epilogue(ops, oracle, trans_b, dtype):
    # silu(a @ gate) * (a @ up) in the epilogue, b = [gate | up]; widths that fill several tiles,
    # a ragged last tile, and sizes that go to the general kernels (12, 100)
    for idx, (sizes, hin, hout) in enumerate([([300, 0, 17, 195], 256, 384), ([1, 255, 257, 64], 136, 200),
                                              ([1000], 520, 776), ([5] * 40, 264, 72), ([130, 7], 100, 12)]):
        _announce("swiglu", trans_b, dtype, sizes, hin, hout)
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype)
        b = (torch.randn(len(sizes), *((2 * hout, hin) if trans_b else (hin, 2 * hout)), generator=g) * hin ** -0.5).to(dtype)
        out = ops.backend.gmm_swiglu(a.cuda(), b.cuda(), bs.cuda() if idx % 2 else bs, trans_b=trans_b)
        assert out.shape == (t, hout) and out.dtype == dtype
        check(out, oracle.swiglu_loop(a, b, bs, trans_b=trans_b), f"case {idx}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("trans_b", [False, True])
def test_swiglu_epilogue_deep_unscaled_against_float64(ops, oracle, trans_b, dtype):
    # Deep products of unscaled operands (depth 8192 and 9600: pre-activations of size ~90, outputs
    # up to ~10^5): against a float64 truth (per-expert loop in float64 on the GPU, with CPU float64
    # rows beside it), under the rule that adds what an fp32 summation error of one pre-activation
    # becomes once the other multiplies it (oracle.swiglu_tolerance).  Where gate is near 0 and
    # |up| is a few hundred, no fp32-accumulating implementation meets atol + rtol |want|: the
    # oracle's own fp32 loop is held to the same rule here and needs the added term as well.
    # float16 overflows beyond 65504; both sides are clamped there.
    for idx, (sizes, hin, hout) in enumerate([([700, 800, 0, 1500], 8192, 640), ([300, 5, 2100, 0, 64, 257], 9600, 560)]):
        _announce("swiglu deep", trans_b, dtype, sizes, hin, hout)
        g = torch.Generator().manual_seed(40 + idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype).cuda()
        b = torch.randn(len(sizes), *((2 * hout, hin) if trans_b else (hin, 2 * hout)), generator=g).to(dtype).cuda()
        out = ops.backend.gmm_swiglu(a, b, bs.cuda() if idx % 2 else bs, trans_b=trans_b)
        assert out.shape == (t, hout) and out.dtype == dtype
        want, gate, up = oracle.swiglu_parts(a, b, bs, trans_b=trans_b)
        # the float64 truth itself, on the CPU, for sampled rows
        starts = torch.cumsum(bs, 0) - bs
        for r in torch.randint(0, t, (6,), generator=g).tolist():
            e = int((starts <= r).sum()) - 1
            w = b[e].double().cpu()
            gu = a[r].double().cpu() @ (w.t() if trans_b else w)
            assert float((gu[:hout] - gate[r].cpu()).abs().max()) < 1e-9 * hin
            assert float((gu[hout:] - up[r].cpu()).abs().max()) < 1e-9 * hin
        limit = 65504.0 if dtype == torch.float16 else 3.0e38
        want_c = want.clamp(-limit, limit)
        tol = oracle.swiglu_tolerance(want_c, gate, up, hin)
        plain = oracle.atol_for(want_c.float()) + RTOL * want_c.abs()
        err = (out.double().clamp(-limit, limit) - want_c).abs()
        assert bool((err <= tol).all()), f"case {idx}: outside the tolerance by {float((err - tol).max())}"
        # the added term matters for a handful of ill-conditioned elements only, and the oracle's
        # fp32 loop is no better on them
        assert int((err > plain).sum()) <= max(8, err.numel() // 100000), int((err > plain).sum())
        loop = oracle.swiglu_loop(a, b, bs, trans_b=trans_b).double().clamp(-limit, limit)
        assert bool(((loop - want_c).abs() <= tol).all()), "the fp32 loop leaves the same tolerance"


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("trans_b", [False, True])
def test_swiglu_epilogue_float8(ops, oracle, trans_b, dtype):
    # fp8 operands: b stored transposed runs on the streaming kernel (depth a multiple of 16), the
    # other layout and other sizes on the general ones; the output is bfloat16
    for idx, (sizes, hin, hout) in enumerate([([300, 0, 17, 195], 256, 384), ([1, 255, 257, 64], 144, 200),
                                              ([1000], 528, 776), ([130, 7], 100, 12)]):
        _announce("swiglu fp8", trans_b, dtype, sizes, hin, hout)
        g = torch.Generator().manual_seed(idx)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype)
        b = (torch.randn(len(sizes), *((2 * hout, hin) if trans_b else (hin, 2 * hout)), generator=g) * hin ** -0.5 * 4).to(dtype)
        out = ops.backend.gmm_swiglu(a.cuda(), b.cuda(), bs.cuda() if idx % 2 else bs, trans_b=trans_b)
        assert out.shape == (t, hout) and out.dtype == torch.bfloat16
        check(out, oracle.swiglu_loop(a, b, bs, trans_b=trans_b), f"case {idx}")


@pytest.mark.parametrize("trans_b", [False, True])
def test_swiglu_with_gathered_and_scattered_rows(ops, oracle, trans_b):
    hin, hout = 136, 264
    row_index, sizes, order = _routing(300, 5, 2, seed=87)
    g = torch.Generator().manual_seed(88)
    x = torch.randn(300, hin, generator=g).to(torch.bfloat16)
    w = (torch.randn(5, *((2 * hout, hin) if trans_b else (hin, 2 * hout)), generator=g) * hin ** -0.5).to(torch.bfloat16)
    want = oracle.swiglu_loop(x[row_index.long()], w, sizes, trans_b=trans_b)
    _announce("swiglu gathered", trans_b)
    got = ops.backend.gmm_swiglu(x.cuda(), w.cuda(), sizes.cuda(), trans_b=trans_b, a_rows=row_index.cuda())
    check(got, want, "gathered")
    c = torch.zeros(600, hout, dtype=torch.bfloat16, device="cuda")
    ops.backend.gmm_swiglu(x.cuda(), w.cuda(), sizes.cuda(), trans_b=trans_b, c=c, a_rows=row_index.cuda(),
                           c_rows=order.cuda())
    want_c = torch.zeros(600, hout)
    want_c[order.long()] = want
    check(c, want_c, "gathered and scattered")


@pytest.mark.parametrize("trans_b", [False, True])
def test_swiglu_autograd(ops, oracle, trans_b):
    # forward through the fused epilogue, backward by recomputation: against fp32 autograd through
    # the oracle's formula
    g = torch.Generator().manual_seed(89)
    sizes = torch.tensor([100, 0, 156])
    hin, hout = 136, 200
    a0 = torch.randn(256, hin, generator=g).to(torch.bfloat16)
    w0 = (torch.randn(3, *((2 * hout, hin) if trans_b else (hin, 2 * hout)), generator=g) * hin ** -0.5).to(torch.bfloat16)
    grad = torch.randn(256, hout, generator=g).to(torch.bfloat16)
    a, w = a0.cuda().requires_grad_(True), w0.cuda().requires_grad_(True)
    out = ops.gmm_swiglu(a, w, sizes.cuda(), trans_b)
    out.backward(grad.cuda())
    # Reference: the same steps from the oracle's loops, with a bf16 rounding wherever the operator
    # stores a bf16 tensor (the recomputed gate | up, the gradient with respect to them), so that
    # only fp32 summation order separates the two; the derivative itself is checked against
    # torch's autograd of silu(gate) * up.
    bf = lambda t: t.to(torch.bfloat16)
    check(out.detach(), oracle.swiglu_loop(a0, w0, sizes, trans_b=trans_b), "forward")
    gu = bf(oracle.gmm_loop(a0, w0, sizes, trans_b=trans_b)).float().requires_grad_(True)
    (torch.nn.functional.silu(gu[:, :hout]) * gu[:, hout:]).backward(grad.float())
    dgu = bf(gu.grad)
    want_a = oracle.gmm_loop(dgu, w0, sizes, trans_b=not trans_b)
    lhs, rhs = (dgu, a0) if trans_b else (a0, dgu)
    want_w = oracle.gmm_loop(lhs, rhs, sizes, trans_a=True)
    scale = lambda t: max(1.0, float(t.double().pow(2).mean().sqrt()))
    check(a.grad.float().cpu() / scale(want_a), want_a / scale(want_a), "input gradient")
    check(w.grad.float().cpu() / scale(want_w), want_w / scale(want_w), "weight gradient")
    assert (w.grad[1] == 0).all()


@pytest.mark.parametrize("config", [2, 5])
def test_fused_rows_and_swiglu_at_benchmark_shapes(ops, oracle, config):
    # the gather-fused load, the scatter-fused store and the SwiGLU epilogue at the row counts and
    # hidden sizes of configurations 2 and 5 (the output width halved for gate | up), against the
    # oracle's loop in fp32 on the GPU and CPU fp64 rows
    from grouped_gemm_amd import workloads
    w = workloads.make(config, device="cuda")
    sizes = w.batch_sizes
    t = w.tokens
    g = torch.Generator().manual_seed(90)
    perm = torch.randperm(t, generator=g).to(torch.int32).cuda()
    _announce("fused at full size", config)
    with torch.no_grad():
        want = oracle.gmm_loop(w.a[perm.long()], w.b, sizes, trans_b=w.trans_b)
        got = ops.backend.gmm_indexed(w.a, w.b, sizes.cuda(), trans_b=w.trans_b, a_rows=perm)
        check(got, want, "gathered rows")
        fp64_rows_check(w.a[perm.long()], w.b, sizes, w.trans_b, got)
        c = torch.empty_like(got)
        ops.backend.gmm_indexed(w.a, w.b, sizes.cuda(), trans_b=w.trans_b, c=c, a_rows=perm, c_rows=perm)
        want_c = torch.empty_like(want)
        want_c[perm.long()] = want
        check(c, want_c, "gathered and scattered rows")
        del want, want_c, c, got
        out = ops.backend.gmm_swiglu(w.a, w.b, sizes.cuda(), trans_b=w.trans_b)
        check(out, oracle.swiglu_loop(w.a, w.b, sizes, trans_b=w.trans_b), "swiglu")


# ------------------------------------------------- fp32-accumulated weight gradient

@pytest.mark.parametrize("on_device", [False, True])
@pytest.mark.parametrize("sizes,hin,hout", [
    ([128] * 8, 128, 128),
    ([300, 0, 17, 1000, 0, 129], 520, 776),        # empty experts, ragged depth and width
    ([0, 0, 0], 64, 72),
    ([5] * 70, 264, 136),
])
def test_accumulated_weight_gradient(ops, oracle, sizes, hin, hout, on_device):
    bs = torch.tensor(sizes, dtype=torch.int64)
    t = int(bs.sum())
    g = torch.Generator().manual_seed(31)
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
    b = torch.randn(t, hout, generator=g).to(torch.bfloat16)
    c0 = torch.randn(len(sizes), hin, hout, generator=g) * 8
    _announce("accumulate", sizes, hin, hout, on_device)
    c = c0.clone().cuda()
    dev_bs = bs.cuda() if on_device else bs
    got = ops.backend.accumulate_weight_gradient(a.cuda(), b.cuda(), dev_bs, c)
    assert got is c
    want = oracle.accumulate_weight_gradient_loop(a, b, bs, c0)
    # fp32 accumulation of exact bf16 products: the only error is the order of fp32 sums
    depth = max(sizes) if sizes else 0
    tol = 1e-6 * (depth ** 0.5 + 4) * (want.abs().max().item() + 8 * depth ** 0.5 + 1)
    assert (c.double().cpu() - want).abs().max().item() <= tol
    for e, size in enumerate(sizes):                   # an empty expert's slice is untouched
        if size == 0:
            assert torch.equal(c[e].cpu(), c0[e])
    # a second call adds the same product again: (c - c0) doubles, up to fp32 rounding
    first = c.double().cpu() - c0.double()
    ops.backend.accumulate_weight_gradient(a.cuda(), b.cuda(), dev_bs, c)
    second = c.double().cpu() - c0.double()
    assert (second - 2 * first).abs().max().item() <= 4 * tol


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_accumulated_weight_gradient_float8(ops, oracle, dtype):
    # fp8 operands added to an fp32 weight gradient: shallow groups (read-add-write), deep ones
    # (atomic additions), sizes the streaming kernels take and sizes they do not
    g = torch.Generator().manual_seed(66)
    for sizes, hin, hout in [([300, 0, 17, 129], 272, 144), ([3000, 2500], 256, 512), ([70, 5], 100, 24)]:
        _announce("accumulate fp8", dtype, sizes, hin, hout)
        bs = torch.tensor(sizes, dtype=torch.int64)
        t = int(bs.sum())
        a = torch.randn(t, hin, generator=g).to(dtype)
        b = torch.randn(t, hout, generator=g).to(dtype)
        c0 = torch.randn(len(sizes), hin, hout, generator=g)
        c = c0.clone().cuda()
        ops.backend.accumulate_weight_gradient(a.cuda(), b.cuda(), bs.cuda(), c)
        want = oracle.accumulate_weight_gradient_loop(a, b, bs, c0)
        # The fp8 matrix instruction sums the 64 products of one step aligned to the largest of
        # them and drops what lies more than 12 binary places below it (see the test below), so
        # the fp32 sum is not the exact one: per product at most 2^-12 of the largest product, and
        # the deviations of a sum add up like a random walk over its depth.
        amax, bmax = float(a.float().abs().max()), float(b.float().abs().max())
        tol = 2.0 ** -12 * amax * bmax * max(sizes) ** 0.5 + 1e-6 * float(want.abs().max())
        assert float((c.double().cpu() - want).abs().max()) <= tol
        for e, m in enumerate(sizes):
            if m == 0:
                assert torch.equal(c[e].cpu(), c0[e])


def test_float8_products_far_below_the_largest_of_a_step(ops):
    # What the fp8 matrix instruction (v_mfma_scale_f32_32x32x64_f8f6f4) does with products of very
    # different sizes, seen through the fp32-accumulated weight gradient: nine rows whose products
    # are 16 and eight smaller ones, two of them (-13 * 2^-13 and -45 * 2^-13) more than 11 binary
    # places below 16.  The exact sum is 15.383544921875 (every product and every partial sum is
    # exact in fp32, and bf16 operands give exactly that); the fp8 instruction returns
    # 15.38671875 on this device: the small products cut off below 2^-8.  The acceptance rule
    # for fp8 with an fp32 result follows from it: an error of at most 2^-12 of the largest product
    # of the step per product.  (After rounding to bf16, 8 binary places, none of it shows.)
    av = [4.0, -0.40625, 1.0, -0.75, -0.01953125, -1.125, -0.5625, -0.5, -1.875]
    bv = [4.0, 0.00390625, 0.75, 1.375, 0.28125, 1.125, -0.625, -0.46875, -0.1875]
    exact = sum(x * y for x, y in zip(av, bv))
    assert exact == 15.383544921875
    sizes = torch.tensor([9])
    for dtype in (torch.bfloat16, torch.float8_e4m3fn):
        a, b = torch.zeros(9, 32), torch.zeros(9, 32)
        a[:, 0], b[:, 0] = torch.tensor(av), torch.tensor(bv)
        a, b = a.to(dtype).cuda(), b.to(dtype).cuda()
        assert a[:, 0].float().tolist() == av and b[:, 0].float().tolist() == bv   # representable as they are
        c = torch.zeros(1, 32, 32, device="cuda")
        ops.backend.accumulate_weight_gradient(a, b, sizes, c)
        got = float(c[0, 0, 0])
        _announce("fp8 products", dtype, repr(got))
        if dtype == torch.bfloat16:
            assert got == exact
        else:
            assert abs(got - exact) <= 9 * 2.0 ** -12 * 16.0
        assert float(ops.backend.gmm(a, b, sizes, trans_a=True)[0, 0, 0]) == 15.375   # bf16(exact)
    # without the large product the small ones are summed exactly
    a, b = torch.zeros(8, 32), torch.zeros(8, 32)
    a[:, 0], b[:, 0] = torch.tensor(av[1:]), torch.tensor(bv[1:])
    c = torch.zeros(1, 32, 32, device="cuda")
    ops.backend.accumulate_weight_gradient(a.to(torch.float8_e4m3fn).cuda(), b.to(torch.float8_e4m3fn).cuda(),
                                           torch.tensor([8]), c)
    assert float(c[0, 0, 0]) == exact - 16.0


def test_accumulated_weight_gradient_full_size_and_errors(ops, oracle):
    from grouped_gemm_amd import workloads
    w = workloads.make(4, device="cuda")                # 8 x 4096 rows, 4096 x 14336
    sd = w.batch_sizes.cuda()
    c = torch.zeros(8, w.hidden_in, w.hidden_out, device="cuda")
    ops.backend.accumulate_weight_gradient(w.a, w.grad, sd, c)
    bf16 = ops.backend.gmm(w.a, w.grad, sd, trans_a=True)
    # same products, same fp32 accumulation order: rounding the fp32 result gives the bf16 one
    assert torch.equal(c.to(torch.bfloat16), bf16)
    ops.backend.accumulate_weight_gradient(w.a, w.grad, sd, c)
    assert torch.equal(c.to(torch.bfloat16), (2 * bf16.float()).to(torch.bfloat16))
    with pytest.raises(RuntimeError, match="float32"):
        ops.backend.accumulate_weight_gradient(w.a, w.grad, sd, c.to(torch.bfloat16))
    with pytest.raises(RuntimeError):
        ops.backend.accumulate_weight_gradient(w.a, w.grad, sd, c[:, :, :-8].contiguous())
    with pytest.raises(RuntimeError):
        ops.backend.accumulate_weight_gradient(w.a, w.grad[:-1], sd, c)


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
@pytest.mark.parametrize("long_side", ["in", "out"])
def test_hidden_sizes_at_the_documented_limit(ops, oracle, layout, long_side):
    # hidden_in or hidden_out = 2**22 - 8, the largest allowed: the 32-bit byte offsets inside a
    # tile (row * leading dimension) are then at their largest
    trans_a, trans_b = layout
    big, small = (1 << 22) - 8, 8
    hin, hout = (big, small) if long_side == "in" else (small, big)
    sizes = [3, 0, 6]
    bs = torch.tensor(sizes, dtype=torch.int64)
    t = int(bs.sum())
    g = torch.Generator().manual_seed(37)
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
    if trans_a:
        b = torch.randn(t, hout, generator=g).to(torch.bfloat16)
    else:
        b = torch.randn(len(sizes), *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
    _announce("limit", layout, hin, hout)
    out = ops.backend.gmm(a.cuda(), b.cuda(), bs.cuda(), trans_a=trans_a, trans_b=trans_b)
    want = oracle.gmm_loop(a, b, bs, trans_a=trans_a, trans_b=trans_b)
    # a depth of four million: compare with a tolerance that grows like sqrt(depth)
    scale = max(1.0, (hin if not trans_a else max(sizes)) ** 0.5 / 64)
    err = (out.float().cpu() - want).abs()
    assert bool((err <= scale * (ATOL + RTOL * want.abs())).all()), err.max().item()
    with pytest.raises(RuntimeError, match="2\\^22"):
        too_big = torch.zeros(1, (1 << 22), dtype=torch.bfloat16, device="cuda")
        ops.backend.gmm(too_big, torch.zeros(1, (1 << 22), 8, dtype=torch.bfloat16, device="cuda"),
                        torch.tensor([1]))


# ------------------------------------------------------------------------ edge cases

def test_output_fully_overwritten_and_tail_rows_untouched(ops, oracle):
    g = torch.Generator().manual_seed(3)
    sizes = torch.tensor([40, 0, 300])
    a = torch.randn(400, 64, generator=g).to(torch.bfloat16).cuda()     # 60 rows past the groups
    b = torch.randn(3, 64, 72, generator=g).to(torch.bfloat16).cuda()
    c = torch.full((400, 72), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.backend.gmm(a, b, sizes, c=c)
    assert not torch.isnan(c[:340]).any()
    assert torch.isnan(c[340:]).all()
    check(c[:340], oracle.gmm_loop(a.cpu(), b.cpu(), sizes)[:340], "forward")


def test_clamped_device_sizes_are_reported(ops, oracle):
    # host-resident sizes that are negative or sum past the rows of a raise; device-resident ones
    # are clamped by the kernel (it must not follow them) and the fact is left in a status word
    be = ops.backend.backend
    dev = torch.device("cuda", torch.cuda.current_device())
    be.size_status(dev)                                                   # clear
    g = torch.Generator().manual_seed(13)
    a = torch.randn(150, 64, generator=g).to(torch.bfloat16).cuda()
    b = torch.randn(3, 64, 72, generator=g).to(torch.bfloat16).cuda()
    ops.backend.gmm(a, b, torch.tensor([100, 30, 20]).cuda())
    assert be.size_status(dev) == 0
    for sizes, bits, used in [([100, 100, 100], be.status_rows_past_end, [100, 50, 0]),
                              ([-5, 100, 50], be.status_negative_size, [0, 100, 50]),
                              ([-1, 149, 7], be.status_negative_size | be.status_rows_past_end, [0, 149, 1])]:
        with pytest.raises(RuntimeError):
            ops.backend.gmm(a, b, torch.tensor(sizes))
        out = ops.backend.gmm(a, b, torch.tensor(sizes).cuda())
        assert be.size_status(dev) == bits, sizes
        assert be.size_status(dev) == 0                                   # reading clears
        rows = sum(used)
        check(out[:rows], oracle.gmm_loop(a.cpu(), b.cpu(), torch.tensor(used))[:rows], f"clamped {sizes}")


def test_all_experts_empty(ops):
    a = torch.zeros(0, 64, dtype=torch.bfloat16, device="cuda")
    b = torch.randn(4, 64, 72, device="cuda").to(torch.bfloat16)
    sizes = torch.zeros(4, dtype=torch.int64)
    out = ops.backend.gmm(a, b, sizes)
    assert out.shape == (0, 72)
    c = torch.ones(4, 64, 72, dtype=torch.bfloat16, device="cuda")
    ops.backend.gmm(a, torch.zeros(0, 72, dtype=torch.bfloat16, device="cuda"), sizes.cuda(), trans_a=True, c=c)
    assert (c == 0).all()


def test_more_than_512_experts(ops, oracle):
    g = torch.Generator().manual_seed(5)
    e = 700
    sizes = torch.randint(0, 6, (e,), generator=g)
    t = int(sizes.sum())
    a = torch.randn(t, 32, generator=g).to(torch.bfloat16)
    b = torch.randn(e, 32, 40, generator=g).to(torch.bfloat16)
    out = ops.backend.gmm(a.cuda(), b.cuda(), sizes)                      # host sizes: split launches
    check(out, oracle.gmm_loop(a, b, sizes), "forward")
    grad = torch.randn(t, 40, generator=g).to(torch.bfloat16)
    bg = ops.backend.gmm(a.cuda(), grad.cuda(), sizes, trans_a=True)
    check(bg, oracle.gmm_loop(a, grad, sizes, trans_a=True), "bgrad")
    # device-resident sizes: the reference stops at 512 experts (csrc/grouped_gemm.cu:120-124);
    # here every launch after the first sums up the sizes of the groups before it on the device
    out_dev = ops.backend.gmm(a.cuda(), b.cuda(), sizes.cuda())
    assert torch.equal(out_dev, out)
    bg_dev = ops.backend.gmm(a.cuda(), grad.cuda(), sizes.cuda(), trans_a=True)
    assert torch.equal(bg_dev, bg)


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False)])
def test_many_experts_device_sizes(ops, oracle, layout):
    # 1500 experts of 0..40 rows, sizes on the device: three launches, offsets of the later ones
    # derived in the kernel; equal to the host-resident call bit for bit and to the oracle
    trans_a, trans_b = layout
    g = torch.Generator().manual_seed(6)
    e, hin, hout = 1500, 72, 136
    sizes = torch.randint(0, 41, (e,), generator=g)
    sizes[::7] = 0
    t = int(sizes.sum())
    a = torch.randn(t, hin, generator=g).to(torch.bfloat16)
    if trans_a:
        b = torch.randn(t, hout, generator=g).to(torch.bfloat16)
    else:
        b = torch.randn(e, *((hout, hin) if trans_b else (hin, hout)), generator=g).to(torch.bfloat16)
    _announce("1500 experts", layout)
    dev = ops.backend.gmm(a.cuda(), b.cuda(), sizes.cuda(), trans_a=trans_a, trans_b=trans_b)
    host = ops.backend.gmm(a.cuda(), b.cuda(), sizes, trans_a=trans_a, trans_b=trans_b)
    assert torch.equal(dev, host)
    check(dev, oracle.gmm_loop(a, b, sizes, trans_a=trans_a, trans_b=trans_b), "1500 experts")


def test_gpu_validation_errors(ops):
    a = torch.zeros(8, 16, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(2, 16, 24, dtype=torch.bfloat16, device="cuda")
    bs = torch.tensor([3, 5])
    with pytest.raises(RuntimeError):
        ops.backend.gmm(a, b.cpu(), bs)
    with pytest.raises(RuntimeError):
        ops.backend.gmm(a, b, bs.int())
    with pytest.raises(RuntimeError):
        ops.backend.gmm(a, b, torch.tensor([3, 6]))                       # sums past the rows of a
    with pytest.raises(RuntimeError):
        ops.backend.gmm(a, b, bs, c=torch.zeros(8, 32, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(AssertionError):
        ops.backend.gmm(a, b, bs, trans_a=True, trans_b=True)


def test_needs_input_grad_is_respected(ops):
    a = torch.randn(64, 32, device="cuda").to(torch.bfloat16).requires_grad_(True)
    b = torch.randn(2, 32, 40, device="cuda").to(torch.bfloat16)
    out = ops.gmm(a, b, torch.tensor([30, 34]))
    out.sum().backward()
    assert a.grad is not None and b.grad is None


def test_runs_on_the_current_stream(ops, oracle):
    g = torch.Generator().manual_seed(11)
    sizes = torch.tensor([500, 12])
    a = torch.randn(512, 256, generator=g).to(torch.bfloat16).cuda()
    b = torch.randn(2, 256, 128, generator=g).to(torch.bfloat16).cuda()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        a2 = a * 2          # produced on s; the kernel must be ordered after it on s
        out = ops.backend.gmm(a2, b, sizes.cuda())
    s.synchronize()
    check(out / 2, oracle.gmm_loop(a.cpu(), b.cpu(), sizes), "forward")

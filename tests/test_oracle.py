"""Pins the CPU oracle before anything is compared against it.

Checks are chosen so that a plausible mistake fails one of them: non-square shapes
(a transposed operand changes the result or the shape), ragged sizes with zeros (an
off-by-one in the running offsets moves data between experts), a known answer that
does not come from the oracle's own formula (ones x ones = k), and a brute-force walk
in Python integers for the problem table.
"""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st


def _rand_bf16(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(torch.bfloat16)


# sizes include 0, 1 and values that are not multiples of anything
SIZES = [3, 0, 17, 1, 0, 40]


@pytest.mark.parametrize("trans_b", [False, True])
def test_c_loop_matches_library_matmul_nn_nt(oracle, trans_b):
    k, n = 24, 40                      # k != n so a swapped b layout cannot pass
    a = _rand_bf16(sum(SIZES), k, seed=1)
    b = _rand_bf16(len(SIZES), n, k, seed=2) if trans_b else _rand_bf16(len(SIZES), k, n, seed=2)
    bs = torch.tensor(SIZES)
    c32, c16 = oracle.gmm_c(a, b, bs, trans_b=trans_b)
    # library routine, one expert at a time, written out here independently
    start = 0
    for e, m in enumerate(SIZES):
        rhs = b[e].float().t() if trans_b else b[e].float()
        want = a[start:start + m].float() @ rhs
        torch.testing.assert_close(c32[start:start + m], want, rtol=1e-5, atol=1e-5)
        start += m
    torch.testing.assert_close(c16.float(), c32, rtol=2 ** -8, atol=0)  # one bf16 rounding
    torch.testing.assert_close(oracle.gmm_loop(a, b, bs, trans_b=trans_b), c32, rtol=1e-5, atol=1e-5)


def test_c_loop_matches_library_matmul_tn(oracle):
    m, n = 24, 40
    a = _rand_bf16(sum(SIZES), m, seed=3)
    b = _rand_bf16(sum(SIZES), n, seed=4)
    bs = torch.tensor(SIZES)
    c32, _ = oracle.gmm_c(a, b, bs, trans_a=True)
    assert c32.shape == (len(SIZES), m, n)
    start = 0
    for e, k in enumerate(SIZES):
        want = a[start:start + k].float().t() @ b[start:start + k].float()
        torch.testing.assert_close(c32[e], want, rtol=1e-5, atol=1e-5)
        if k == 0:
            assert (c32[e] == 0).all()
        start += k
    torch.testing.assert_close(oracle.gmm_loop(a, b, bs, trans_a=True), c32, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("trans_b", [False, True])
def test_autograd_loop_matches_c_loops(oracle, trans_b):
    # gmm_autograd_loop (forward and both gradients by autograd through the per-expert loop) against
    # the plain-C loops: forward is the NN / NT loop, the input gradient the loop with the opposite
    # layout of b, the weight gradient the TN loop with the operands in the order ops.py:25 uses
    k, n = 24, 40
    a = _rand_bf16(sum(SIZES), k, seed=11)
    b = _rand_bf16(len(SIZES), n, k, seed=12) if trans_b else _rand_bf16(len(SIZES), k, n, seed=12)
    grad = _rand_bf16(sum(SIZES), n, seed=13)
    bs = torch.tensor(SIZES)
    out, agrad, bgrad = oracle.gmm_autograd_loop(a, b, bs, trans_b, grad)
    torch.testing.assert_close(out, oracle.gmm_c(a, b, bs, trans_b=trans_b)[0], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(agrad, oracle.gmm_c(grad, b, bs, trans_b=not trans_b)[0], rtol=1e-5, atol=1e-5)
    lhs, rhs = (grad, a) if trans_b else (a, grad)
    want_bg = oracle.gmm_c(lhs, rhs, bs, trans_a=True)[0]
    assert bgrad.shape == b.shape == want_bg.shape
    torch.testing.assert_close(bgrad, want_bg, rtol=1e-5, atol=1e-5)


def test_tolerance_scales_with_the_data(oracle):
    # an all-zero answer against small expected values must fail; unit-scale data keeps atol 1e-2
    want = torch.full((64, 64), 3e-3)
    assert oracle.max_violation(torch.zeros(64, 64), want) > 0
    assert oracle.max_violation(want * 1.01, want) <= 0
    assert abs(oracle.atol_for(torch.randn(1000, 100)) - 1e-2) < 1e-3
    assert oracle.atol_for(torch.full((8, 8), 50.0)) == 1e-2


def test_swiglu_loop_known_values(oracle):
    # one expert, one depth: the products are the inputs themselves, so the result must be the
    # closed form at points fixed by hand: silu(0) = 0, silu(ln 3) = ln(3) * 3 / 4, silu(-ln 3) =
    # -ln(3) / 4, large negative gate -> 0, and the up value multiplies it
    import math
    ln3 = math.log(3.0)
    a = torch.ones(1, 1, dtype=torch.bfloat16)
    for gate, up, want in [(0.0, 5.0, 0.0), (2.0, 1.0, 2.0 / (1.0 + math.exp(-2.0))),
                           (-2.0, 3.0, -6.0 / (1.0 + math.exp(2.0))), (-60.0, 1.0, 0.0), (4.0, -0.5, -2.0 / (1 + math.exp(-4.0)))]:
        b = torch.tensor([[[gate, up]]], dtype=torch.bfloat16)               # (1, 1, 2): gate | up
        got = float(oracle.swiglu_loop(a, b, torch.tensor([1]))[0, 0])
        assert abs(got - want) <= 1e-6 * max(1.0, abs(want)), (gate, up, got, want)
    assert abs(ln3 * 0.75 - float(oracle.swiglu_loop(torch.ones(1, 1), torch.tensor([[[ln3, 1.0]]]), torch.tensor([1]))[0, 0])) < 1e-6
    # trans_b layout: rows of b are columns of the product, gate rows first
    g = torch.Generator().manual_seed(3)
    a2 = torch.randn(7, 5, generator=g).to(torch.bfloat16)
    b2 = torch.randn(2, 5, 6, generator=g).to(torch.bfloat16)
    bs = torch.tensor([3, 4])
    nn = oracle.swiglu_loop(a2, b2, bs)
    nt = oracle.swiglu_loop(a2, b2.transpose(1, 2).contiguous(), bs, trans_b=True)
    assert nn.shape == (7, 3) and torch.equal(nn, nt)
    want = torch.nn.functional.silu(oracle.gmm_loop(a2, b2[:, :, :3].contiguous(), bs)) * oracle.gmm_loop(a2, b2[:, :, 3:].contiguous(), bs)
    torch.testing.assert_close(nn, want, rtol=1e-6, atol=1e-6)


def test_swiglu_parts_and_tolerance_rule(oracle):
    import math
    # swiglu_parts: the float64 form agrees with the closed form at hand-fixed points and with the
    # fp32 loop on random data
    a = torch.ones(1, 1, dtype=torch.bfloat16)
    out, gate, up = oracle.swiglu_parts(a, torch.tensor([[[2.0, 3.0]]], dtype=torch.bfloat16), torch.tensor([1]))
    assert out.dtype == torch.float64 and float(gate) == 2.0 and float(up) == 3.0
    assert abs(float(out) - 6.0 / (1.0 + math.exp(-2.0))) < 1e-12
    g = torch.Generator().manual_seed(4)
    a2 = torch.randn(9, 24, generator=g).to(torch.bfloat16)
    b2 = torch.randn(3, 24, 10, generator=g).to(torch.bfloat16)
    bs = torch.tensor([4, 0, 5])
    for tb in (False, True):
        bb = b2.transpose(1, 2).contiguous() if tb else b2
        out, gate, up = oracle.swiglu_parts(a2, bb, bs, trans_b=tb)
        torch.testing.assert_close(out.float(), oracle.swiglu_loop(a2, bb, bs, trans_b=tb), rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(gate.float(), oracle.gmm_loop(a2, b2[:, :, :5].contiguous(), bs), rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(up.float(), oracle.gmm_loop(a2, b2[:, :, 5:].contiguous(), bs), rtol=1e-6, atol=1e-6)
    # the derivative the rule uses, against central differences of x / (1 + exp(-x)) in float64
    silu = lambda x: x / (1.0 + math.exp(-x))
    for x in (-30.0, -3.0, -0.5, 0.0, 0.7, 4.0, 25.0):
        sgm = 1.0 / (1.0 + math.exp(-x))
        assert abs(sgm * (1.0 + x * (1.0 - sgm)) - (silu(x + 1e-6) - silu(x - 1e-6)) / 2e-6) < 1e-8
    # the rule itself at a point worked out by hand: gate = 0, up = 200 (silu'(0) = 1/2, silu(0) = 0),
    # depth 8192 (sqrt(8192 / 16) = 22.627), pre-activation rms = sqrt((0 + 200^2) / 2) = 141.42:
    # delta = 10 * 2^-24 * 22.627 * 141.42 = 1.9073e-3, added term = 200 * 0.5 * delta = 0.19073
    want = torch.zeros(1, 1, dtype=torch.float64)
    tol = oracle.swiglu_tolerance(want, torch.zeros(1, 1), torch.full((1, 1), 200.0), 8192)
    assert abs(float(tol) - (0.0 + 0.19073)) < 2e-5, float(tol)    # rms(want) = 0: no absolute term
    # unit-size pre-activations: the added term is far below the plain tolerance
    gate, up = torch.randn(64, 64, generator=g).double(), torch.randn(64, 64, generator=g).double()
    want = gate * torch.sigmoid(gate) * up
    tol = oracle.swiglu_tolerance(want, gate, up, 512)
    plain = oracle.atol_for(want.float()) + oracle.RTOL * want.abs()
    assert float((tol - plain).max()) < 0.01 * oracle.atol_for(want.float())
    # and a dropped product (one term of size 1 missing from a pre-activation of a deep sum) is
    # still far outside it: d out = up * silu'(gate) * 1
    gate, up = torch.full((1, 1), 0.3, dtype=torch.float64), torch.full((1, 1), 150.0, dtype=torch.float64)
    want = gate * torch.sigmoid(gate) * up
    wrong = (gate - 1.0) * torch.sigmoid(gate - 1.0) * up
    assert float((wrong - want).abs()) > 50 * float(oracle.swiglu_tolerance(want, gate, up, 8192))


def test_float8_decode_known_values():
    # the oracle for fp8 operands is the per-expert loop on torch's fp32 decode of the bytes; pin the
    # decode on values fixed by the OCP formats (1.0, the largest finite value, the smallest
    # subnormal, a negative value), so that the fnuz variants or a wrong bias would fail
    e4 = torch.tensor([0x38, 0x7E, 0x01, 0xB8, 0x40], dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    assert e4.tolist() == [1.0, 448.0, 2.0 ** -9, -1.0, 2.0]
    e5 = torch.tensor([0x3C, 0x7B, 0x01, 0xBC, 0x40], dtype=torch.uint8).view(torch.float8_e5m2).float()
    assert e5.tolist() == [1.0, 57344.0, 2.0 ** -16, -1.0, 2.0]


def test_zero_k_known_answer(oracle):
    # grouped_gemm/ops_test.py:143-158: ones x ones over k rows is exactly k
    a = torch.ones(192, 128, dtype=torch.bfloat16)
    b = torch.ones(192, 128, dtype=torch.bfloat16)
    bs = torch.tensor([0, 128, 0, 64])
    for c in (oracle.gmm_c(a, b, bs, trans_a=True)[1].float(), oracle.gmm_loop(a, b, bs, trans_a=True)):
        assert (c[0] == 0).all() and (c[1] == 128).all() and (c[2] == 0).all() and (c[3] == 64).all()


def test_both_transposes_rejected(oracle):
    a = torch.ones(4, 8, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        oracle.gmm_c(a, a, torch.tensor([4]), trans_a=True, trans_b=True)


def test_linearity_in_a(oracle):
    # gmm(a1 + a2, b) == gmm(a1, b) + gmm(a2, b) up to fp32 rounding, with exactly
    # representable inputs (small integers) so the identity is exact
    g = torch.Generator().manual_seed(5)
    a1 = torch.randint(-3, 4, (sum(SIZES), 16), generator=g).to(torch.bfloat16)
    a2 = torch.randint(-3, 4, (sum(SIZES), 16), generator=g).to(torch.bfloat16)
    b = torch.randint(-3, 4, (len(SIZES), 16, 8), generator=g).to(torch.bfloat16)
    bs = torch.tensor(SIZES)
    lhs = oracle.gmm_c(a1 + a2, b, bs)[0]
    rhs = oracle.gmm_c(a1, b, bs)[0] + oracle.gmm_c(a2, b, bs)[0]
    assert torch.equal(lhs, rhs)


def _brute_table(sizes, hidden_in, hidden_out, trans_a, trans_b):
    """Walk in Python ints; offsets are sums of the element counts of earlier experts."""
    rows = []
    for e, s in enumerate(sizes):
        m, n, k = (hidden_in, hidden_out, s) if trans_a else (s, hidden_out, hidden_in)
        before = sizes[:e]
        a_off = sum((hidden_in * t) for t in before)                # both layouts: rows*hidden_in
        b_off = sum(t * hidden_out for t in before) if trans_a else e * hidden_in * hidden_out
        c_off = e * hidden_in * hidden_out if trans_a else sum(t * hidden_out for t in before)
        rows.append([m, n, k, m if trans_a else k, k if trans_b else n, n, a_off, b_off, c_off])
    return np.array(rows, dtype=np.int64).reshape(len(sizes), 9)


@settings(max_examples=200, deadline=None)
@given(st.lists(st.integers(0, 70000), min_size=1, max_size=40),
       st.sampled_from([(8, 16), (4096, 14336), (7168, 2048), (2048, 1408)]),
       st.sampled_from([(False, False), (False, True), (True, False)]))
def test_problem_tables_agree(oracle, sizes, hidden, trans):
    hidden_in, hidden_out = hidden
    trans_a, trans_b = trans
    walk, zero_fill, order = oracle.table_walk(sizes, hidden_in, hidden_out, trans_a, trans_b)
    closed = oracle.table_closed(sizes, hidden_in, hidden_out, trans_a, trans_b)
    viacumsum = oracle.table_numpy(sizes, hidden_in, hidden_out, trans_a, trans_b)
    brute = _brute_table(sizes, hidden_in, hidden_out, trans_a, trans_b)
    assert np.array_equal(walk, brute)
    assert np.array_equal(closed, brute)
    assert np.array_equal(viacumsum, brute)
    if trans_a:
        assert np.array_equal(zero_fill, (np.array(sizes) == 0).astype(np.int64))
        ks = np.array(sizes)[order]
        assert sorted(order.tolist()) == list(range(len(sizes)))
        assert (np.diff(ks) <= 0).all()
        # stable: equal k keep index order
        for i in range(len(order) - 1):
            if ks[i] == ks[i + 1]:
                assert order[i] < order[i + 1]
    else:
        assert not zero_fill.any() or hidden_in == 0
        assert np.array_equal(order, np.arange(len(sizes)))


def test_table_offsets_past_int32(oracle):
    # 256 experts x 7168 x 2048 elements of b: the last expert starts past 2**31
    sizes = [256] * 256
    t = oracle.table_closed(sizes, 7168, 2048, False, True)
    assert t[-1, 7] == 255 * 7168 * 2048 > 2 ** 31
    assert np.array_equal(t, oracle.table_numpy(sizes, 7168, 2048, False, True))


def test_zero_size_vector_from_reference_tests(oracle):
    # grouped_gemm/ops_test.py:124
    sizes = [219, 2246, 5, 8103, 1, 1117, 4693, 0]
    assert sum(sizes) == 16384
    t = oracle.table_numpy(sizes, 4096, 14336, False, False)
    assert t[:, 0].tolist() == sizes
    assert t[-1, 8] == 16384 * 14336 and t[-1, 6] == 16384 * 4096


def test_reference_generator_quirk(oracle):
    torch.manual_seed(0)
    x = oracle.ops_test_randn(2, 4, 8).float()
    assert (x <= 0).all() and (x > -1.0 / 32 - 1e-3).all()


def test_reference_acceptance_rule(oracle):
    x = torch.ones(100)
    y = x.clone()
    y[:2] = 2.0
    assert oracle.allclose_ops_test(x, y)          # 2 % differ: accepted
    y[:3] = 2.0
    assert not oracle.allclose_ops_test(x, y)      # 3 % differ: rejected

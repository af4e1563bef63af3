"""CPU oracle for the grouped-GEMM path (Python side).

TEST INFRASTRUCTURE ONLY.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import this module, and only as the checker.
The product (grouped_gemm_amd) never imports it.

Contents
  gmm_loop            per-expert torch.matmul loop; restates the test oracle of the
                      reference (grouped_gemm/ops_test.py:44-53) and extends it to
                      the trans_a layout by the definition at
                      csrc/grouped_gemm.cu:418-435.  With dtype=float32 the slices are
                      up-cast first, which gives the fp32-accumulated result the
                      tolerance is stated against.
  swiglu_loop         the gated activation silu(a @ gate) * (a @ up) on top of that loop.
  swiglu_parts / swiglu_tolerance
                      the same in float64 together with its two pre-activations, and the
                      acceptance rule for it when the pre-activations are large (deep products of
                      unscaled operands): the output tolerance plus what an fp32 accumulation
                      error of a pre-activation becomes once the other one multiplies it.
  gmm_c               same result from the plain-C triple loop in gg_oracle.c
                      (small shapes only).
  table_walk / table_closed / table_numpy
                      per-expert problem table (m, n, k, lda, ldb, ldc, a/b/c element
                      offsets): host walk (csrc/grouped_gemm.cu:159-190), closed forms
                      (csrc/fill_arguments.cuh:63-78) in C, and the same closed forms
                      from numpy.cumsum in int64.
  ops_test_randn      the reference tests' input generator (ops_test.py:39-41),
                      operator-precedence quirk included.
  allclose_ops_test   the reference tests' own acceptance rule (ops_test.py:10-17).
  assert_close_bf16   this build's acceptance rule: every element within
                      rtol 1.6e-2, atol 1e-2 of the fp32-accumulated oracle, the absolute
                      term scaled down to the output's root-mean-square where that is below 1.

Pinned in tests/test_oracle.py; no function here is "parity unpinned".
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgg_oracle.so")

RTOL = 1.6e-2
ATOL = 1e-2

TABLE_COLS = ("m", "n", "k", "lda", "ldb", "ldc", "a_off", "b_off", "c_off")


def build(force=False):
    """Compile gg_oracle.c with gcc (seconds)."""
    src = os.path.join(_HERE, "gg_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libgg_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = ctypes.CDLL(_LIB_PATH)
        i64p = ctypes.POINTER(ctypes.c_int64)
        lib.gg_oracle_gmm.restype = ctypes.c_int
        lib.gg_oracle_gmm.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                      ctypes.c_void_p, i64p, ctypes.c_int64, ctypes.c_int64,
                                      ctypes.c_int64, ctypes.c_int, ctypes.c_int]
        lib.gg_oracle_table_walk.restype = None
        lib.gg_oracle_table_walk.argtypes = [i64p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                             ctypes.c_int, ctypes.c_int, i64p, i64p, i64p]
        lib.gg_oracle_table_closed.restype = None
        lib.gg_oracle_table_closed.argtypes = [i64p, ctypes.c_int64, ctypes.c_int64,
                                               ctypes.c_int64, ctypes.c_int, ctypes.c_int, i64p]
        lib.gg_oracle_table_cols.restype = ctypes.c_int
        assert lib.gg_oracle_table_cols() == len(TABLE_COLS)
        _lib = lib
    return _lib


def _i64(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.int64))


def _i64p(arr):
    return arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int64))


# --------------------------------------------------------------------------- GEMM

def output_shape(a, b, batch_sizes, trans_a, trans_b):
    """Output shape rule of grouped_gemm/backend.py:17-21."""
    if trans_a:
        return (int(batch_sizes.shape[0]), a.shape[1], b.shape[1])
    return (a.shape[0], b.shape[1] if trans_b else b.shape[2])


def gmm_loop(a, b, batch_sizes, trans_a=False, trans_b=False, dtype=torch.float32):
    """Per-expert matmul loop on whatever device `a` lives on.

    NN/NT: rows [start, start+size) of `a` times b[e] (or b[e].t()), concatenated
    (ops_test.py:44-53).  TN: c[e] = a_e.t() @ b_e over the same row slices, zeros for
    an empty slice (csrc/grouped_gemm.cu:426-434, fill_arguments.cuh:100-119).
    Rows of the NN/NT output past sum(batch_sizes) are left zero.
    """
    assert not (trans_a and trans_b)
    sizes = [int(s) for s in batch_sizes.cpu().tolist()]
    shape = output_shape(a, b, batch_sizes, trans_a, trans_b)
    out = torch.zeros(shape, dtype=dtype, device=a.device)
    start = 0
    for e, size in enumerate(sizes):
        lhs = a[start:start + size].to(dtype)
        if trans_a:
            rhs = b[start:start + size].to(dtype)
            if size:
                out[e] = lhs.t() @ rhs
        else:
            rhs = b[e].to(dtype)
            if size:
                out[start:start + size] = lhs @ (rhs.t() if trans_b else rhs)
        start += size
    return out


def swiglu_loop(a, b, batch_sizes, trans_b=False, dtype=torch.float32):
    """silu(a_e @ gate_e) * (a_e @ up_e) per expert with b = [gate | up] side by side (gate first):
    the per-expert loop above on the two halves of b, combined elementwise in `dtype` with
    silu(x) = x / (1 + exp(-x)).  The products are the pinned loop; the activation is pinned against
    its closed form at known points in tests/test_oracle.py."""
    half = (b.shape[1] if trans_b else b.shape[2]) // 2
    gate_w = b[:, :half] if trans_b else b[:, :, :half]
    up_w = b[:, half:] if trans_b else b[:, :, half:]
    gate = gmm_loop(a, gate_w.contiguous(), batch_sizes, trans_b=trans_b, dtype=dtype)
    up = gmm_loop(a, up_w.contiguous(), batch_sizes, trans_b=trans_b, dtype=dtype)
    return gate / (1.0 + torch.exp(-gate)) * up


def swiglu_parts(a, b, batch_sizes, trans_b=False):
    """(out, gate, up) in float64: the two pre-activations a_e @ gate_e and a_e @ up_e from the
    per-expert loop above and out = silu(gate) * up."""
    half = (b.shape[1] if trans_b else b.shape[2]) // 2
    gate_w = b[:, :half] if trans_b else b[:, :, :half]
    up_w = b[:, half:] if trans_b else b[:, :, half:]
    gate = gmm_loop(a, gate_w.contiguous(), batch_sizes, trans_b=trans_b, dtype=torch.float64)
    up = gmm_loop(a, up_w.contiguous(), batch_sizes, trans_b=trans_b, dtype=torch.float64)
    return gate * torch.sigmoid(gate) * up, gate, up


# A pre-activation summed in fp32 over K products carries an error of about 2^-24 times the size of
# its partial sums per addition.  The matrix instruction adds 16 products at a time, so there are
# K / 16 additions; with errors that do not line up their sum grows like the square root of that
# count.  The factor in front covers the largest of ~10^7 such sums and partial sums a few times
# the typical pre-activation (measured on deep unscaled products: a tenth of this bound).
PREACT_ERROR_FACTOR = 10.0


def swiglu_tolerance(want, gate, up, hidden_in, rtol=RTOL, atol=ATOL):
    """Per-element tolerance for silu(gate) * up computed from fp32-accumulated pre-activations.

    out = silu(g) * u has d out = u * silu'(g) * dg + silu(g) * du: where one pre-activation is
    near zero and the other is large (|u| of a few hundred with unscaled operands and a depth of
    thousands), the output is small and an fp32 summation error dg of 1e-4 moves it by more than
    any tolerance proportional to the output.  No fp32-accumulating implementation can meet
    atol + rtol * |want| there (the per-expert loop in fp32 does not either), so the rule adds
    exactly that term: (|u * silu'(g)| + |silu(g)|) * delta with
    delta = PREACT_ERROR_FACTOR * 2^-24 * sqrt(hidden_in / 16) * rms(pre-activations),
    silu'(g) = s * (1 + g * (1 - s)), s = sigmoid(g).  For pre-activations of unit size the added
    term is far below atol and the rule is the plain one."""
    want, gate, up = want.double(), gate.double(), up.double()
    sig = torch.sigmoid(gate)
    dsilu = sig * (1.0 + gate * (1.0 - sig))
    scale = float(torch.cat([gate.flatten(), up.flatten()]).pow(2).mean().sqrt()) if gate.numel() else 0.0
    delta = PREACT_ERROR_FACTOR * 2.0 ** -24 * (max(hidden_in, 16) / 16.0) ** 0.5 * scale
    plain = atol_for(want.float(), atol) + rtol * want.abs()
    return plain + ((up * dsilu).abs() + (gate * sig).abs()) * delta


def accumulate_weight_gradient_loop(a, b, batch_sizes, c0, dtype=torch.float64):
    """c0[e] + a_e.t() @ b_e per expert: the accumulating form of the trans_a loop above.  The
    product is the same loop (pinned as gmm_loop is), the accumulation an exact addition in
    `dtype`; an empty expert leaves c0[e] as it is."""
    return c0.to(dtype) + gmm_loop(a, b, batch_sizes, trans_a=True, dtype=dtype)


def gmm_autograd_loop(a, b, batch_sizes, trans_b, grad, dtype=torch.float32):
    """Forward and both gradients by torch.autograd through the loop, on cloned fp32
    leaves, as the reference tests do (ops_test.py:67-80)."""
    a_ref = a.detach().to(dtype).clone().requires_grad_(True)
    b_ref = b.detach().to(dtype).clone().requires_grad_(True)
    sizes = [int(s) for s in batch_sizes.cpu().tolist()]
    outs, start = [], 0
    for e, size in enumerate(sizes):
        rhs = b_ref[e].t() if trans_b else b_ref[e]
        outs.append(a_ref[start:start + size] @ rhs)
        start += size
    out = torch.cat(outs)
    out.backward(grad.to(dtype)[:out.shape[0]])
    return out.detach(), a_ref.grad, b_ref.grad


def gmm_c(a, b, batch_sizes, trans_a=False, trans_b=False):
    """fp32-accumulated result (not rounded) and its bf16 rounding from the C loops."""
    lib = _load()
    a = a.detach().cpu().contiguous()
    b = b.detach().cpu().contiguous()
    assert a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16
    sizes = _i64(batch_sizes.cpu().numpy())
    shape = output_shape(a, b, batch_sizes, trans_a, trans_b)
    c32 = torch.zeros(shape, dtype=torch.float32)
    c16 = torch.zeros(shape, dtype=torch.bfloat16)
    hidden_in = a.shape[1]
    hidden_out = b.shape[1] if (trans_a or trans_b) else b.shape[2]
    rc = lib.gg_oracle_gmm(a.data_ptr(), b.data_ptr(), c16.data_ptr(), c32.data_ptr(),
                           _i64p(sizes), len(sizes), hidden_in, hidden_out,
                           int(trans_a), int(trans_b))
    if rc != 0:
        raise ValueError("trans_a and trans_b cannot both be set")
    return c32, c16


# ------------------------------------------------------------------ problem table

def table_walk(batch_sizes, hidden_in, hidden_out, trans_a, trans_b):
    lib = _load()
    sizes = _i64(batch_sizes)
    e = len(sizes)
    table = np.zeros((e, len(TABLE_COLS)), dtype=np.int64)
    zero_fill = np.zeros(e, dtype=np.int64)
    order = np.zeros(e, dtype=np.int64)
    lib.gg_oracle_table_walk(_i64p(sizes), e, hidden_in, hidden_out, int(trans_a), int(trans_b),
                             _i64p(table), _i64p(zero_fill), _i64p(order))
    return table, zero_fill, order


def table_closed(batch_sizes, hidden_in, hidden_out, trans_a, trans_b):
    lib = _load()
    sizes = _i64(batch_sizes)
    table = np.zeros((len(sizes), len(TABLE_COLS)), dtype=np.int64)
    lib.gg_oracle_table_closed(_i64p(sizes), len(sizes), hidden_in, hidden_out, int(trans_a),
                               int(trans_b), _i64p(table))
    return table


def table_numpy(batch_sizes, hidden_in, hidden_out, trans_a, trans_b):
    """Closed forms of csrc/fill_arguments.cuh:63-78 from an int64 exclusive cumsum."""
    sizes = _i64(batch_sizes)
    e = len(sizes)
    cumsum = np.cumsum(sizes, dtype=np.int64) - sizes
    idx = np.arange(e, dtype=np.int64)
    m = np.full(e, hidden_in, np.int64) if trans_a else sizes
    n = np.full(e, hidden_out, np.int64)
    k = sizes if trans_a else np.full(e, hidden_in, np.int64)
    lda = m if trans_a else k
    ldb = k if trans_b else n
    ldc = n
    if trans_a:
        a_off, b_off, c_off = m * cumsum, cumsum * n, idx * m * n
    else:
        a_off, b_off, c_off = cumsum * k, idx * k * n, cumsum * n
    return np.stack([m, n, k, lda, ldb, ldc, a_off, b_off, c_off], axis=1)


# ------------------------------------------------------- generators and criteria

def ops_test_randn(bs, x, y):
    """(U[0,1) - 1.0) / (x*y): values in (-1/(xy), 0] (ops_test.py:39-41)."""
    return ((torch.rand(bs, x, y) - 0.5 * 2) / (y * x)).to(torch.bfloat16)


def allclose_ops_test(x, y, pct=2.0):
    """At most `pct` percent of elements outside rtol=1e-5 (ops_test.py:10-17)."""
    mask = torch.isclose(x.float().cpu(), y.float().cpu(), rtol=1e-5)
    pct_diff = float(mask.numel() - mask.sum()) / max(mask.numel(), 1) * 100
    return pct_diff <= pct


def atol_for(want_fp32, atol=ATOL):
    """The absolute term of the tolerance, scaled to the data: `atol` where the expected output
    has unit scale or more, `atol` times its root-mean-square where it is smaller, so that an
    output of small numbers cannot pass by being small (an all-zero answer against expected
    values of a few thousandths, say)."""
    want = want_fp32.float()
    if want.numel() == 0:
        return atol
    rms = float(want.double().pow(2).mean().sqrt())
    return atol * min(1.0, rms)


def max_violation(got, want_fp32, rtol=RTOL, atol=ATOL):
    """max over elements of |got-want| - (atol_for(want) + rtol*|want|); <= 0 means pass."""
    got = got.float()
    want = want_fp32.float()
    if got.numel() == 0:
        return 0.0
    return float(((got - want).abs() - (atol_for(want, atol) + rtol * want.abs())).max())


def assert_close_bf16(got, want_fp32, rtol=RTOL, atol=ATOL, what=""):
    assert tuple(got.shape) == tuple(want_fp32.shape), (what, got.shape, want_fp32.shape)
    v = max_violation(got, want_fp32, rtol, atol)
    assert v <= 0.0, f"{what}: element outside rtol={rtol} atol={atol} (scaled to the data) by {v}"


def cpu_loop_bf16(a, b, batch_sizes, trans_a=False, trans_b=False):
    """The CPU baseline: the same loop on bf16 CPU tensors through torch's CPU matmul."""
    return gmm_loop(a, b, batch_sizes, trans_a, trans_b, dtype=torch.bfloat16)

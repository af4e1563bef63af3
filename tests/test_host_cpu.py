"""CPU-only checks of the host side: the Python surface mirrors the reference's, every
validation rule raises before the device is touched, the C-ABI library loads and
exports what include/grouped_gemm_hip.h declares, and the golden fixture of
configuration 1 still matches the oracle.  No GPU, no compute calls."""
import ctypes
import importlib.util
import inspect
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIP_LIB = os.path.join(ROOT, "grouped_gemm_amd", "libgrouped_gemm_hip.so")


def bf16(*shape):
    return torch.zeros(*shape, dtype=torch.bfloat16)


# ------------------------------------------------------------------ Python surface

def test_extension_module_imports_top_level_first():
    # setup.py:35 of the reference installs the extension under the top-level name
    # grouped_gemm_backend; here it resolves once either package has been imported, whichever
    # comes first, and torch before it (backend.py:1-3)
    import subprocess
    import sys
    for pkg in ("grouped_gemm", "grouped_gemm_amd"):
        code = (f"import sys; sys.path.insert(0, {ROOT!r}); import {pkg}; import grouped_gemm_backend as m; "
                "assert callable(m.gmm)")
        subprocess.run([sys.executable, "-c", code], check=True)


def test_package_layout_matches_reference():
    # grouped_gemm/__init__.py:1-2, ops.py:1, ops_test.py:5,154
    import grouped_gemm
    from grouped_gemm import ops
    import grouped_gemm.backend as be
    import grouped_gemm_backend
    assert ops.backend is be
    assert be.backend is grouped_gemm_backend
    assert list(inspect.signature(ops.gmm).parameters) == ["a", "b", "batch_sizes", "trans_b"]
    assert list(inspect.signature(be.gmm).parameters) == ["a", "b", "batch_sizes", "trans_a", "trans_b", "c"]
    assert inspect.signature(be.gmm).parameters["c"].default is None
    assert issubclass(ops.GroupedGemm, torch.autograd.Function)


def test_allocate_output_shapes_and_asserts():
    # grouped_gemm/backend.py:11-22
    from grouped_gemm_amd.backend import _allocate_output
    bs = torch.tensor([3, 5])
    assert _allocate_output(bf16(8, 16), bf16(2, 16, 24), bs, False, False).shape == (8, 24)
    assert _allocate_output(bf16(8, 16), bf16(2, 24, 16), bs, False, True).shape == (8, 24)
    out = _allocate_output(bf16(8, 16), bf16(8, 24), bs, True, False)
    assert out.shape == (2, 16, 24) and out.dtype == torch.bfloat16
    with pytest.raises(AssertionError):
        _allocate_output(bf16(8, 16), bf16(8, 24), bs, True, True)
    with pytest.raises(AssertionError):
        _allocate_output(bf16(8, 16), bf16(2, 16, 24), bs.view(1, 2), False, False)
    with pytest.raises(AssertionError):
        _allocate_output(bf16(2, 4, 16), bf16(2, 16, 24), bs, False, False)
    with pytest.raises(AssertionError):
        _allocate_output(bf16(8, 16), bf16(16, 24), bs, False, False)
    with pytest.raises(AssertionError):
        _allocate_output(bf16(8, 16), bf16(2, 8, 24), bs, True, False)


def test_cpu_tensors_are_rejected_by_gmm():
    # csrc/grouped_gemm.cu:490: a must be on the GPU; surfaces as RuntimeError
    from grouped_gemm import ops
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ops.gmm(bf16(8, 16), bf16(2, 16, 24), torch.tensor([3, 5]))


GOOD = dict(a=(8, 16), b=(2, 16, 24), c=(8, 24), bs=[3, 5], ta=False, tb=False)


def _validate(**kw):
    import grouped_gemm_backend
    cfg = dict(GOOD)
    cfg.update(kw)
    a = cfg.get("a_t", bf16(*cfg["a"]))
    b = cfg.get("b_t", bf16(*cfg["b"]))
    c = cfg.get("c_t", bf16(*cfg["c"]))
    bs = cfg.get("bs_t", torch.tensor(cfg["bs"], dtype=torch.int64))
    grouped_gemm_backend.validate(a, b, c, bs, cfg["ta"], cfg["tb"])


def test_validate_accepts_the_three_layouts():
    _validate()
    _validate(b=(2, 24, 16), tb=True)
    _validate(b=(8, 24), c=(2, 16, 24), ta=True)


@pytest.mark.parametrize("kw", [
    dict(ta=True, tb=True),                                     # grouped_gemm.cu:476
    dict(bs_t=torch.tensor([[3, 5]])),                          # :485
    dict(bs_t=torch.tensor([3, 5], dtype=torch.int32)),         # :486
    dict(a=(2, 4, 16)),                                         # :491
    dict(a_t=torch.zeros(8, 16)),                               # :492
    dict(b_t=torch.zeros(2, 16, 24, dtype=torch.float16)),      # :505
    dict(c_t=torch.zeros(8, 24)),                               # :506
    dict(ta=True, b=(2, 4, 24), c=(2, 16, 24)),                 # :517
    dict(ta=True, b=(8, 24), c=(2 * 16, 24)),                   # :518
    dict(ta=True, b=(7, 24), c=(2, 16, 24)),                    # :519
    dict(ta=True, b=(8, 24), c=(3, 16, 24)),                    # :520
    dict(ta=True, b=(8, 24), c=(2, 8, 24)),                     # :521
    dict(ta=True, b=(8, 24), c=(2, 16, 32)),                    # :522
    dict(b=(16, 24)),                                           # :524
    dict(c=(2, 4, 24)),                                         # :525
    dict(b=(2, 8, 24)),                                         # :531 contraction mismatch
    dict(tb=True),                                              # :531 with trans_b: b.size(2) != a.size(1)
    dict(bs=[3, 4, 1]),                                         # :534
    dict(c=(8, 32)),                                            # output shape (checked here, not in the reference)
    dict(a_t=bf16(16, 8).t()),                                  # :538
    dict(b_t=bf16(2, 24, 16).transpose(1, 2)),                  # :539
    dict(c_t=bf16(24, 8).t()),                                  # :540
])
def test_validate_rejects(kw):
    with pytest.raises(RuntimeError):
        _validate(**kw)


# ------------------------------------------------------------------------ C ABI

def _declared_functions():
    text = open(os.path.join(ROOT, "include", "grouped_gemm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gg_[a-z0-9_]+)\s*\(", text)))


def test_c_abi_exports_every_declared_symbol():
    names = _declared_functions()
    assert {"gg_gmm_bf16", "gg_gmm", "gg_gmm_no_alloc", "gg_init", "gg_gmm_bf16_acc_f32", "gg_debug_schedule",
            "gg_last_error", "gg_version", "gg_tile_shape"} <= set(names)
    lib = ctypes.CDLL(HIP_LIB)
    for n in names:
        assert hasattr(lib, n), n


def test_c_abi_argument_errors_need_no_device():
    lib = ctypes.CDLL(HIP_LIB)
    lib.gg_last_error.restype = ctypes.c_char_p
    i64 = ctypes.c_int64
    sizes = (i64 * 2)(3, 5)
    call = lambda hin, hout, ta, tb, tokens=8, e=2: lib.gg_gmm_bf16(
        None, None, None, sizes, 0, i64(e), i64(tokens), i64(hin), i64(hout), ta, tb, None)
    assert call(16, 24, 1, 1) == -1 and b"both" in lib.gg_last_error()
    assert call(-8, 24, 0, 0) == -1
    assert call(16, 24, 0, 0, tokens=1 << 31) == -2
    assert call(16, 24, 0, 0, e=0) == 0                       # nothing to do
    # fake, never dereferenced pointers: the alignment check comes before any device call
    ptr = ctypes.c_void_p
    misaligned = lib.gg_gmm_bf16(ptr(4096), ptr(8192 + 1), ptr(12288), sizes, 0, i64(2), i64(8), i64(16),
                                 i64(24), 0, 0, None)
    assert misaligned == -2 and b"aligned to their element size" in lib.gg_last_error()
    # the accumulating form: tighter limit on the hidden sizes, checked before anything else
    acc = lib.gg_gmm_bf16_acc_f32(ptr(4096), ptr(8192), ptr(12288), sizes, 0, i64(2), i64(8), i64(1 << 20),
                                  i64(24), None)
    assert acc == -2 and b"2^20" in lib.gg_last_error()
    # host-resident sizes that would wrap a running sum are rejected one by one, before any device call
    huge = (i64 * 2)(10, (1 << 63) - 1)
    rc = lib.gg_gmm_bf16(ptr(4096), ptr(8192), ptr(12288), huge, 0, i64(2), i64(16), i64(16), i64(24), 0, 0, None)
    assert rc == -1 and b"sum past" in lib.gg_last_error()
    bm, bn, bk = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert lib.gg_tile_shape(i64(8), i64(32768), 0, 0, ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(bk)) == 0
    assert (bm.value, bn.value, bk.value) == (256, 256, 64)
    assert lib.gg_tile_shape(i64(256), i64(25600), 0, 1, ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(bk)) == 0
    assert bm.value == 128          # few rows per group: the shorter tile
    assert bm.value > 0 and bn.value > 0 and bk.value > 0
    assert lib.gg_version() >= 100


def test_validate_element_types():
    # past the reference (bfloat16 only, grouped_gemm.cu:492, 505-506): float16 for all three
    # tensors alike; float8 operands with a bfloat16 output
    _validate(a_t=torch.zeros(8, 16, dtype=torch.float16), b_t=torch.zeros(2, 16, 24, dtype=torch.float16),
              c_t=torch.zeros(8, 24, dtype=torch.float16))
    for f8 in (torch.float8_e4m3fn, torch.float8_e5m2):
        _validate(a_t=torch.zeros(8, 16, dtype=f8), b_t=torch.zeros(2, 16, 24, dtype=f8))     # c bfloat16
        with pytest.raises(RuntimeError):
            _validate(a_t=torch.zeros(8, 16, dtype=f8), b_t=torch.zeros(2, 16, 24, dtype=f8),
                      c_t=torch.zeros(8, 24, dtype=f8))
    with pytest.raises(RuntimeError):
        _validate(a_t=torch.zeros(8, 16, dtype=torch.float16), b_t=torch.zeros(2, 16, 24, dtype=torch.float16))
    with pytest.raises(RuntimeError):
        _validate(a_t=torch.zeros(8, 16, dtype=torch.float8_e4m3fn), b_t=torch.zeros(2, 16, 24, dtype=torch.float8_e5m2))


class _Args(ctypes.Structure):
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


def test_general_entry_point_argument_errors_need_no_device():
    lib = ctypes.CDLL(HIP_LIB)
    lib.gg_last_error.restype = ctypes.c_char_p
    lib.gg_gmm.argtypes = [ctypes.c_void_p]
    sizes = (ctypes.c_int64 * 2)(3, 5)

    def call(**kw):
        g = _Args()
        g.struct_bytes = ctypes.sizeof(_Args)
        g.a, g.b, g.c = 4096, 8192, 12288            # never dereferenced: every case fails before the device
        g.batch_sizes = ctypes.addressof(sizes)
        g.num_groups, g.tokens, g.hidden_in, g.hidden_out = 2, 8, 16, 24
        for k, v in kw.items():
            setattr(g, k, v)
        return lib.gg_gmm(ctypes.byref(g)), lib.gg_last_error()

    assert call(struct_bytes=8)[0] == -1
    assert lib.gg_gmm(None) == -1
    assert call(dtype=9) == (-1, b"dtype must be one of GG_DTYPE_*")
    assert call(epilogue=7)[0] == -1
    rc, msg = call(epilogue=1, trans_a=1)
    assert rc == -1 and b"SwiGLU" in msg
    rc, msg = call(accumulate_f32=1)
    assert rc == -1 and b"trans_a" in msg
    rc, msg = call(trans_a=1, c_row_index=64)
    assert rc == -1 and b"c_row_index" in msg
    rc, msg = call(b_row_index=64)
    assert rc == -1 and b"b_row_index" in msg
    assert call(a_num_rows=-1)[0] == -1
    assert call(b_num_rows=-1)[0] == -1
    assert call(c_num_rows=-1)[0] == -1
    rc, msg = call(c=12288 + 1)
    assert rc == -2 and b"element size" in msg


def test_workspace_bytes_for_needs_no_device():
    """gg_workspace_bytes_for: nothing for calls that can never cut tiles along the depth, the
    full workspace for deep products and weight gradients."""
    lib = ctypes.CDLL(HIP_LIB)
    lib.gg_workspace_bytes_for.argtypes = [ctypes.c_void_p]
    lib.gg_workspace_bytes_for.restype = ctypes.c_uint64
    full = 4096 + 256 * 256 * 256 * 4

    def want(**kw):
        g = _Args()
        g.struct_bytes = ctypes.sizeof(_Args)
        g.a, g.b, g.c = 4096, 8192, 12288
        g.num_groups, g.tokens, g.hidden_in, g.hidden_out = 8, 32768, 4096, 14336
        for k, v in kw.items():
            setattr(g, k, v)
        return lib.gg_workspace_bytes_for(ctypes.byref(g))

    assert lib.gg_workspace_bytes_for(None) == 0
    assert want(struct_bytes=4) == 0
    assert want() == 0                                     # 64 depth slices: too shallow
    assert want(hidden_in=14336, hidden_out=4096) == full  # 224 slices
    assert want(hidden_in=6144) == full and want(hidden_in=6080) == 0
    # the depth is a group's rows, and one group may hold them all (deep groups among shallow ones
    # are cut along the depth)
    assert want(trans_a=1) == full
    assert want(trans_a=1, tokens=6144) == full and want(trans_a=1, tokens=6080) == 0
    assert want(trans_a=1, tokens=65536, hidden_in=4097) == 0   # general kernels
    assert want(trans_a=1, tokens=65536, a=4096 + 2) == 0       # off the 4-byte boundary
    assert want(hidden_in=14336, a_row_index=64) == 0      # scattered or gathered tiles stay whole
    assert want(hidden_in=14336, hidden_out=2048, epilogue=1) == 0
    assert want(hidden_in=14336, flags=1) == 0 and want(hidden_in=14336, flags=4) == 0
    assert want(dtype=2, hidden_in=12288) == full and want(dtype=2, hidden_in=12160) == 0


def test_row_index_bounds_reach_every_kernel():
    """The C ABI hands the row counts that bound a row index to the general kernels as it does to
    the streaming ones (checked in the sources: no GPU test feeds bad indices on purpose)."""
    api = open(os.path.join(ROOT, "grouped_gemm_amd", "csrc", "gmm_api.hip")).read()
    for field in ("gp.a_num_rows = index_rows.a", "gp.b_num_rows = index_rows.b", "gp.c_num_rows = index_rows.c",
                  "p.a_index_rows =", "p.c_index_rows ="):
        assert field in api, field
    generic = open(os.path.join(ROOT, "grouped_gemm_amd", "csrc", "gmm_generic.hpp")).read()
    assert "strided < index_rows" in generic and "mem_row >= gp.c_num_rows" in generic


# ----------------------------------------------------------------- workloads

def test_workload_generators():
    from grouped_gemm_amd import workloads
    g = torch.Generator().manual_seed(0)
    s2 = workloads.router_sizes(16384, 8, 2, g)
    assert int(s2.sum()) == 32768 and s2.numel() == 8 and int(s2.min()) > 0
    s3 = workloads.zipf_sizes(49152, 64, 1.2, 4, g)
    assert int(s3.sum()) == 49152 and int((s3 == 0).sum()) >= 4
    s5 = workloads.poisson_sizes(65536, 256, g)
    assert int(s5.sum()) == 65536 and s5.numel() == 256 and int(s5.min()) >= 0
    w = workloads.make(3, device="cpu", shrink=16)
    assert w.a.shape == (49152 // 16, 128) and w.b.shape == (64, 128, 88) and not w.trans_b
    assert int(w.batch_sizes.sum()) == w.tokens
    w5 = workloads.make(5, device="cpu", shrink=32)
    assert w5.trans_b and w5.b.shape == (256, 64, 224)
    assert w5.flops_per_gemm() == 2 * w5.tokens * 224 * 64


# -------------------------------------------------------------- golden fixture

def test_config1_fixture_matches_oracle(oracle):
    spec = importlib.util.spec_from_file_location(
        "make_config1", os.path.join(ROOT, "tests", "golden", "make_config1.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    a, b, grad, sizes = mod.inputs()
    fwd, agrad, bgrad = mod.expected(a, b, grad, sizes)
    gold = np.load(os.path.join(ROOT, "tests", "golden", "config1.npz"))
    assert np.array_equal(gold["fwd"], fwd[::8].numpy())
    assert np.array_equal(gold["agrad"], agrad[::8].numpy())
    assert np.array_equal(gold["bgrad"], bgrad[:, ::8].numpy())
    # the same numbers from the library routine, by autograd through the loop
    out, ag, bg = oracle.gmm_autograd_loop(a, b, sizes, False, grad)
    torch.testing.assert_close(out, fwd, rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(ag, agrad, rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(bg, bgrad, rtol=1e-5, atol=1e-4)


# ----------------------------------------------------------------- traceable operator

def test_traceable_operator_shapes_without_a_device():
    # the torch.library form of the operator: output shapes for all three layouts from fake
    # tensors alone (what torch.compile needs), no kernel runs
    from torch._subclasses.fake_tensor import FakeTensorMode
    from grouped_gemm_amd import ops
    with FakeTensorMode():
        a = torch.empty(100, 64, dtype=torch.bfloat16)
        bs = torch.empty(4, dtype=torch.int64)
        assert ops.gmm_traceable(a, torch.empty(4, 64, 96, dtype=torch.bfloat16), bs).shape == (100, 96)
        assert ops.gmm_traceable(a, torch.empty(4, 96, 64, dtype=torch.bfloat16), bs, trans_b=True).shape == (100, 96)
        wgrad = torch.ops.grouped_gemm_amd.gmm(a, torch.empty(100, 96, dtype=torch.bfloat16), bs, True, False)
        assert wgrad.shape == (4, 64, 96) and wgrad.dtype == torch.bfloat16


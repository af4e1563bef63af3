#!/usr/bin/env python3
"""Benchmark: grouped GEMM forward + backward at the Mixtral-8x7B w1 shape on one MI355X.

One step = the three grouped GEMMs of one training step of the expert FFN weight w1,
exactly the calls grouped_gemm.ops.GroupedGemm makes: forward (NN), input gradient
(NT) and weight gradient (TN), with device-resident batch_sizes.  Inputs are synthetic
(seeded randn * 0.02, router-multinomial group sizes) and resident in HBM before the
timed region.  Prints ONE JSON line.

  value      TFLOP/s over the timed steps (2*T*K*N flops per GEMM, padding never counted)
  roofline   the slowest of the three kernels against the roof that bounds the workload (bf16
             dense MFMA peak, or the HBM peak when flops / algorithmic bytes is below the ridge), its
             duration taken from HIP events recorded around each launch inside the timed
             region (same stream the kernels run on)
  cpu_baseline  the oracle's per-expert loop (bf16 CPU tensors, torch CPU matmul) on a
             bounded slice of the same workload, all host cores
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6   # 256 CU x 4096 flop/clk x 2.4 GHz, dense
PEAK_HBM_GBPS = 8000.0

# Bytes per launch between L2 and the fabric, from two rocprofv3 --pmc runs of this file per
# configuration (FETCH_SIZE scaled x2.0 and WRITE_SIZE x1.0 by a 1 GiB device copy, both in KiB).
# Profiled once, not in this run: the table belongs to one revision of the kernel sources, named by
# the hash below (kernel_sources_sha16), and is reported only while the sources still have that
# hash; the summary under profiles/ holds the figures, the commands and the commit.
_TRAFFIC_KERNEL_SOURCES = ("gmm_kernel.hpp", "gmm_api.hip", "gmm_variants.hpp", "gmm_variants.def", "gmm_variant.hip")
_TRAFFIC_KERNEL_SHA16 = "7b530b46563c7867"
_TRAFFIC_SOURCE = ("profiles/gmm_kernel_mixtral_w1_hbm_traffic.md and profiles/gmm_kernel_configs_3_4_5_stats_and_traffic.md "
                   "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, kernel sources sha16 " + _TRAFFIC_KERNEL_SHA16 +
                   ", commit 6d629b3; profiled once, not in this run)")


def kernel_sources_sha16():
    """First 16 hex digits of the SHA-256 over the streaming kernel's sources."""
    import hashlib
    h = hashlib.sha256()
    for name in _TRAFFIC_KERNEL_SOURCES:
        with open(os.path.join(ROOT, "grouped_gemm_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def _traffic(fetch_kib, write_kib):
    return {"bytes": (fetch_kib * 2.0 + write_kib) * 1024, "source": _TRAFFIC_SOURCE}


MEASURED_TRAFFIC = {
    2: {"fwd": _traffic(3987640, 917582), "agrad": _traffic(3327810, 289978), "bgrad": _traffic(2753890, 917538)},
    3: {"fwd": _traffic(414260, 135176)},
    4: {"bgrad": _traffic(2753050, 917541)},
    5: {"fwd": _traffic(4225870, 262249), "agrad": _traffic(4955900, 917720), "bgrad": _traffic(1851750, 7344000)},
}


def mfma_rate(zero_operands, launches):
    """TFLOP/s of the bf16 matrix instruction alone (bench_mfma_probe.hip, built next to this file
    by grouped_gemm_amd/build.py: a helper of the benchmark, not of the library)."""
    import ctypes
    path = os.path.join(ROOT, "libbench_mfma_probe.so")
    if not os.path.exists(path):
        from grouped_gemm_amd import build as _build
        _build.build_bench_probe()
    lib = ctypes.CDLL(path)
    lib.bench_mfma_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
    lib.bench_mfma_rate.restype = ctypes.c_int
    tflops = ctypes.c_float(0.0)
    rc = lib.bench_mfma_rate(1 if zero_operands else 0, launches, ctypes.byref(tflops))
    if rc != 0:
        raise RuntimeError(f"bench_mfma_rate failed with hipError_t {rc}")
    return tflops.value


def cpu_baseline(w, budget_s=12.0):
    """Oracle loop on the host cores: forward, input gradient and weight gradient of the
    same workload through torch's CPU bf16 matmul.  A calibration run on a slice of expert 0
    sizes the sample: whole passes over all experts if one pass fits the budget, else the
    leading experts that do."""
    import torch
    from oracle import gmm_oracle
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    hin, hout = w.hidden_in, w.hidden_out
    sizes = w.batch_sizes

    def run(a, b, g, bs):
        t0 = time.perf_counter()
        gmm_oracle.cpu_loop_bf16(a, b, bs, trans_b=w.trans_b)
        gmm_oracle.cpu_loop_bf16(g, b, bs, trans_b=not w.trans_b)
        lhs, rhs = (g, a) if w.trans_b else (a, g)
        gmm_oracle.cpu_loop_bf16(lhs, rhs, bs, trans_a=True)
        return time.perf_counter() - t0

    rows = max(1, min(256, int(sizes[0])))
    cal = (w.a[:rows].cpu(), w.b[0:1].cpu(), w.grad[:rows].cpu(), torch.tensor([rows]))
    run(*cal)
    per_row = run(*cal) / rows
    total_rows = int(sizes.sum())
    est_pass = per_row * total_rows
    if est_pass <= budget_s:
        experts, reps_planned = sizes.numel(), 1
    else:
        cum = torch.cumsum(sizes, 0) * per_row
        experts, reps_planned = max(1, int((cum <= budget_s).sum())), 1
    n_rows = int(sizes[:experts].sum())
    a, b, g = w.a[:n_rows].cpu(), w.b[:experts].cpu(), w.grad[:n_rows].cpu()
    bs = sizes[:experts].clone()
    # whole passes until about 10 s of CPU work are on the clock (at most 20)
    t, reps = 0.0, 0
    while reps < max(1, reps_planned) or (t < 10.0 and reps < 20 and experts == sizes.numel()):
        t += run(a, b, g, bs)
        reps += 1
    flops = 3 * 2 * n_rows * hin * hout * reps
    what = "all" if experts == sizes.numel() else f"the first {experts} of {sizes.numel()}"
    return {"value": round(flops / t / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{reps} pass(es) over {what} experts ({n_rows} rows) at the real K={hin}, N={hout}: "
                      f"forward + input gradient + weight gradient through the oracle's per-expert loop "
                      f"(torch CPU bf16 matmul, {cores} threads), {t:.1f} s"}


WORKLOAD_NAMES = {
    2: ("bf16 grouped-GEMM TFLOP/s, Mixtral-8x7B w1 shape fwd+bwd",
        "forward + input-gradient + weight-gradient grouped GEMMs"),
    3: ("bf16 grouped-GEMM TFLOP/s, ragged fine-grained MoE forward", "forward grouped GEMM"),
    4: ("bf16 grouped-GEMM TFLOP/s, weight gradient (trans_a) alone", "weight-gradient grouped GEMM"),
    5: ("bf16 grouped-GEMM TFLOP/s, DeepSeek-V3-style expert share fwd+bwd",
        "forward + input-gradient + weight-gradient grouped GEMMs (b stored transposed)"),
}


# After an idle period the device runs through a power-management transient: about 5 launches at a
# boosted clock, then up to 35 % slower than the steady state, which it reaches again after 20-25
# ms of continuous work.  A workload whose step takes a fraction of a millisecond would be timed
# inside that transient after a handful of warm-up steps, so warm-up goes on until the device has
# been busy this long (the default workload's 10 warm-up steps are 88 ms: nothing is added there).
WARMUP_BUSY_MS = 60.0


def run_workload(config, steps, warmup, accumulate=False, zeros=False, flags=0, only=None, min_timed_ms=0.0):
    """Times the grouped GEMMs of one configuration; returns (workload, names, layout, ms_per_step,
    per-launch samples in ms, steps timed, warm-up steps run).  At least `warmup` warm-up steps,
    more until the device has been busy for WARMUP_BUSY_MS; at least `steps` timed steps, more
    until they cover `min_timed_ms`."""
    import torch
    from grouped_gemm import backend
    from grouped_gemm_amd import workloads

    w = workloads.make(config, device="cuda")
    if zeros:
        w.a.zero_(), w.b.zero_(), w.grad.zero_()
    sizes_dev = w.batch_sizes.cuda()
    lhs, rhs = (w.grad, w.a) if w.trans_b else (w.a, w.grad)

    def gmm(a, b, trans_a=False, trans_b=False):
        if not flags:
            return backend.gmm(a, b, sizes_dev, trans_a=trans_a, trans_b=trans_b)
        c = backend._allocate_output(a, b, sizes_dev, trans_a, trans_b)
        backend.backend.gmm_with_flags(a, b, c, sizes_dev, trans_a, trans_b, flags)
        return c

    calls = {
        "fwd": lambda: gmm(w.a, w.b, trans_b=w.trans_b),
        "agrad": lambda: gmm(w.grad, w.b, trans_b=not w.trans_b),
        "bgrad": lambda: gmm(lhs, rhs, trans_a=True),
    }
    names = [n for n in ("fwd", "agrad", "bgrad") if n in (only or w.gemms)]
    if accumulate:
        main_grad = torch.zeros(w.batch_sizes.numel(), lhs.shape[1], rhs.shape[1], device="cuda")
        calls["bgrad"] = lambda: backend.accumulate_weight_gradient(lhs, rhs, sizes_dev, main_grad)
        names = ["bgrad"]
    layout = {"fwd": "NT" if w.trans_b else "NN", "agrad": "NN" if w.trans_b else "NT",
              "bgrad": "TN, fp32 +=" if accumulate else "TN"}

    def step(events=None):
        for n in names:
            if events is not None:
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
                calls[n]()
                e1.record()
                events[n].append((e0, e1))
            else:
                calls[n]()

    # (the first step also loads the kernels: the step time is taken from the steps after it)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    for i in range(warmup):
        step()
        if i == 0:
            marks[0].record()
    if warmup < 2:
        step()
        warmup += 1
    marks[1].record()
    torch.cuda.synchronize()
    step_ms = max(marks[0].elapsed_time(marks[1]) / (warmup - 1), 1e-3)
    if step_ms * warmup < WARMUP_BUSY_MS:
        extra = min(int((WARMUP_BUSY_MS - step_ms * warmup) / step_ms) + 1, 2000)
        for _ in range(extra):
            step()
        torch.cuda.synchronize()
        warmup += extra
    steps = max(steps, min(int(min_timed_ms / step_ms) + 1, 500))
    events = {n: [] for n in names}
    t0 = time.perf_counter()
    for _ in range(steps):
        step(events)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    samples = {n: sorted(a.elapsed_time(b) for a, b in ev) for n, ev in events.items()}
    return w, names, layout, ms_per_step, samples, steps, warmup


def summarize(w, names, layout, ms_per_step, samples, accumulate=False):
    """value, roofline object and per-kernel table of one timed workload."""
    flops_gemm = w.flops_per_gemm()
    bytes_gemm = w.bytes_per_gemm()
    if accumulate:   # the fp32 output is read and written: 8 bytes per element instead of 2
        bytes_gemm += 6 * w.batch_sizes.numel() * w.hidden_in * w.hidden_out
    value = flops_gemm * len(names) / (ms_per_step * 1e-3) / 1e12
    kernel_ms = {n: sum(v) / len(v) for n, v in samples.items()}
    slowest = max(kernel_ms, key=kernel_ms.get)
    # which roof bounds the workload: arithmetic intensity against the ridge of the two peaks
    hbm_bound = flops_gemm / bytes_gemm < PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBPS * 1e9)
    if hbm_bound:
        achieved, peak, unit = bytes_gemm / (kernel_ms[slowest] * 1e-3) / 1e9, PEAK_HBM_GBPS, "GB/s"
    else:
        achieved, peak, unit = flops_gemm / (kernel_ms[slowest] * 1e-3) / 1e12, PEAK_BF16_TFLOPS, "TFLOP/s"
    roofline = {
        "bound": "hbm" if hbm_bound else "mfma",
        "kernel": f"gmm_kernel {layout[slowest]} ({slowest})",
        "achieved": round(achieved, 2),
        "peak": peak,
        "unit": unit,
        "frac": round(achieved / peak, 4),
        "algorithmic_bytes": bytes_gemm,
        "launch_ms": round(kernel_ms[slowest], 4),
        "flops_per_launch": flops_gemm,
        "per_kernel": {
            f"{layout[n]} ({n})": {
                "ms": round(ms, 4),
                "median_ms": round(samples[n][len(samples[n]) // 2], 4),
                "min_ms": round(samples[n][0], 4),
                "TFLOP/s": round(flops_gemm / (ms * 1e-3) / 1e12, 2),
                "frac_mfma": round(flops_gemm / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
                "GB/s": round(bytes_gemm / (ms * 1e-3) / 1e9, 1),
                "frac_hbm": round(bytes_gemm / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
            } for n, ms in kernel_ms.items()},
    }
    return value, roofline, slowest, kernel_ms


def other_paths(steps=7, warmup=4):
    """The paths past the reference's surface, timed shortly on the forward GEMM of the default
    workload (8 experts, 32768 rows, 4096 x 14336): fused row gather and scatter, the SwiGLU
    epilogue (the same b read as gate | up, so half the output width), float16, fp8 (e4m3, b as
    stored and b stored transposed, and the weight gradient), and hidden sizes that are not
    multiples of 8 (odd ones through zero-padded copies and on the general kernels, even ones
    as they are)."""
    import torch
    from grouped_gemm import backend
    from grouped_gemm_amd import workloads

    w = workloads.make(2, device="cuda")
    sd = w.batch_sizes.cuda()
    t, flops = w.tokens, w.flops_per_gemm()
    perm = torch.randperm(t, device="cuda").to(torch.int32)
    out = torch.empty(t, w.hidden_out, dtype=torch.bfloat16, device="cuda")

    def timed(fn, reps=steps, f=flops):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        return {"ms": round(ms, 4), "TFLOP/s": round(f / (ms * 1e-3) / 1e12, 1)}

    res = {
        "gather fused (gmm_indexed a_rows)": timed(lambda: backend.gmm_indexed(w.a, w.b, sd, a_rows=perm, c=out)),
        "scatter fused (gmm_indexed c_rows)": timed(lambda: backend.gmm_indexed(w.a, w.b, sd, c=out, c_rows=perm)),
        "swiglu epilogue (gmm_swiglu)": timed(lambda: backend.gmm_swiglu(w.a, w.b, sd)),
    }
    a16, b16 = w.a.half(), w.b.half()
    res["float16"] = timed(lambda: backend.gmm(a16, b16, sd, c=out.view(torch.float16)))
    del a16, b16
    a8, b8 = w.a.to(torch.float8_e4m3fn), w.b.transpose(1, 2).contiguous().to(torch.float8_e4m3fn)
    res["float8_e4m3fn, b stored transposed"] = timed(lambda: backend.gmm(a8, b8, sd, trans_b=True, c=out))
    del b8
    b8 = w.b.to(torch.float8_e4m3fn)
    res["float8_e4m3fn"] = timed(lambda: backend.gmm(a8, b8, sd, c=out))
    del b8
    g8 = w.grad.to(torch.float8_e4m3fn)
    wgrad = torch.empty_like(w.b)
    res["float8_e4m3fn, weight gradient (trans_a)"] = timed(lambda: backend.gmm(a8, g8, sd, trans_a=True, c=wgrad))
    for key in ("float8_e4m3fn, b stored transposed", "float8_e4m3fn", "float8_e4m3fn, weight gradient (trans_a)"):
        res[key]["frac_of_fp8_mfma_peak"] = round(res[key]["TFLOP/s"] / (2 * PEAK_BF16_TFLOPS), 4)
    del a8, g8, wgrad
    # odd hidden sizes: through zero-padded copies (what gmm does), and on the general kernels
    hin, hout = w.hidden_in - 3, w.hidden_out - 3
    au, bu = w.a[:, :hin].contiguous(), w.b[:, :hin, :hout].contiguous()
    res[f"hidden sizes {hin} x {hout} (zero-padded copies, streaming kernel)"] = timed(
        lambda: backend.gmm(au, bu, sd), reps=2, f=2 * t * hin * hout)
    cu = torch.empty(t, hout, dtype=torch.bfloat16, device="cuda")
    res[f"hidden sizes {hin} x {hout} (general kernels, the extension called directly)"] = timed(
        lambda: backend.backend.gmm(au, bu, cu, sd, False, False), reps=2, f=2 * t * hin * hout)
    del au, bu, cu
    # even hidden sizes that are no multiples of 8 stream as they are: the forward product and the
    # input gradient (whose rows run along the ragged hidden size) of such a layer
    hin, hout = w.hidden_in - 4, w.hidden_out - 4
    au, bu = w.a[:, :hin].contiguous(), w.b[:, :hin, :hout].contiguous()
    cu = torch.empty(t, hout, dtype=torch.bfloat16, device="cuda")
    res[f"hidden sizes {hin} x {hout} (streaming kernel, no copies)"] = timed(
        lambda: backend.gmm(au, bu, sd, c=cu), f=2 * t * hin * hout)
    gu = torch.empty(t, hin, dtype=torch.bfloat16, device="cuda")
    res[f"hidden sizes {hin} x {hout}, input gradient (streaming kernel, no copies)"] = timed(
        lambda: backend.gmm(cu, bu, sd, trans_b=True, c=gu), f=2 * t * hin * hout)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration (2 = Mixtral w1)")
    ap.add_argument("--only", default=None, help="time only these GEMMs of the configuration: a comma-separated "
                    "subset of fwd,agrad,bgrad (bgrad also for a configuration that lists only its forward GEMM)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short runs of the other configurations that the default run appends")
    ap.add_argument("--zeros", action="store_true",
                    help="diagnostic: all-zero inputs (no data toggling), to separate the power "
                         "limit from the kernel's cycle efficiency; not a valid benchmark result")
    ap.add_argument("--flags", type=int, default=0,
                    help="diagnostic: GG_FLAG_* scheduling switches of include/grouped_gemm_hip.h "
                         "(1 whole tiles, 2 one tile class, 4 row pieces); results are unchanged")
    ap.add_argument("--accumulate", action="store_true",
                    help="time only the weight gradient in its accumulating form: c (fp32) += a^T b "
                         "(backend.accumulate_weight_gradient) instead of the bf16 launch")
    ap.add_argument("--vendor-loop", action="store_true",
                    help="also time the reference's default algorithm on this GPU: one vendor GEMM "
                         "(torch.matmul) per expert with host-resident sizes, for the workload's "
                         "NN launch only (csrc/grouped_gemm.cu:396-413); adds a 'vendor_loop' object")
    ap.add_argument("--copy-bytes", type=int, default=0,
                    help="only run a plain device copy of this many bytes, 5 times (a known "
                         "traffic to scale the FETCH_SIZE / WRITE_SIZE counters by)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; expert-parallel sharding across GPUs "
                 "needs no exchange inside this operator and is left to the caller. Use --gpus 1.")

    import torch

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    if args.copy_bytes:
        src = torch.ones(args.copy_bytes, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copied_bytes": args.copy_bytes, "times": 5}))
        return
    only = tuple(args.only.split(",")) if args.only else None
    w, names, layout, ms_per_step, samples, _, warmup_run = run_workload(args.config, args.steps, args.warmup,
                                                                         args.accumulate, args.zeros, args.flags, only)
    value, roofline, slowest, kernel_ms = summarize(w, names, layout, ms_per_step, samples, args.accumulate)
    flops_gemm = w.flops_per_gemm()
    traffic = MEASURED_TRAFFIC.get(args.config, {}).get(slowest) if not (args.zeros or args.accumulate or args.flags or only) else None
    sources_now = kernel_sources_sha16()
    if traffic and sources_now != _TRAFFIC_KERNEL_SHA16:
        # the kernel sources have changed since the counters were read: no figure rather than a stale one
        roofline["traffic"] = None
        roofline["traffic_source"] = (f"not reported: the kernel sources (sha16 {sources_now}) are not the revision the "
                                      f"counters were read on ({_TRAFFIC_KERNEL_SHA16})")
    else:
        roofline["traffic"] = round(traffic["bytes"]) if traffic else None
        roofline["traffic_source"] = traffic["source"] if traffic else None
    metric, what = WORKLOAD_NAMES[args.config]
    if args.accumulate:
        metric, what = ("bf16 grouped-GEMM TFLOP/s, weight gradient accumulated into fp32",
                        "weight-gradient grouped GEMM added to an fp32 output")

    out = {
        "metric": metric,
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": warmup_run,   # args.warmup, or more for a short step (see WARMUP_BUSY_MS)
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "zeros (diagnostic, not a benchmark result)" if args.zeros else "synthetic",
        "config": {
            "workload": f"configs[{args.config - 1}]: {w.batch_sizes.numel()} experts, {w.tokens} routed rows, "
                        f"{w.hidden_in}x{w.hidden_out}, " + (what if not only else "only: " + ", ".join(names)),
            "batch_sizes": w.batch_sizes.tolist() if w.batch_sizes.numel() <= 16 else "see workloads.make",
            "batch_sizes_on_device": True,
        },
        "frac_of_bf16_mfma_peak": round(value / PEAK_BF16_TFLOPS, 4),
        "roofline": roofline,
    }
    if args.flags:
        out["config"]["diagnostic_flags"] = args.flags
    # What the chip sustains on the matrix instruction alone (operands in registers, no memory
    # traffic), right after the timed region: on operands with the bit statistics of this data the
    # power limit lowers the clock, on zeros it does not.  The first figure is the ceiling of any
    # bf16 GEMM on this device and data.  (A helper of this file, not of the library.)
    pipe_random = mfma_rate(False, 10)
    pipe_zeros = mfma_rate(True, 10)
    out["matrix_pipe_alone"] = {
        "what": "v_mfma_f32_32x32x16_bf16 on register operands, 256 workgroups of 4 waves, 10 launches of about 2.5 ms",
        "random_operands_TFLOP/s": round(pipe_random, 1),
        "zero_operands_TFLOP/s": round(pipe_zeros, 1),
        "random_operands_frac_of_peak": round(pipe_random / PEAK_BF16_TFLOPS, 4),
        "value_over_random_operands_rate": round(value / pipe_random, 4),
    }
    if args.vendor_loop:
        # the NN launch of this workload: forward, or the input gradient when b is stored transposed
        which = "agrad" if w.trans_b else "fwd"
        lhs_nn = w.grad if w.trans_b else w.a
        sizes_host = w.batch_sizes.tolist()
        res = torch.empty(lhs_nn.shape[0], w.b.shape[2], dtype=torch.bfloat16, device="cuda")

        def loop():
            start = 0
            for e, m in enumerate(sizes_host):
                if m:
                    torch.matmul(lhs_nn[start:start + m], w.b[e], out=res[start:start + m])
                start += m

        for _ in range(3):
            loop()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = max(3, min(args.steps, 20))
        e0.record()
        for _ in range(reps):
            loop()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        out["vendor_loop"] = {"launch": f"NN ({which})", "experts": len(sizes_host), "ms": round(ms, 4),
                              "TFLOP/s": round(flops_gemm / (ms * 1e-3) / 1e12, 2),
                              "this_library_ms": round(kernel_ms[which], 4),
                              "speedup": round(ms / kernel_ms[which], 3)}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w)
    # The other measured configurations, shortly, so that one default run shows all of them.
    default_run = not (args.no_other_configs or args.zeros or args.flags or args.accumulate or args.vendor_loop or only)
    if default_run and args.config == 2:
        del w
        others = {}
        # (configs[2] is a forward GEMM; its weight gradient, with Zipf depths and empty groups, is
        # timed beside it as the ragged case of the trans_a layout)
        for cfg, acc, only in ((3, False, None), (3, False, ("bgrad",)), (4, False, None), (4, True, None),
                               (5, False, None)):
            torch.cuda.empty_cache()
            res = run_workload(cfg, min(args.steps, 10), min(args.warmup, 3), accumulate=acc, only=only,
                               min_timed_ms=30.0)
            v, roof, _, _ = summarize(*res[:5], accumulate=acc)
            others[f"configs[{cfg - 1}]" + (" accumulate" if acc else "") + (" weight gradient" if only else "")] = {
                "workload": ("weight-gradient grouped GEMM of the same workload" if only else
                             WORKLOAD_NAMES[cfg][1] if not acc else "weight gradient added to an fp32 output"),
                "experts": res[0].batch_sizes.numel(), "rows": res[0].tokens,
                "hidden": f"{res[0].hidden_in}x{res[0].hidden_out}", "steps": res[5], "warmup": res[6],
                "ms_per_step": round(res[3], 4), "TFLOP/s": round(v, 2),
                "bound": roof["bound"], "achieved": roof["achieved"], "unit": roof["unit"], "frac": roof["frac"],
                "slowest_kernel": roof["kernel"],
                "per_kernel_ms": {k: d["ms"] for k, d in roof["per_kernel"].items()},
            }
            del res
        out["other_configs"] = others
        torch.cuda.empty_cache()
        out["other_paths"] = other_paths()
    print(json.dumps(out))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the MXFP hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--skip-hbm]

One step = one mxfp_linear(..., layer_type="XqWqB", backend="fused") call on the headline shape: x [16384, 4096] bf16
~N(0,1), W [14336, 4096] bf16 ~N(0,0.02) held as MXFP8 E4M3 components (block 32 along K), activations quantised to
MXFP8 E4M3 on the fly, bf16 output, fp32 accumulation.  At this shape "fused" is three kernels: x quantised straight
into FP8 bytes + E8M0 scales, the weight components brought into the same form (inside the call: a functional call
has nowhere to keep it; a layer builds it once), and the GEMM on the block-scaled FP8 matrix instruction.  Inputs are
resident in HBM before the timed region.  The same run also times the bf16-MFMA kernel family on the same shape, the
SwiGLU block of configuration C5, the bandwidth-bound cast kernels on their own configurations ("hbm_kernels") and the
reference's CPU path (tensor-op restatement under oracle/) on bounded samples.

Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "mase-triton_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
MFMA_FP8_PEAK_TFLOPS = 5000.0   # MI355X dense fp8, published
# HBM-side bytes per launch (roofline.traffic) are not measured by this run: they come from the committed summary of two
# rocprofv3 --pmc runs of `bench.py --counter-probe` (FETCH_SIZE, then WRITE_SIZE), written by
# `bench.py --summarize-counters`.  Every entry carries a fingerprint of the kernel sources it was taken with; when the
# sources have changed since, the figure is reported as null (with a note on stderr) instead of a stale number.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "hbm_counters_gemm_c4_c5_casts_c1_c2_c3.md")
CSRC = os.path.join(ROOT, "mase-triton_amd", "csrc")
GEMM_SOURCES = ("gemm_tall.h", "gemm_impl.h", "mxfp_compose.h", "mase_device.h")
SCALED_SOURCES = ("gemm_scaled.h", "gemm_tall.h", "mase_device.h")
CAST_SOURCES = ("cast_kernels.hip", "swiglu.h", "mxfp_compose.h", "mase_device.h")
ROWS_SOURCES = ("gemm_scaled_rows.h", "mase_device.h")


def sources_fingerprint(names) -> str:
    import hashlib

    h = hashlib.sha256()
    for n in names:
        with open(os.path.join(CSRC, n), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


_traffic_table = None


def traffic_bytes(key: str, sources):
    """HBM bytes per launch of kernel/workload `key` from the committed counter summary, or None."""
    global _traffic_table
    if _traffic_table is None:
        _traffic_table = {}
        try:
            text = open(TRAFFIC_SUMMARY).read()
            block = text[text.index("```json") + 7:]
            _traffic_table = json.loads(block[:block.index("```")])
        except (OSError, ValueError) as exc:
            print(f"bench.py: no usable counter summary at {TRAFFIC_SUMMARY} ({exc}): traffic reported as null", file=sys.stderr)
    row = _traffic_table.get(key)
    if row is None:
        return None
    if row.get("sources") != sources_fingerprint(sources):
        print(f"bench.py: the kernel sources behind '{key}' changed after {os.path.basename(TRAFFIC_SUMMARY)} was taken: "
              "traffic reported as null until the counters are collected again", file=sys.stderr)
        return None
    return int(row["traffic_bytes"])


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--skip-hbm", action="store_true", help="skip the cast-kernel bandwidth section")
    ap.add_argument("--only-gemm-kernel", choices=("scaled", "bf16", "bf16-components"), default=None,
                    help="profiling aid: launch only that GEMM kernel (block-scaled FP8; bf16 MFMA on the prepared weight; bf16 MFMA on "
                         "the weight components) on the headline shape, --steps times after --warmup, and print nothing")
    ap.add_argument("--rows", type=int, default=0, help="with --only-gemm-kernel: the first ROWS rows of C4's x instead of all 16384")
    ap.add_argument("--summarize-sq", metavar="COUNTER_CSV",
                    help="no GPU needed: per-kernel table (stdout, markdown) from the counter_collection.csv of a rocprofv3 --pmc run with "
                         "SQ_BUSY_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU SQ_INSTS_LDS SQ_WAIT_ANY SQ_WAVE_CYCLES SQ_WAVES [SQ_LDS_BANK_CONFLICT]")
    ap.add_argument("--summarize-trace", metavar="KERNEL_TRACE_CSV",
                    help="no GPU needed: per-kernel durations (stdout, markdown) from the kernel_trace.csv of a rocprofv3 --kernel-trace run")
    ap.add_argument("--counter-probe", action="store_true",
                    help="profiling aid for rocprofv3 --pmc: a plain 256 MiB device copy (calibration), then 3 launches "
                         "each of the GEMM and of the C3 extract / compose kernels; prints nothing to time")
    ap.add_argument("--summarize-counters", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="no GPU needed: turn the output folders of two `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs of "
                         "`bench.py --counter-probe` into the markdown summary kept under profiles/ (stdout)")
    ap.add_argument("--shape-sweep", action="store_true",
                    help="context run, not the metric: mxfp_linear fused vs separate over M at N=14336, K=4096, and the "
                         "in-place casts along a non-last axis against the permuted-copy route; prints its own JSON line")
    return ap.parse_args()


def event_ms(pairs):
    return [a.elapsed_time(b) for a, b in pairs]


def settle(torch, fn, group=5, tol=0.01, most=100):
    """Run fn in groups until the time per call stops changing; returns what the first and the last group took."""
    first = prev = ms = None
    done = 0
    while done < most:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(group):
            fn()
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_time(e1) / group
        done += group
        if first is None:
            first = ms
        elif done >= 3 * group and abs(ms - prev) <= tol * prev:
            break
        prev = ms
    return {"steps": done, "first_group_ms_per_step": round(first, 4), "settled_ms_per_step": round(ms, 4)}


def timed_loop(torch, fn, steps, warmup):
    """ms per call: `steps` calls between two device synchronisations, after `warmup` uncounted ones."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def bench_linear(args, torch, MXFP_F, kernels, fmt):
    import workloads
    from mase_hip.mxfp.functional import linear as L

    dev = "cuda:0"
    x_cpu, w_cpu = workloads.make_c4()          # the very tensors of the parity test (CPU generator, seeds 3 and 4)
    M, K = x_cpu.shape
    N = w_cpu.shape[0]
    x, w = x_cpu.to(dev), w_cpu.to(dev)
    del x_cpu, w_cpu
    w_sc, w_el, w_tm = MXFP_F.extract_mxfp_components(w, block_dim=1, mxfp_meta=fmt)
    del w
    call = dict(x=x, x_meta=fmt, w=None, w_scales=w_sc, w_elements=w_el, w_tensor_meta=w_tm, b=None, b_scales=None,
                b_elements=None, b_tensor_meta=None, layer_type="XqWqB")
    flop = 2.0 * M * N * K

    def step(ev=None):
        # the three kernels of MXFP_F.mxfp_linear(**call, backend="fused") at this shape, split so that events can
        # bracket the GEMM
        a_op = kernels.scaled_operand_from_dense(x, fmt)
        w_op = L.scaled_weight_operand(w_sc, w_el, w_tm)
        if ev is not None:
            ev[0].record()
        y = kernels.mxfp_gemm_scaled(a_op, w_op, None, torch.bfloat16)
        if ev is not None:
            ev[1].record()
        return y

    def step_bf16(ev=None):
        # backend="fused_bf16": single-pass QDQ of x to bf16, then the GEMM that composes W to bf16 in registers
        a = kernels.quantize_dequantize(x.view(-1), fmt, torch.bfloat16).view(M, K)
        if ev is not None:
            ev[0].record()
        y = kernels.mxfp_gemm(a, None, None, None, w_sc, w_el, fmt, None, M, N, K, torch.bfloat16)
        if ev is not None:
            ev[1].record()
        return y

    def step_bf16_kept(ev=None):
        # the same with the weight operand a layer keeps: the 512 x 128 kernel reads the prepared form
        a = kernels.quantize_dequantize(x.view(-1), fmt, torch.bfloat16).view(M, K)
        if ev is not None:
            ev[0].record()
        y = kernels.mxfp_gemm_prepared_w(a, w_kept, None, torch.bfloat16)
        if ev is not None:
            ev[1].record()
        return y

    w_kept = L.scaled_weight_operand(w_sc, w_el, w_tm)      # what a layer keeps
    if args.only_gemm_kernel:
        if args.rows:
            M = args.rows
            x = x[:M].contiguous()
        a_op = kernels.scaled_operand_from_dense(x, fmt)
        a = kernels.quantize_dequantize(x.view(-1), fmt, torch.bfloat16).view(M, K)
        fn = ((lambda: kernels.mxfp_gemm_scaled(a_op, w_kept, None, torch.bfloat16)) if args.only_gemm_kernel == "scaled" else
              (lambda: kernels.mxfp_gemm_prepared_w(a, w_kept, None, torch.bfloat16)) if args.only_gemm_kernel == "bf16" else
              (lambda: kernels.mxfp_gemm(a, None, None, None, w_sc, w_el, fmt, None, M, N, K, torch.bfloat16)))
        timed_loop(torch, fn, args.steps, args.warmup)
        return None

    y_api = MXFP_F.mxfp_linear(**call, backend="fused")
    assert torch.equal(step().view(torch.int16), y_api.view(torch.int16)), "bench step differs from mxfp_linear(backend='fused')"
    assert torch.equal(step_bf16().view(torch.int16), MXFP_F.mxfp_linear(**call, backend="fused_bf16").view(torch.int16))
    assert torch.equal(step_bf16_kept().view(torch.int16), MXFP_F.mxfp_linear(**call, backend="fused_bf16", w_operand=w_kept).view(torch.int16))
    del y_api
    # The shader clock settles over the first few dozen launches after idle (the step gets faster), so a short counted
    # warm-up would time the ramp.  Before the counted warm-up: steps in groups of five until two consecutive groups agree
    # within 1 %, at most 100 steps.  Both figures are reported.
    prewarm = settle(torch, step)

    def measure(step_fn):
        for _ in range(args.warmup):
            step_fn()
        torch.cuda.synchronize()
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        t0 = time.perf_counter()
        for i in range(args.steps):
            step_fn(pairs[i])
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        return ms, sum(event_ms(pairs)) / args.steps

    ms_per_step, gemm_ms = measure(step)
    settle(torch, step_bf16_kept)
    bf16_ms, bf16_gemm_ms = measure(step_bf16_kept)
    bf16c_ms, bf16c_gemm_ms = measure(step_bf16)
    # context, not the metric
    half = max(3, args.warmup // 2)
    prepared_ms = timed_loop(torch, lambda: MXFP_F.mxfp_linear(**call, backend="fused", w_operand=w_kept), args.steps, half)
    # backend="separate": extract x, compose x, compose W to bf16 in HBM, the vendor library's dense bf16 GEMM
    sep_ms = timed_loop(torch, lambda: MXFP_F.mxfp_linear(**call, backend="separate"), args.steps, half)
    a_dq = kernels.quantize_dequantize(x.view(-1), fmt, torch.bfloat16).view(M, K)
    w_dq = kernels.compose_mxfp_tensor(w_sc, w_el, fmt, torch.bfloat16).view(N, K)
    dense_ms = timed_loop(torch, lambda: torch.nn.functional.linear(a_dq, w_dq), args.steps, 5)
    del a_dq, w_dq
    tf = lambda ms: flop / (ms * 1e-3) / 1e12
    return {
        "prewarm": prewarm, "shape": (M, N, K), "flop": flop,
        "ms_per_step": ms_per_step, "tflops_step": tf(ms_per_step), "gemm_ms": gemm_ms, "tflops_gemm": tf(gemm_ms),
        "bf16_ms_per_step": bf16_ms, "bf16_tflops_step": tf(bf16_ms), "bf16_gemm_ms": bf16_gemm_ms, "bf16_tflops_gemm": tf(bf16_gemm_ms),
        "bf16c_ms_per_step": bf16c_ms, "bf16c_gemm_ms": bf16c_gemm_ms, "bf16c_tflops_gemm": tf(bf16c_gemm_ms),
        "prepared_ms": prepared_ms, "separate_ms": sep_ms, "dense_ms": dense_ms,
    }


def time_kernel(torch, launch, n_variants, iters=48, warmup=8, reps=5):
    """Average duration of one launch: `iters` back-to-back launches, rotating through n_variants
    independent buffer sets so that consecutive launches do not hit the same lines, are captured in
    a HIP graph (removes the host's launch cost from the GPU timeline) and the replay is bracketed
    by HIP events on the launch stream.  Returns (mean over replays, best replay) per launch in ms."""
    for i in range(warmup):
        launch(i % n_variants)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        launch(0)
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(iters):
                launch(i % n_variants)
        times = []
        for _ in range(reps + 1):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            graph.replay()
            e1.record(stream)
            e1.synchronize()
            times.append(e0.elapsed_time(e1) / iters)
    stream.synchronize()
    times = times[1:]
    return sum(times) / len(times), min(times)


def load_bench_lib():
    """lib/libmase_bench.so: the tuned streaming copy used as the yardstick of the bandwidth-bound kernels."""
    import ctypes

    path = os.path.join(ROOT, "mase-triton_amd", "mase_hip", "lib", "libmase_bench.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `python mase-triton_amd/build.py`")
    lib = ctypes.CDLL(path)
    lib.mase_bench_stream_copy.restype = ctypes.c_int
    lib.mase_bench_stream_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    return lib


def cpu_cast_baselines(torch):
    """The reference's CPU path for the casts (tensor-op restatement under oracle/), on bounded samples of the same
    workloads; GB/s by the same algorithmic bytes per element as the GPU rows.  Keyed by (kernel, config)."""
    from oracle import torch_fake
    import workloads

    threads = torch.get_num_threads()
    out = {}

    def timed(fn):
        fn()                      # first call pays for allocator growth
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    def entry(nbytes, dt, sample):
        return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port", "sample": f"{sample}, {dt:.2f} s"}

    for tag, full, rows, (e, m) in (("C1", workloads.make_c1, 2048, (4, 3)), ("C3", workloads.make_c3, 2048, (2, 1))):
        x = full(rows, 4096).reshape(-1)
        n = x.numel()
        sc, el = torch_fake.mxfp_split(x, 32, e, m)
        sample = f"{rows} rows of {tag}"
        t_ext = timed(lambda: torch_fake.mxfp_split(x, 32, e, m))
        t_cmp = timed(lambda: torch_fake.mxfp_join(sc, el, e, m, True, torch.bfloat16))
        out[("extract_mxfp", tag)] = entry(n * (3 + 1 / 32), t_ext, sample)
        out[("compose_mxfp", tag)] = entry(n * (3 + 1 / 32), t_cmp, sample)
        out[("extract+compose_mxfp", tag)] = entry(n * (6 + 1 / 16), t_ext + t_cmp, sample)
        out[("qdq_mxfp_fused", tag)] = entry(n * 4.0, t_ext + t_cmp, sample + " (extract then compose)")
    x = workloads.make_c2(1 << 22)
    n = x.numel()
    for e, m in ((4, 3), (5, 2)):
        codes = torch_fake.minifloat_encode(x, e, m)
        sample = "2^22 of C2"
        t_ext = timed(lambda: torch_fake.minifloat_encode(x, e, m))
        t_cmp = timed(lambda: torch_fake.minifloat_decode(codes, e, m, True, torch.float32))
        tag = f"C2/E{e}M{m}"
        out[("extract_minifloat", tag)] = entry(n * 6.0, t_ext, sample)
        out[("compose_minifloat", tag)] = entry(n * 6.0, t_cmp, sample)
        out[("qdq_minifloat_fused", tag)] = entry(n * 8.0, t_ext + t_cmp, sample + " (encode then decode)")
    return out


def bench_hbm(torch, with_cpu):
    """Cast kernels on their own configurations, on the configurations' own value distributions (tests/workloads.py: C3 with
    its all-zero blocks and planted inf / NaN, C2 with its outliers, zeros and subnormals).  Algorithmic bytes per element:
    MXFP extract from bf16 2 + 1 + 1/32, compose to bf16 1 + 1/32 + 2, fused minifloat QDQ fp32 -> fp32 4 + 4."""
    import workloads
    from mase_hip import _lib

    dev = "cuda:0"
    out = []
    copy_cache = {}
    lib = _lib.load()
    blib = load_bench_lib()
    sp_of = lambda: _lib.stream_ptr(torch.device(dev))
    cpu = cpu_cast_baselines(torch) if with_cpu else {}

    def tuned_copy_gbps(nbytes):
        """The hand-tuned streaming copy (csrc/bench/stream_copy.hip) moving the same number of bytes, half read and half
        written, timed the same way; the better of its two launch shapes."""
        half = int(nbytes // 2) // 16 * 16
        if half not in copy_cache:
            k = max(2, (320 << 20) // (2 * half) + 1)
            src = [torch.empty(half, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(k)]
            dst = [torch.empty_like(t) for t in src]
            best = 0.0
            for form in (0, 1):
                def cp(i):
                    assert blib.mase_bench_stream_copy(src[i].data_ptr(), dst[i].data_ptr(), half, form, sp_of()) == 0
                avg, _ = time_kernel(torch, cp, k)
                best = max(best, 2 * half / (avg * 1e-3) / 1e9)
            assert torch.equal(src[0], dst[0])
            copy_cache[half] = round(best, 1)
        return copy_cache[half]

    def roof(name, cfg, workload, bytes_per_launch, avg_ms, best_ms, cached_ms, sources=CAST_SOURCES):
        gbs = bytes_per_launch / (avg_ms * 1e-3) / 1e9
        copy = tuned_copy_gbps(bytes_per_launch)
        out.append({
            "kernel": name, "workload": workload, "bytes_per_launch": bytes_per_launch,
            "avg_ms": round(avg_ms, 5), "best_ms": round(best_ms, 5),
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic_bytes(f"{name} {cfg}", sources)},
            "cache_resident_GBps": round(bytes_per_launch / (cached_ms * 1e-3) / 1e9, 1),
            "tuned_copy_same_bytes_GBps": copy, "frac_of_tuned_copy": round(gbs / copy, 3),
            "cpu_baseline": cpu.get((name, cfg)),
        })

    def mxfp_case(tag, x_cpu, e, m, copies):
        rows, cols = x_cpu.shape
        n = rows * cols
        x0 = x_cpu.reshape(-1).to(dev)
        xs = [x0] + [x0.clone() for _ in range(copies - 1)]      # the same values in rotating buffers
        sc0 = torch.empty(n // 32, dtype=torch.uint8, device=dev)
        el0 = torch.empty(n, dtype=torch.uint8, device=dev)
        _lib.check(lib.mase_hip_extract_mxfp(x0.data_ptr(), 2, sc0.data_ptr(), el0.data_ptr(), n, 32, e, m, 1, 0, sp_of()))
        comps = [(sc0, el0)] + [(sc0.clone(), el0.clone()) for _ in range(copies - 1)]
        ext_bytes = n * (2 + 1 + 1 / 32)
        cmp_bytes = n * (1 + 1 / 32 + 2)
        # pre-allocated outputs so that the timed region holds only the kernel
        sc_o = [torch.empty_like(c[0]) for c in comps]
        el_o = [torch.empty_like(c[1]) for c in comps]
        y_o = [torch.empty_like(x) for x in xs]

        def ext(i):
            _lib.check(lib.mase_hip_extract_mxfp(xs[i].data_ptr(), 2, sc_o[i].data_ptr(), el_o[i].data_ptr(), n, 32, e, m, 1, 0, sp_of()))

        def cmp(i):
            _lib.check(lib.mase_hip_compose_mxfp(comps[i][0].data_ptr(), comps[i][1].data_ptr(), y_o[i].data_ptr(), 2, n, 32, e, m, 1, sp_of()))

        def both(i):
            ext(i)
            cmp(i)

        def qdq(i):
            _lib.check(lib.mase_hip_qdq_mxfp(xs[i].data_ptr(), 2, y_o[i].data_ptr(), 2, n, 32, e, m, 1, 0, sp_of()))

        wl = f"{tag}: {rows}x{cols} bf16, E{e}M{m}, block 32"
        for name, fn, nbytes in (("extract_mxfp", ext, ext_bytes), ("compose_mxfp", cmp, cmp_bytes),
                                 ("extract+compose_mxfp", both, ext_bytes + cmp_bytes), ("qdq_mxfp_fused", qdq, n * 4.0)):
            avg, best = time_kernel(torch, fn, copies)
            cavg, _ = time_kernel(torch, lambda i: fn(0), 1)
            roof(name, tag, wl, nbytes, avg, best, cavg)
        assert torch.equal(sc_o[0], comps[0][0]) and torch.equal(el_o[0], comps[0][1])

    mxfp_case("C1", workloads.make_c1(), 4, 3, copies=12)   # 12 x (32 + 16.5) MiB in flight > 256 MiB cache
    mxfp_case("C3", workloads.make_c3(), 2, 1, copies=4)

    # C2: minifloat casts on 2^24 fp32
    n = 1 << 24
    x0 = workloads.make_c2().to(dev)
    xs = [x0] + [x0.clone() for _ in range(5)]
    ys = [torch.empty_like(x) for x in xs]
    cs = [torch.empty(n, dtype=torch.uint16, device=dev) for _ in xs]
    for e, m in ((4, 3), (5, 2)):
        def qdq(i):
            _lib.check(lib.mase_hip_qdq_minifloat(xs[i].data_ptr(), 0, ys[i].data_ptr(), 0, n, e, m, 1, 0, sp_of()))

        def ext(i):
            _lib.check(lib.mase_hip_extract_minifloat(xs[i].data_ptr(), 0, cs[i].data_ptr(), n, e, m, 1, 0, sp_of()))

        def cmp(i):
            _lib.check(lib.mase_hip_compose_minifloat(cs[i].data_ptr(), ys[i].data_ptr(), 0, n, e, m, 1, sp_of()))

        wl = f"C2: 2^24 fp32, FP8 E{e}M{m}"
        for i in range(len(xs)):
            ext(i)                # codes for the compose rows
        for name, fn, nbytes in (("qdq_minifloat_fused", qdq, n * 8.0), ("extract_minifloat", ext, n * 6.0),
                                 ("compose_minifloat", cmp, n * 6.0)):
            avg, best = time_kernel(torch, fn, len(xs))
            cavg, _ = time_kernel(torch, lambda i: fn(0), 1)
            roof(name, f"C2/E{e}M{m}", wl, nbytes, avg, best, cavg)
    del xs, ys, cs

    # Decode-sized mxfp_linear is a read of W: C4's weight against the first 16 rows of C4's x, both as the operands a layer
    # keeps / builds, on the block-scaled weight-streaming kernel; the weight rotates through seven copies (424 MB) so that
    # none of it is served from the 256 MB memory-side cache.  The bf16 weight-streaming kernel on the same data beside it.
    from mase_hip.mxfp import kernels
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn

    x_cpu, w_cpu = workloads.make_c4()
    N, K = w_cpu.shape
    x64 = x_cpu[:64].contiguous().to(dev)
    w_sc, w_el = kernels.extract_mxfp_components(w_cpu.to(dev).reshape(-1), MXFP8_E4M3_fn)
    del x_cpu, w_cpu
    comps = [(w_sc, w_el)] + [(w_sc.clone(), w_el.clone()) for _ in range(6)]
    wops = [kernels.scaled_operand_from_mxfp(sc, el, MXFP8_E4M3_fn, N, K) for sc, el in comps]
    w_bytes = N * K * (1 + 1 / 32)
    for rows in (16, 64):      # one and four operand tiles of x in the wavefronts' registers
        xr = x64[:rows].contiguous()
        a_op = kernels.scaled_operand_from_dense(xr, MXFP8_E4M3_fn)
        a_dq = kernels.quantize_dequantize(xr.view(-1), MXFP8_E4M3_fn, torch.bfloat16).view(rows, K)
        y = torch.empty(rows, N, dtype=torch.bfloat16, device=dev)

        def rows_gemm(i):
            kernels.mxfp_gemm_scaled(a_op, wops[i], None, torch.bfloat16, out=y)

        def rows_gemm_bf16(i):
            kernels.mxfp_gemm(a_dq, None, None, None, comps[i][0], comps[i][1], MXFP8_E4M3_fn, None, rows, N, K, torch.bfloat16, out=y)

        for name, fn in (("mxfp_gemm_scaled_rows", rows_gemm), ("mxfp_gemm_skinny (bf16)", rows_gemm_bf16)):
            avg, best = time_kernel(torch, fn, len(wops))
            cavg, _ = time_kernel(torch, lambda i: fn(0), 1)
            roof(name, f"C4 W x {rows} rows", f"decode: {rows} rows of C4's x against W [{N},{K}] MXFP8 E4M3, bf16 out (bytes = W's codes and scales)", w_bytes,
                 avg, best, cavg, ROWS_SOURCES if fn is rows_gemm else GEMM_SOURCES)
    return out


def cpu_baseline(torch):
    """The reference's CPU path (quantise x, dequantise x and W with tensor ops, then F.linear) on a
    bounded sample of the headline workload: the first `rows` of the 16384 activation rows against
    the full weight.  A probe with 512 rows sizes the sample to roughly 12 s of CPU work."""
    from oracle import torch_fake

    K, N, M = 4096, 14336, 16384
    g = torch.Generator().manual_seed(3)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    w_sc, w_el = torch_fake.mxfp_split(w, 32, 4, 3)
    del w
    threads = torch.get_num_threads()

    def run(rows):
        x = torch.randn(rows, K, generator=g).to(torch.bfloat16)
        t0 = time.perf_counter()
        y = torch_fake.mxfp_linear_xq_wq(x, w_sc, w_el, (N, K), torch.bfloat16, (4, 3), (4, 3))
        dt = time.perf_counter() - t0
        assert y.shape == (rows, N)
        return dt

    t_probe = run(512)
    rows = int(min(M, max(512, 512 * (12.0 / max(t_probe, 1e-3)))) // 256 * 256)
    dt = run(rows)
    flop = 2.0 * rows * N * K
    return {"value": round(flop / dt / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{rows} of {M} activation rows x full W [{N},{K}]: tensor-op restatement of the reference's CPU "
                      f"path (quantise x, dequantise x and W, F.linear), {dt:.1f} s"}


def shape_sweep(torch, MXFP_F, mxk, fmt, steps=30, warmup=15):
    """Host-timed (launch overhead included) context figures; every shape takes a different GEMM kernel."""
    from mase_hip.mxfp.helpers import flatten_for_quantize

    dev = "cuda:0"
    N, K = 14336, 4096
    gen = torch.Generator(device=dev).manual_seed(5)

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e6 / steps

    def linear_rows(n_out, k_in, Ms):
        from mase_hip.mxfp.functional import linear as L

        wt = (0.02 * torch.randn(n_out, k_in, generator=gen, device=dev)).to(torch.bfloat16)
        sc, el, tm = MXFP_F.extract_mxfp_components(wt, block_dim=1, mxfp_meta=fmt)
        w_op = L.scaled_weight_operand(sc, el, tm)
        out = []
        for M in Ms:
            x = torch.randn(M, k_in, generator=gen, device=dev).to(torch.bfloat16)
            call = dict(x=x, x_meta=fmt, w=None, w_scales=sc, w_elements=el, w_tensor_meta=tm, b=None, b_scales=None,
                        b_elements=None, b_tensor_meta=None, layer_type="XqWqB")
            b_us = timed(lambda: MXFP_F.mxfp_linear(**call, backend="fused_bf16"))
            s_us = timed(lambda: MXFP_F.mxfp_linear(**call, backend="fused_scaled"))
            p_us = timed(lambda: MXFP_F.mxfp_linear(**call, backend="fused_scaled", w_operand=w_op))
            f_us = timed(lambda: MXFP_F.mxfp_linear(**call, backend="fused"))
            sep_us = timed(lambda: MXFP_F.mxfp_linear(**call, backend="separate"))
            out.append({"M": M, "fused_us": round(f_us, 1), "fused_bf16_us": round(b_us, 1), "fused_scaled_us": round(s_us, 1),
                        "fused_scaled_kept_weight_us": round(p_us, 1), "separate_us": round(sep_us, 1),
                        "fused_TFLOPs": round(2.0 * M * n_out * k_in / f_us / 1e6, 1)})
        return out

    rows = linear_rows(N, K, (16, 32, 64, 128, 256, 384, 512, 768, 1024, 2048, 4096, 8192))
    rows_down = linear_rows(K, N, (16, 32, 64, 256, 512, 1024, 2048, 4096))  # the transposed layer shape: few W rows, long K
    rows_sq = linear_rows(K, K, (32, 128, 256, 512, 1024, 2048, 4096))
    w = (0.02 * torch.randn(N, K, generator=gen, device=dev)).to(torch.bfloat16)
    n = w.numel()
    cast = {
        "shape": [N, K], "block_axis": 0,
        "extract_in_place_us": round(timed(lambda: mxk.extract_mxfp_components_strided(w, 0, fmt)), 1),
        "extract_permuted_copy_us": round(timed(lambda: mxk.extract_mxfp_components(flatten_for_quantize(w, 0), fmt)), 1),
        "qdq_in_place_us": round(timed(lambda: mxk.quantize_dequantize_strided(w, 0, fmt, torch.bfloat16)), 1),
        "qdq_permuted_copy_us": round(timed(lambda: mxk.quantize_dequantize(flatten_for_quantize(w, 0), fmt, torch.bfloat16)), 1),
    }
    cast["extract_in_place_GBps"] = round(n * (3 + 1 / 32) / cast["extract_in_place_us"] / 1e3, 0)
    cast["qdq_in_place_GBps"] = round(n * 4 / cast["qdq_in_place_us"] / 1e3, 0)
    return {"linear_N14336_K4096": rows, "linear_N4096_K14336": rows_down, "linear_N4096_K4096": rows_sq, "casts_along_axis0": cast,
            "casts_over_size": casts_over_size(torch, fmt)}


def casts_over_size(torch, fmt):
    """The MXFP casts of configuration C1 (bf16, E4M3, block 32) and the tuned streaming copy at 1, 2, 4 and 8 times C1's
    16.8 M elements: kernel time per launch (HIP graph of 48 launches over rotating buffers, as in the benchmark), and a
    least-squares line  t = t0 + bytes / bandwidth  through the four points of each kernel.  t0 is what a launch costs
    whatever its size (ramp and tail); the slope is the rate the kernel sustains."""
    import workloads
    from mase_hip import _lib

    dev = "cuda:0"
    lib = _lib.load()
    blib = load_bench_lib()
    sp = lambda: _lib.stream_ptr(torch.device(dev))
    e, m = fmt.element_exp_bits, fmt.element_frac_bits
    base = workloads.make_c1().reshape(-1).to(dev)
    points = {k: [] for k in ("extract_mxfp", "compose_mxfp", "qdq_mxfp_fused", "tuned_copy (bytes of extract)")}
    for mult in (1, 2, 4, 8):
        x0 = base.repeat(mult)
        n = x0.numel()
        copies = max(2, int((400 << 20) // (3 * n)) + 1)
        xs = [x0] + [x0.clone() for _ in range(copies - 1)]
        scs = [torch.empty(n // 32, dtype=torch.uint8, device=dev) for _ in xs]
        els = [torch.empty(n, dtype=torch.uint8, device=dev) for _ in xs]
        ys = [torch.empty_like(x) for x in xs]

        def ext(i):
            _lib.check(lib.mase_hip_extract_mxfp(xs[i].data_ptr(), 2, scs[i].data_ptr(), els[i].data_ptr(), n, 32, e, m, 1, 0, sp()))

        def cmp(i):
            _lib.check(lib.mase_hip_compose_mxfp(scs[i].data_ptr(), els[i].data_ptr(), ys[i].data_ptr(), 2, n, 32, e, m, 1, sp()))

        def qdq(i):
            _lib.check(lib.mase_hip_qdq_mxfp(xs[i].data_ptr(), 2, ys[i].data_ptr(), 2, n, 32, e, m, 1, 0, sp()))

        half = int(n * (3 + 1 / 32) / 2) // 16 * 16
        src = [x.view(torch.uint8)[:half] for x in xs]
        dst = [y.view(torch.uint8)[:half] for y in ys]

        def cp(i):
            assert blib.mase_bench_stream_copy(src[i].data_ptr(), dst[i].data_ptr(), half, 1, sp()) == 0

        for i in range(copies):
            ext(i)
        for name, fn, nbytes in (("extract_mxfp", ext, n * (3 + 1 / 32)), ("compose_mxfp", cmp, n * (3 + 1 / 32)), ("qdq_mxfp_fused", qdq, n * 4.0),
                                 ("tuned_copy (bytes of extract)", cp, 2.0 * half)):
            avg, _ = time_kernel(torch, fn, copies)
            points[name].append({"elements": n, "bytes": int(nbytes), "us": round(avg * 1e3, 2), "GBps": round(nbytes / (avg * 1e-3) / 1e9, 0)})
        del xs, scs, els, ys, src, dst, x0
    out = {}
    for name, pts in points.items():
        bx, ty = [p["bytes"] for p in pts], [p["us"] for p in pts]
        k = len(pts)
        mx, my = sum(bx) / k, sum(ty) / k
        slope = sum((a - mx) * (b - my) for a, b in zip(bx, ty)) / sum((a - mx) ** 2 for a in bx)      # us per byte
        out[name] = {"points": pts, "fit": {"t0_us": round(my - slope * mx, 2), "sustained_GBps": round(1e-3 / slope, 0)}}
    return out


def counter_probe(torch, MXFP_F, mxk, fmt8, fmt4):
    """Three launches of each kernel next to a copy of known size, for hardware-counter runs (see --summarize-counters)."""
    import workloads
    from mase_hip import _lib
    from mase_hip.mxfp.functional import linear as L

    dev = "cuda:0"
    lib = _lib.load()
    blib = load_bench_lib()
    sp = _lib.stream_ptr(torch.device(dev))
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):                                      # calibration: reads 256 MiB, writes 256 MiB
        assert blib.mase_bench_stream_copy(src.data_ptr(), dst.data_ptr(), src.numel(), 1, sp) == 0
    del src, dst
    x_cpu, w_cpu = workloads.make_c4()
    M, K = x_cpu.shape
    N = w_cpu.shape[0]
    x, w = x_cpu.to(dev), w_cpu.to(dev)
    w_sc, w_el, w_tm = MXFP_F.extract_mxfp_components(w, block_dim=1, mxfp_meta=fmt8)
    a = mxk.quantize_dequantize(x.view(-1), fmt8, torch.bfloat16).view(M, K)
    for _ in range(3):
        mxk.mxfp_gemm(a, None, None, None, w_sc, w_el, fmt8, None, M, N, K, torch.bfloat16)
    for _ in range(3):
        a_op = mxk.scaled_operand_from_dense(x, fmt8)
        w_op = L.scaled_weight_operand(w_sc, w_el, w_tm)
        mxk.mxfp_gemm_scaled(a_op, w_op, None, torch.bfloat16)
    a16, a64 = mxk.scaled_operand_from_dense(x[:16].contiguous(), fmt8), mxk.scaled_operand_from_dense(x[:64].contiguous(), fmt8)
    for _ in range(3):
        mxk.mxfp_gemm_scaled(a16, w_op, None, torch.bfloat16)          # decode-sized: the weight-streaming kernels
        mxk.mxfp_gemm_scaled(a64, w_op, None, torch.bfloat16)
    del x, w, w_sc, w_el, a, a_op, w_op, a16, a64
    # C5's kernels on the block-scaled route: gate + up GEMM, SwiGLU operand, down GEMM (after C4's launches of the same kernels)
    from mase_hip.mxfp.meta import MXFPMeta

    x5, wg, wu, wd = workloads.make_c5()
    fmt6 = MXFPMeta(32, 8, 3, 2, True, "rn")
    inter = wg.shape[0]
    x5 = x5.to(dev).view(-1, x5.shape[-1])
    ops = []
    for w5 in (torch.cat([wg, wu]), wd):
        sc5, el5, tm5 = MXFP_F.extract_mxfp_components(w5.to(dev), block_dim=1, mxfp_meta=fmt6)
        ops.append(L.scaled_weight_operand(sc5, el5, tm5))
        del sc5, el5
    for _ in range(3):
        t5 = mxk.mxfp_gemm_scaled(mxk.scaled_operand_from_dense(x5, fmt8), ops[0], None, torch.bfloat16)
    for _ in range(3):
        a5 = mxk.scaled_operand_from_swiglu(t5[:, :inter], t5[:, inter:], fmt8)
    for _ in range(3):
        mxk.mxfp_gemm_scaled(a5, ops[1], None, torch.bfloat16)
    del x5, t5, a5, ops
    for make, fmt in ((workloads.make_c1, fmt8), (workloads.make_c3, fmt4)):
        t = make().reshape(-1).to(dev)
        for _ in range(3):
            sc, el = mxk.extract_mxfp_components(t, fmt)
            mxk.compose_mxfp_tensor(sc, el, fmt, torch.bfloat16)
            mxk.quantize_dequantize(t, fmt, torch.bfloat16)
        del t
    x2 = workloads.make_c2().to(dev)
    y2 = torch.empty_like(x2)
    c2 = torch.empty(x2.numel(), dtype=torch.uint16, device=dev)
    for e, m in ((4, 3), (5, 2)):
        for _ in range(3):
            _lib.check(lib.mase_hip_qdq_minifloat(x2.data_ptr(), 0, y2.data_ptr(), 0, x2.numel(), e, m, 1, 0, sp))
            _lib.check(lib.mase_hip_extract_minifloat(x2.data_ptr(), 0, c2.data_ptr(), x2.numel(), e, m, 1, 0, sp))
            _lib.check(lib.mase_hip_compose_minifloat(c2.data_ptr(), y2.data_ptr(), 0, x2.numel(), e, m, 1, sp))
    torch.cuda.synchronize()


# kernel-name fragments of the counter probe's launches ('a|b': all must occur; the last template argument of
# mxfp_bf16_b32_kernel is its mode: 0 extract, 1 fused QDQ) -> (key in the summary, algorithmic bytes
# read, written, sources).  A key is "<kernel row of hbm_kernels> <config>" for the cast rows.
_N1, _N3, _N2 = 4096 * 4096, 14336 * 4096, 1 << 24
_M4, _N4, _K4 = 16384, 14336, 4096
_M5, _H5, _I5 = 8192, 4096, 14336
COUNTER_ROWS = (
    ("stream_copy_kernel", "calibration copy (256 MiB read, 256 MiB written)", 256 << 20, 256 << 20, None),
    ("mxfp_gemm_scaled_kernel", "mxfp_gemm_scaled_kernel C4", (_M4 + _N4) * _K4 * 33 // 32, _M4 * _N4 * 2, SCALED_SOURCES),
    ("mxfp_gemm_scaled_rows_regs_kernel<2, 1, 8>", "mxfp_gemm_scaled_rows C4 W x 16 rows", _N4 * _K4 * 33 // 32 + 16 * _K4 * 33 // 32, 16 * _N4 * 2, ROWS_SOURCES),
    ("mxfp_gemm_tall_kernel", "mxfp_gemm_tall_kernel C4", _M4 * _K4 * 2 + _N4 * _K4 * 33 // 32, _M4 * _N4 * 2, GEMM_SOURCES),
    ("mxfp_gemm_scaled_kernel", "mxfp_gemm_scaled_kernel C5 gate+up", (_M5 + 2 * _I5) * _H5 * 33 // 32, _M5 * 2 * _I5 * 2, SCALED_SOURCES),
    ("mxfp_gemm_scaled_kernel", "mxfp_gemm_scaled_kernel C5 down", (_M5 + _H5) * _I5 * 33 // 32, _M5 * _H5 * 2, SCALED_SOURCES),
    ("mxfp_gemm_scaled_rows_regs_kernel<2, 4, 8>", "mxfp_gemm_scaled_rows C4 W x 64 rows", _N4 * _K4 * 33 // 32 + 64 * _K4 * 33 // 32, 64 * _N4 * 2, ROWS_SOURCES),
    ("scaled_from_dense_kernel|0>, 1>(", "scaled_operand_from_swiglu C5", _M5 * _I5 * 4, _M5 * _I5 * 33 // 32, CAST_SOURCES),
    ("scaled_from_dense_kernel|0>, 0>(", "scaled_operand_from_dense C4 x", _M4 * _K4 * 2, _M4 * _K4 * 33 // 32, CAST_SOURCES),
    ("scaled_operand_kernel<mase::SFmt<4, 3", "scaled_operand_from_mxfp C4 W", _N4 * _K4 * 33 // 32, _N4 * _K4 * 33 // 32, CAST_SOURCES),
    ("mxfp_bf16_b32_kernel<mase::SFmt<4, 3|, 0>(", "extract_mxfp C1", _N1 * 2, _N1 + _N1 // 32, CAST_SOURCES),
    ("compose_mxfp_bf16_kernel<mase::SFmt<4, 3", "compose_mxfp C1", _N1 + _N1 // 32, _N1 * 2, CAST_SOURCES),
    ("mxfp_bf16_b32_kernel<mase::SFmt<4, 3|, 1>(", "qdq_mxfp_fused C1", _N1 * 2, _N1 * 2, CAST_SOURCES),
    ("mxfp_bf16_b32_kernel<mase::SFmt<2, 1|, 0>(", "extract_mxfp C3", _N3 * 2, _N3 + _N3 // 32, CAST_SOURCES),
    ("compose_mxfp_bf16_kernel<mase::SFmt<2, 1", "compose_mxfp C3", _N3 + _N3 // 32, _N3 * 2, CAST_SOURCES),
    ("mxfp_bf16_b32_kernel<mase::SFmt<2, 1|, 1>(", "qdq_mxfp_fused C3", _N3 * 2, _N3 * 2, CAST_SOURCES),
    ("minifloat_f32_kernel<2, mase::SFmt<4, 3", "qdq_minifloat_fused C2/E4M3", _N2 * 4, _N2 * 4, CAST_SOURCES),
    ("minifloat_f32_kernel<0, mase::SFmt<4, 3", "extract_minifloat C2/E4M3", _N2 * 4, _N2 * 2, CAST_SOURCES),
    ("minifloat_f32_kernel<1, mase::SFmt<4, 3", "compose_minifloat C2/E4M3", _N2 * 2, _N2 * 4, CAST_SOURCES),
    ("minifloat_f32_kernel<2, mase::SFmt<5, 2", "qdq_minifloat_fused C2/E5M2", _N2 * 4, _N2 * 4, CAST_SOURCES),
    ("minifloat_f32_kernel<0, mase::SFmt<5, 2", "extract_minifloat C2/E5M2", _N2 * 4, _N2 * 2, CAST_SOURCES),
    ("minifloat_f32_kernel<1, mase::SFmt<5, 2", "compose_minifloat C2/E5M2", _N2 * 2, _N2 * 4, CAST_SOURCES),
)
# launches of one kernel name at several sizes (the probe also quantises the headline's x and W): the size that is meant, in threads
_COUNTER_THREADS = {"extract_mxfp C1": _N1 // 16, "extract_mxfp C3": _N3 // 16, "qdq_mxfp_fused C1": _N1 // 16, "qdq_mxfp_fused C3": _N3 // 16,
                    "scaled_operand_from_dense C4 x": _M4 * _K4 // 16, "scaled_operand_from_mxfp C4 W": _N4 * _K4 // 64}
# launches of one kernel name at one launch size (the block-scaled GEMM is always one workgroup per compute unit): which of
# the probe's launches, in dispatch order
_COUNTER_LAUNCHES = {"mxfp_gemm_scaled_kernel C4": (0, 3), "mxfp_gemm_scaled_kernel C5 gate+up": (3, 6), "mxfp_gemm_scaled_kernel C5 down": (6, 9)}


def summarize_counters(fetch_dir, write_dir):
    """Markdown summary (stdout) of the two rocprofv3 --pmc runs of `--counter-probe`: KiB per dispatch of FETCH_SIZE and
    WRITE_SIZE for each kernel, scaled by what the same counters read for the calibration copy, next to the algorithmic
    bytes; ends with the machine-readable block that the benchmark reads roofline.traffic from."""
    import csv
    import glob

    csv.field_size_limit(1 << 30)

    def per_kernel(folder, counter):
        files = glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            raise SystemExit(f"no *counter_collection.csv under {folder}")
        vals = {}
        recs = sorted((r for r in csv.DictReader(open(files[0])) if r["Counter_Name"] == counter), key=lambda r: int(r["Dispatch_Id"]))
        for r in recs:   # keyed by kernel name and launch size: the probe also extracts the GEMM's weight
            vals.setdefault((r["Kernel_Name"], int(r["Grid_Size"])), []).append(float(r["Counter_Value"]))
        return vals

    fetch, write = per_kernel(fetch_dir, "FETCH_SIZE"), per_kernel(write_dir, "WRITE_SIZE")

    def pick(table, frag, threads, launches):
        hits = [(k[0], v) for k, v in table.items() if all(part in k[0] for part in frag.split("|")) and (threads is None or k[1] == threads)]
        if len(hits) != 1:
            raise SystemExit(f"{len(hits)} kernels match '{frag}' with {threads} threads: {[k[:80] for k, _ in hits]}")
        name, v = hits[0]
        if launches is not None:
            if len(v) < launches[1]:
                raise SystemExit(f"'{frag}': {len(v)} launches recorded, launches {launches} asked for")
            v = v[launches[0]:launches[1]]
        return name, sum(v) / len(v)

    rows = []
    for frag, key, rd, wr, sources in COUNTER_ROWS:
        threads = _COUNTER_THREADS.get(key)   # one lane per 2 x 8 elements
        launches = _COUNTER_LAUNCHES.get(key)
        (name, f_kib), (_, w_kib) = pick(fetch, frag, threads, launches), pick(write, frag, threads, launches)
        rows.append((key, name, f_kib, w_kib, rd, wr, sources))
    cal = rows[0]
    f_fac, w_fac = (cal[4] / 1024) / cal[2], (cal[5] / 1024) / cal[3]
    print("| kernel / workload | FETCH_SIZE (KiB) | WRITE_SIZE (KiB) | fetched (scaled) | written (scaled) | algorithmic read / write (KiB) | ratio |")
    print("|---|---|---|---|---|---|---|")
    table = {}
    for key, name, f_kib, w_kib, rd, wr, sources in rows:
        fs, ws = f_kib * f_fac, w_kib * w_fac
        print(f"| {key} (`{name.split('(')[0][:70]}`) | {f_kib:.1f} | {w_kib:.1f} | {fs:.0f} KiB | {ws:.0f} KiB | {rd / 1024:.0f} / {wr / 1024:.0f} | "
              f"{fs * 1024 / rd:.2f} / {ws * 1024 / wr:.2f} |")
        if sources is not None:
            table[key] = {"traffic_bytes": int((fs + ws) * 1024), "fetch_bytes": int(fs * 1024), "write_bytes": int(ws * 1024),
                          "algorithmic_bytes": rd + wr, "sources": sources_fingerprint(sources)}
    table["extract+compose_mxfp C1"] = {k: (table["extract_mxfp C1"][k] + table["compose_mxfp C1"][k]) if k != "sources" else table["extract_mxfp C1"][k]
                                        for k in table["extract_mxfp C1"]}
    table["extract+compose_mxfp C3"] = {k: (table["extract_mxfp C3"][k] + table["compose_mxfp C3"][k]) if k != "sources" else table["extract_mxfp C3"][k]
                                        for k in table["extract_mxfp C3"]}
    print(f"\nCalibration: the copy of known size gives the factors {f_fac:.3f} (FETCH_SIZE) and {w_fac:.3f} (WRITE_SIZE).\n")
    print("Read by `bench.py` (`roofline.traffic`; `sources` = fingerprint of the kernel sources the counters were taken with):\n")
    print("```json")
    print(json.dumps(table, indent=1))
    print("```")


def c5_traffic():
    """HBM bytes of the block's two GEMM launches together, from the counter summary."""
    parts = [traffic_bytes(f"mxfp_gemm_scaled_kernel C5 {k}", SCALED_SOURCES) for k in ("gate+up", "down")]
    return None if None in parts else sum(parts)


def bench_c5(torch, with_cpu, steps=20, warmup=8):
    """Configuration C5: a Llama-3-8B SwiGLU MLP block of MXFPLinearPTQ layers, down(silu(gate(x)) * up(x)), weights
    gate / up [14336, 4096] and down [4096, 14336] ~N(0, 0.02) stored as MXFP6 E3M2, MXFP8 E4M3 activations, block 32,
    x [4 x 2048, 4096] bf16 ~N(0, 1) (tests/workloads.py: make_c5).  Gate and up are stacked into one [28672, 4096] layer
    (MXFP blocks run along in_features, so stacking rows changes no value): x is quantised once and one GEMM serves both.
    Per block on backend "fused": quantise x, GEMM, one kernel for SiLU, product and quantisation, GEMM
    (MXFPLinearPTQ.forward_swiglu); on the other backends SiLU and the product are torch's."""
    import workloads
    from mase_hip.mxfp import kernels
    from mase_hip.mxfp.layers import MXFPLinearPTQ
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn, MXFPMeta

    dev = "cuda:0"
    x_cpu, wg, wu, wd = workloads.make_c5()
    x = x_cpu.to(dev)
    wfmt = MXFPMeta(32, 8, 3, 2, True, "rn")
    inter = wg.shape[0]
    flop = 3 * 2.0 * x.shape[0] * x.shape[1] * wg.shape[0] * wg.shape[1]
    ms = {}
    for backend in ("fused", "fused_bf16", "separate"):
        ls = []
        for w in (torch.cat([wg, wu]), wd):
            lin = torch.nn.Linear(w.shape[1], w.shape[0], bias=False, dtype=torch.bfloat16, device=dev)
            lin.weight.data.copy_(w)
            ls.append(MXFPLinearPTQ.from_linear(lin, MXFP8_E4M3_fn, wfmt, None, "XqWqB", backend))
            del lin
        gu, d = ls

        def mlp():
            t = gu(x)
            if backend == "fused":      # activation, product and quantisation of the down layer's input in one kernel
                return d.forward_swiglu(t[..., :inter], t[..., inter:])
            return d(torch.nn.functional.silu(t[..., :inter]) * t[..., inter:])

        ms[backend] = timed_loop(torch, mlp, steps, warmup)
        if backend == "fused":
            # the block's four kernels launched directly (what the two layer calls above launch), so that events on the
            # launch stream can bracket the two GEMMs inside the timed loop
            rows = x.shape[0] * x.shape[1]
            x2d = x.view(rows, -1)
            w1, w2 = gu._weight_operand(x), d._weight_operand(torch.empty(rows, inter, dtype=x.dtype, device=dev))
            assert w1 is not None and w2 is not None, "the C5 layers did not take the block-scaled route"

            def block(ev=None):
                a1 = kernels.scaled_operand_from_dense(x2d, MXFP8_E4M3_fn)
                if ev is not None:
                    ev[0][0].record()
                t = kernels.mxfp_gemm_scaled(a1, w1, None, torch.bfloat16)
                if ev is not None:
                    ev[0][1].record()
                a2 = kernels.scaled_operand_from_swiglu(t[:, :inter], t[:, inter:], MXFP8_E4M3_fn)
                if ev is not None:
                    ev[1][0].record()
                y = kernels.mxfp_gemm_scaled(a2, w2, None, torch.bfloat16)
                if ev is not None:
                    ev[1][1].record()
                return y

            assert torch.equal(block().view(torch.int16).view(-1), mlp().view(torch.int16).view(-1)), "the event-bracketed block differs from the layers' output"
            for _ in range(warmup):
                block()
            torch.cuda.synchronize()
            evs = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(2)] for _ in range(steps)]
            for i in range(steps):
                block(evs[i])
            torch.cuda.synchronize()
            gemm_ms = [sum(event_ms([e[j] for e in evs])) / steps for j in range(2)]
            del w1, w2
        del ls, gu, d
    tf = lambda t: flop / (t * 1e-3) / 1e12
    kern_tf = tf(sum(gemm_ms))
    out = {
        "workload": "C5 SwiGLU block: x[4x2048,4096] bf16, gate+up stacked [28672,4096], down [4096,14336], W MXFP6 E3M2, X MXFP8 E4M3",
        "ms_per_block": {k: round(v, 4) for k, v in ms.items()},
        "TFLOPs": {k: round(tf(v), 1) for k, v in ms.items()},
        "roofline": {"bound": "mfma", "achieved": round(kern_tf, 1), "peak": MFMA_FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(kern_tf / MFMA_FP8_PEAK_TFLOPS, 4), "frac_of_bf16_peak": round(kern_tf / MFMA_BF16_PEAK_TFLOPS, 4),
                     "kernel": "mxfp_gemm_scaled_kernel", "avg_kernel_ms": {"gate_up": round(gemm_ms[0], 4), "down": round(gemm_ms[1], 4)},
                     "traffic": c5_traffic()},
        "note": "flop = the three GEMMs; ms_per_block = whole block (quantise kernels, GEMMs, SiLU and product; fused: the down layer reads gate and up through forward_swiglu)",
    }
    if with_cpu:
        from oracle import torch_fake

        comps = [torch_fake.mxfp_split(w, 32, 3, 2) for w in (wg, wu, wd)]
        x2 = x_cpu.view(-1, x_cpu.shape[-1])

        def chain(rows):
            t0 = time.perf_counter()
            xs = x2[:rows]
            g = torch_fake.mxfp_linear_xq_wq(xs, *comps[0], tuple(wg.shape), torch.bfloat16, (4, 3), (3, 2))
            u = torch_fake.mxfp_linear_xq_wq(xs, *comps[1], tuple(wu.shape), torch.bfloat16, (4, 3), (3, 2))
            y = torch_fake.mxfp_linear_xq_wq(torch.nn.functional.silu(g) * u, *comps[2], tuple(wd.shape), torch.bfloat16, (4, 3), (3, 2))
            assert y.shape == (rows, wd.shape[0])
            return time.perf_counter() - t0

        t_probe = chain(256)
        rows = int(min(x2.shape[0], max(256, 256 * (10.0 / max(t_probe, 1e-3)))) // 256 * 256)
        dt = chain(rows)
        out["cpu_baseline"] = {"value": round(flop * rows / x2.shape[0] / dt / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                               "kind": "port", "sample": f"{rows} of {x2.shape[0]} rows through the three layers, {dt:.1f} s"}
    return out


def summarize_sq(counter_csv):
    """Markdown table (stdout) of the library's kernels in a rocprofv3 --pmc run: cycles per launch, MFMA pipe busy,
    VALU / LDS instructions per wavefront, share of wavefront time in waits."""
    import collections
    import csv
    import re

    csv.field_size_limit(1 << 30)
    d = collections.OrderedDict()
    for r in csv.DictReader(open(counter_csv)):
        m = re.search(r"mase::(\w+)", r["Kernel_Name"])
        if not m:
            continue
        key = (m.group(1), int(r["Grid_Size"]) // max(1, int(r["Workgroup_Size"])), int(r["Workgroup_Size"]))
        d.setdefault(key, collections.defaultdict(list))[r["Counter_Name"]].append(float(r["Counter_Value"]))
    print("| kernel | workgroups x threads | launches | cycles per launch | MFMA pipe busy | VALU / wavefront | LDS / wavefront | LDS bank conflict | wavefront time in waits |")
    print("|---|---|---|---|---|---|---|---|---|")
    for k, c in d.items():
        mean = {n: sum(v) / len(v) for n, v in c.items()}
        if "SQ_BUSY_CYCLES" not in mean or "SQ_WAVES" not in mean:
            continue
        cyc = mean["SQ_BUSY_CYCLES"] / 32            # summed over 32 shader engines
        waves = mean["SQ_WAVES"]
        busy = f"{mean['SQ_VALU_MFMA_BUSY_CYCLES'] / 1024 / cyc * 100:.1f} %" if "SQ_VALU_MFMA_BUSY_CYCLES" in mean else "-"   # 1024 SIMDs
        valu = f"{mean['SQ_INSTS_VALU'] / waves:.0f}" if "SQ_INSTS_VALU" in mean else "-"
        lds = f"{mean['SQ_INSTS_LDS'] / waves:.0f}" if "SQ_INSTS_LDS" in mean else "-"
        conf = f"{mean['SQ_LDS_BANK_CONFLICT'] / 256 / cyc * 100:.1f} % of cycles" if "SQ_LDS_BANK_CONFLICT" in mean else "-"   # 256 CUs
        wait = f"{mean['SQ_WAIT_ANY'] / mean['SQ_WAVE_CYCLES'] * 100:.1f} %" if "SQ_WAIT_ANY" in mean and "SQ_WAVE_CYCLES" in mean else "-"
        print(f"| `{k[0]}` | {k[1]} x {k[2]} | {len(next(iter(c.values())))} | {cyc:.4g} | {busy} | {valu} | {lds} | {conf} | {wait} |")


def summarize_trace(trace_csv):
    """Markdown table (stdout) of per-kernel durations in a rocprofv3 --kernel-trace run."""
    import collections
    import csv
    import re

    csv.field_size_limit(1 << 30)
    d = collections.OrderedDict()
    meta = {}
    for r in csv.DictReader(open(trace_csv)):
        n = re.sub(r"^void ", "", r["Kernel_Name"])
        n = re.sub(r"\(.*$", "", n)
        if "mase::" not in n and "Cijk" not in n:
            continue
        key = (n[:120], int(r["Grid_Size_X"]) // max(1, int(r["Workgroup_Size_X"])), int(r["Workgroup_Size_X"]))
        d.setdefault(key, []).append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1000.0)
        meta[key] = (r.get("LDS_Block_Size", "-"), r.get("VGPR_Count", "-"), r.get("Accum_VGPR_Count", "-"), r.get("Scratch_Size", "-"))
    print("| kernel | workgroups x threads | launches | mean us | median us | min us | LDS | VGPR | AGPR | scratch |")
    print("|---|---|---|---|---|---|---|---|---|---|")
    for k, v in d.items():
        v = sorted(v)
        m = meta[k]
        print(f"| `{k[0]}` | {k[1]} x {k[2]} | {len(v)} | {sum(v) / len(v):.2f} | {v[len(v) // 2]:.2f} | {v[0]:.2f} | {m[0]} | {m[1]} | {m[2]} | {m[3]} |")


def main():
    args = parse_args()
    if args.summarize_counters:
        summarize_counters(*args.summarize_counters)
        return
    if args.summarize_sq:
        summarize_sq(args.summarize_sq)
        return
    if args.summarize_trace:
        summarize_trace(args.summarize_trace)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this pool has a single MI355X and the path has no "
              "cross-GPU step; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the product has no CPU path)", file=sys.stderr)
        sys.exit(2)
    import mase_hip.mxfp.functional as MXFP_F
    import mase_hip.mxfp.kernels as mxk
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn, MXFPMeta

    torch.cuda.set_device(0)
    if args.counter_probe:
        counter_probe(torch, MXFP_F, mxk, MXFP8_E4M3_fn, MXFPMeta(32, 8, 2, 1, True, "rn"))
        return
    if args.shape_sweep:
        print(json.dumps({"shape_sweep": shape_sweep(torch, MXFP_F, mxk, MXFP8_E4M3_fn)}))
        return
    lin = bench_linear(args, torch, MXFP_F, mxk, MXFP8_E4M3_fn)
    if lin is None:
        return
    M, N, K = lin["shape"]
    tf = lambda ms: round(lin["flop"] / (ms * 1e-3) / 1e12, 2)
    # key order: the driver's record keeps the standard keys and the tail of the line, so the long per-kernel list goes in
    # the middle and the comparisons last
    result = {
        "metric": "mxfp_linear TFLOP/s at 16384x4096x14336 (MXFP8 E4M3 x MXFP8 E4M3, block 32)",
        "value": round(lin["tflops_step"], 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(lin["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8 (E4M3 codes x E8M0 block scales in the matrix unit, fp32 accumulate; MXFP values are exact in it)",
        "data": "synthetic",
        "config": {"workload": "C4 mxfp_linear XqWqB fused: x[16384,4096] bf16 -> MXFP8 E4M3, W[14336,4096] MXFP8 E4M3, bf16 out",
                   "M": M, "N": N, "K": K, "inputs": "tests/workloads.py make_c4 (seeds 3, 4)",
                   "step": "quantise x to FP8 operand + weight components to FP8 operand + block-scaled GEMM"},
        "roofline": {"bound": "mfma", "achieved": round(lin["tflops_gemm"], 2), "peak": MFMA_FP8_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(lin["tflops_gemm"] / MFMA_FP8_PEAK_TFLOPS, 4),
                     "traffic": traffic_bytes("mxfp_gemm_scaled_kernel C4", SCALED_SOURCES),
                     "kernel": "mxfp_gemm_scaled_kernel", "avg_kernel_ms": round(lin["gemm_ms"], 4),
                     "frac_of_bf16_peak": round(lin["tflops_gemm"] / MFMA_BF16_PEAK_TFLOPS, 4),
                     "bf16_kernel": {"kernel": "mxfp_gemm_tall_kernel on the weight operand a layer keeps", "achieved": round(lin["bf16_tflops_gemm"], 2),
                                     "peak": MFMA_BF16_PEAK_TFLOPS, "frac": round(lin["bf16_tflops_gemm"] / MFMA_BF16_PEAK_TFLOPS, 4),
                                     "avg_kernel_ms": round(lin["bf16_gemm_ms"], 4), "traffic": traffic_bytes("mxfp_gemm_tall_kernel C4", GEMM_SOURCES),
                                     "on_weight_components": {"achieved": round(lin["bf16c_tflops_gemm"], 2), "avg_kernel_ms": round(lin["bf16c_gemm_ms"], 4),
                                                              "frac": round(lin["bf16c_tflops_gemm"] / MFMA_BF16_PEAK_TFLOPS, 4)}}},
    }
    result["cpu_baseline"] = None if args.no_cpu else cpu_baseline(torch)
    if not args.skip_hbm:
        result["hbm_kernels"] = bench_hbm(torch, with_cpu=not args.no_cpu)
        result["c5"] = bench_c5(torch, with_cpu=not args.no_cpu)
    result["prewarm"] = lin["prewarm"]
    result["context"] = {
        "same_shape_ms_per_step": {
            "fused (value)": round(lin["ms_per_step"], 4), "fused, weight operand kept by a layer": round(lin["prepared_ms"], 4),
            "fused_bf16, weight operand kept by a layer": round(lin["bf16_ms_per_step"], 4), "fused_bf16": round(lin["bf16c_ms_per_step"], 4),
            "separate": round(lin["separate_ms"], 4),
            "vendor dense bf16 GEMM alone": round(lin["dense_ms"], 4)},
        "same_shape_TFLOPs": {
            "fused (value)": tf(lin["ms_per_step"]), "fused, weight operand kept by a layer": tf(lin["prepared_ms"]),
            "fused_bf16, weight operand kept by a layer": tf(lin["bf16_ms_per_step"]), "fused_bf16": tf(lin["bf16c_ms_per_step"]),
            "separate": tf(lin["separate_ms"]), "vendor dense bf16 GEMM alone": tf(lin["dense_ms"])},
        "note": "fused_bf16 = QDQ of x to bf16 + GEMM composing W to bf16 in registers (bf16 MFMA); separate = extract x + compose x + "
                "compose W to bf16 in HBM + library GEMM; prewarm = uncounted steps until two groups of five agree within 1 %",
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()

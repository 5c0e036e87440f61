#!/usr/bin/env python3
"""Benchmark of the quantized-Linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode|prefill|fp8|block]

A "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM:

  decode  (default; benchmark configuration 1 of 5 (0-based), M=16)  x bf16 [16, 2048] -> per-token int8 quantise ->
          int8 GEMV against W int8 [8192, 2048] -> dequant -> y bf16.  HBM-bound; value = GB/s of
          algorithmic bytes N*K + 4N + 2MK + 2MN.  The weight rotates over 40 distinct buffers
          (671 MB) so that no step finds its weight in the 256 MB last-level cache.
  prefill (configs[2])  x bf16 [4096, 2048] -> per-token int8 quantise -> int8 MFMA GEMM against
          W [2048, 2048] -> fused scale + bias -> y bf16.  value = TOPS of 2*M*N*K.
  fp8     (configs[3])  x bf16 [2048, 8192], W [2048, 8192] e4m3, per-tensor scales.

The K timed steps are captured once into a HIP graph and replayed, so the figure is the GPU's,
not the Python launch loop's; the eager (un-captured) figure is reported beside it.  The
dominant kernel of each workload is also timed on its own (same graph method) for the roofline
object.  The CPU baseline is the C oracle (a scalar restatement, OpenMP over rows) on the same
shapes, timed on the host in the same run.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "quantized-linear TOPS & HBM GB/s (% roofline), decode M=16 and prefill M=4096"
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, published
PEAK_INT8_TOPS = 5000.0      # dense int8 MFMA, published (no sparsity)
PEAK_FP8_TFLOPS = 5000.0     # dense FP8 MFMA, published

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_fetch_write_size.txt")

# What the part delivers on trivial kernels, measured at the start of this run (measure_ceilings): the roofline
# objects quote the kernel against these next to the published peaks.
CEIL = {}


def hbm_ceiling_fields(kernel_us):
    """Same-run ceiling of a decode-sized HBM kernel: the fastest ONE launch that reads 16 MiB once."""
    floor = CEIL.get("one_shot_16mib_read_us")
    if not floor:
        return {}
    return {"floor_us_one_shot_read": floor, "frac_of_floor": floor / kernel_us,
            "empty_kernel_in_graph_us": CEIL.get("empty_kernel_in_graph_us")}


def mfma_ceiling_fields(achieved, fp8, clock_mhz):
    """Same-run ceiling of a matrix-core kernel: an MFMA-only loop on random operands (no memory traffic), the
    clock that loop ran at, and the clock the kernel itself ran at (lab build of the same source, see gemm_clock_mhz)."""
    name = "mfma_fp8_32x32x64_random_operands" if fp8 else "mfma_i8_32x32x32_random_operands"
    unit = "tflops" if fp8 else "tops"
    loop = CEIL.get(f"{name}_{unit}")
    if not loop:
        return {}
    return {"mfma_loop_random_operands_" + unit: loop, "mfma_loop_random_operands_clock_mhz": CEIL.get(f"{name}_clock_mhz"),
            "mfma_loop_constant_operands_" + unit: CEIL.get(name.replace("random", "constant") + "_" + unit),
            "mfma_loop_constant_operands_clock_mhz": CEIL.get(name.replace("random", "constant") + "_clock_mhz"),
            "shader_clock_mhz_during_kernel": clock_mhz, "frac_of_measured_loop": achieved / loop}


def gemm_clock_mhz(torch, ops, kernel_only, steps):
    """The shader clock the tiled GEMM runs at under this workload: the lab library's compile of the same source
    has wavefront 0 of workgroup 0 read the shader-clock and the 100 MHz reference counters at its start and end
    (aq_lab_read_clock); their ratio over a conditioned graph replay of the same calls is the clock."""
    import ctypes

    try:
        with ops._abi.lab_library() as lab:
            graph_time_ms(torch, kernel_only, steps, steps)
            buf = (ctypes.c_longlong * 8)()
            if lab.aq_lab_read_clock(buf) != 0 or buf[1] <= 0:
                return None
            return buf[0] / buf[1] * 100.0
    except Exception as e:  # a probe: never fails the run
        return f"unavailable: {str(e)[:80]}"


def measured_traffic(key):
    """Bytes per launch that the dominant kernel of workload `key` moves past the L2: FETCH_SIZE + WRITE_SIZE of
    two rocprofv3 --pmc runs of this script, scaled by what the same counters read for kernels of known size.
    Counters cannot be read from inside a timed run, so the figure comes from the committed summary of those runs
    (its `traffic` lines), which names the kernel's source file and that file's SHA-256 at the time of the
    measurement: when the source has changed since, the figure is stale and None is reported instead."""
    import hashlib

    try:
        for line in open(TRAFFIC_FILE):
            f = line.split()
            if len(f) >= 2 and f[0] == "traffic" and f[1] == key:
                kv = dict(x.split("=", 1) for x in f[2:])
                src = os.path.join(ROOT, kv["source"])
                if hashlib.sha256(open(src, "rb").read()).hexdigest() != kv["sha256"]:
                    return None, f"stale: {kv['source']} changed since the counters were read"
                return float(kv["fetch_bytes"]) + float(kv["write_bytes"]), f"{os.path.basename(TRAFFIC_FILE)}: {kv['kernel']}"
    except (OSError, KeyError, ValueError) as e:
        return None, f"unreadable: {e}"
    return None, "no counter run recorded for this workload"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=1000)
    ap.add_argument("--workload", default="decode", choices=["decode", "prefill", "fp8", "block", "model"])
    ap.add_argument("--m", type=int, default=16, help="decode rows (1..16)")
    ap.add_argument("--mnk", default=None, help="prefill and fp8 workloads only: M,N,K of the int8 Linear instead of configuration 3's "
                    "4096,2048,2048 (e.g. 8192,8192,8192 for a profile of the GEMM's steady state)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    return ap.parse_args()


CONDITION_MS = 200.0  # untimed replays in front of every timed one, by time (the clocks settle under the load itself)


def graph_time_ms(torch, step, steps, warmup, dist=None, info=None):
    """Warm up, capture `steps` calls of step(i) into one HIP graph, then time one replay with events on
    the launching stream.  Returns ms per step.  The untimed part runs the way the timed one does: a few eager
    calls first (allocations, lazy initialisation), then whole untimed replays of the graph for at least
    CONDITION_MS milliseconds and at least `warmup` steps -- the device reaches its steady clocks only under the
    replayed load, and a replay timed straight after a single warm-up replay reads 2-10 % slower than the ones
    that follow, whatever the number of steps in it.  The K timed steps are one replay between two events.
    dist: a list that receives [p10, p50, p90] of the ms per step of 11 further replays, each timed on its own
    (the spread between replays; not part of the timed region).
    info: a dict that receives conditioning_ms / conditioning_replays of this measurement."""
    for i in range(min(warmup, 20)):
        step(i)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            for i in range(steps):
                step(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    # how long one replay takes, roughly: sizes the conditioning
    t0 = time.perf_counter()
    for _ in range(4):
        g.replay()
    torch.cuda.synchronize()
    per_replay_ms = max((time.perf_counter() - t0) * 1e3 / 4, 1e-3)
    replays = max(1, -(-warmup // steps), int(CONDITION_MS / per_replay_ms) + 1)
    t0 = time.perf_counter()
    for _ in range(replays):
        g.replay()
    torch.cuda.synchronize()
    cond_ms = (time.perf_counter() - t0) * 1e3
    # The timed replay follows two untimed ones on the stream without a gap: the first launch after the device
    # has sat idle in a synchronize() pays for waking up (a fixed 5-10 us here, 2-5 % of a 20-step replay),
    # which is the host's pause and no part of a step.
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(11 if dist is not None else 0)]
    g.replay()
    g.replay()
    e0.record()
    g.replay()
    e1.record()
    for a, b in evs:  # the spread: further replays behind the timed one, each between its own events
        a.record()
        g.replay()
        b.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    if info is not None:
        info["conditioning_ms"] = cond_ms
        info["conditioning_replays"] = replays
    if dist is not None:
        t = sorted(a.elapsed_time(b) / steps for a, b in evs)
        dist[:] = [t[1], t[5], t[9]]
    return ms


def eager_time_ms(torch, step, steps, warmup):
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def make_weights(torch, ops, N, K, nbuf, dev, seed, mode="int8"):
    """nbuf independently drawn weights N(0, 0.02), quantised on the GPU by the library."""
    g = torch.Generator(device=dev).manual_seed(seed)
    out = []
    for _ in range(nbuf):
        w = torch.randn(N, K, generator=g, device=dev) * 0.02
        out.append(ops.quant_rowwise_i8(w) if mode == "int8" else ops.quant_tensor_fp8(w))
    return out


def bench_decode(torch, ops, args, dev):
    M, K, N = args.m, 2048, 8192
    nbuf = 40
    weights = make_weights(torch, ops, N, K, nbuf, dev, seed=1)
    g = torch.Generator(device=dev).manual_seed(2)
    x = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
    ws = torch.empty((ops._abi.load().aq_gemv_w8a8_workspace_bytes(M, K),), dtype=torch.uint8, device=dev)
    ys = [None]

    def step(i):
        wq, sw = weights[i % nbuf]
        ys[0] = ops.gemv_w8a8_decode(x, wq, sw, None, out_dtype=torch.bfloat16, workspace=ws)

    xq, sx = ops.quant_rowwise_i8(x)

    def kernel_only(i):
        wq, sw = weights[i % nbuf]
        ys[0] = ops.gemv_w8a8_codes(xq, sx, wq, sw, None, out_dtype=torch.bfloat16)

    def resident(i):  # same weight every step: served by the last-level cache
        wq, sw = weights[0]
        ys[0] = ops.gemv_w8a8_codes(xq, sx, wq, sw, None, out_dtype=torch.bfloat16)

    # The step is ONE launch: the GEMV kernel quantises its token rows itself (dot-product kernel up to 4 rows,
    # matrix-core kernel from 5 rows on at this N), so the step's time is the dominant kernel's duration.
    # Bytes: the weight once, its scales, the bf16 rows in, the bf16 outputs.
    bytes_alg = N * K + 4 * N + 2 * M * K + 2 * M * N
    d_step, d_k, cond = [], [], {}
    ms = graph_time_ms(torch, step, args.steps, args.warmup, d_step, cond)
    ms_eager = eager_time_ms(torch, step, args.steps, args.warmup)
    ms_k = graph_time_ms(torch, kernel_only, args.steps, args.warmup, d_k)
    ms_res = graph_time_ms(torch, resident, args.steps, args.warmup)
    gbs = bytes_alg / (ms * 1e-3) / 1e9
    traffic, traffic_src = measured_traffic(f"decode_m{M}")
    # The same launch WITHOUT its weight stream (lab build of the same source: token rows requested, rounded,
    # barrier, products of zeros, stores): what the rounding that every workgroup repeats costs on its own.
    # Left out of single-workload (profiling) runs: the lab kernel carries the product kernel's name and would be
    # averaged into its counters.
    no_w_us = None
    if M > 8 and not args.no_extra:
        try:
            with ops._abi.lab_library() as lab:
                lab.aq_lab_set_gemv_skip_weights(1)
                try:
                    no_w_us = graph_time_ms(torch, step, args.steps, args.warmup) * 1e3
                finally:
                    lab.aq_lab_set_gemv_skip_weights(0)
        except Exception as e:
            no_w_us = f"unavailable: {str(e)[:80]}"
    return {
        "workload": f"decode_gemv_w8a8 M={M} K={K} N={N} bf16->int8 per-token, W int8 per-channel, bf16 out",
        "value": gbs, "unit": "GB/s", "ms_per_step": ms, "eager_ms_per_step": ms_eager,
        "ms_per_step_p10_p50_p90": d_step, "bytes_per_step": bytes_alg, "dtype": "int8",
        "roofline": {"bound": "hbm", "kernel": ("gemv_mfma_kernel<.., FQ>" if M > 4 else "gemv_w8a8_kernel<.., FUSED>")
                     + " (quantises its rows itself: the whole step)",
                     "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                     "traffic": traffic, "traffic_source": traffic_src,
                     "kernel_us": ms * 1e3, "kernel_us_p10_p50_p90": [v * 1e3 for v in d_step],
                     "algorithmic_bytes": bytes_alg, "weight_buffers": nbuf, **cond, **hbm_ceiling_fields(ms * 1e3),
                     "same_launch_without_weight_stream_us": no_w_us,
                     # the same GEMV on codes that a separate launch (or a producer kernel) has already made
                     "gemv_on_codes": {"kernel_us": ms_k * 1e3, "kernel_us_p10_p50_p90": [v * 1e3 for v in d_k],
                                       **hbm_ceiling_fields(ms_k * 1e3),
                                       "gbs": (bytes_alg - M * K) / (ms_k * 1e-3) / 1e9,
                                       "frac": (bytes_alg - M * K) / (ms_k * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                       "llc_resident_gbs": (bytes_alg - M * K) / (ms_res * 1e-3) / 1e9}},
        "shape": (M, N, K),
    }


def bench_prefill(torch, ops, args, dev):
    M, K, N = 4096, 2048, 2048
    nbuf = 8
    if getattr(args, "mnk", None) and args.workload == "prefill":
        M, N, K = (int(v) for v in args.mnk.split(","))
        nbuf = 8 if M * K <= (1 << 25) else 2
    weights = make_weights(torch, ops, N, K, nbuf, dev, seed=3)
    g = torch.Generator(device=dev).manual_seed(4)
    xs = []
    for _ in range(nbuf):
        x = torch.randn(M, K, generator=g, device=dev)
        cols = torch.randperm(K, generator=g, device=dev)[:max(1, K // 100)]  # 1 % outlier channels x10
        x[:, cols] *= 10
        xs.append(x.to(torch.bfloat16))
    bias = (torch.randn(N, generator=g, device=dev) * 0.01)
    ys = [None]

    def step(i):
        xq, sx = ops.quant_rowwise_i8(xs[i % nbuf])
        wq, sw = weights[i % nbuf]
        ys[0] = ops.linear_w8a8(xq, sx, wq, sw, bias, out_dtype=torch.bfloat16)

    pre = [ops.quant_rowwise_i8(x) for x in xs]

    def kernel_only(i):
        xq, sx = pre[i % nbuf]
        wq, sw = weights[i % nbuf]
        ys[0] = ops.linear_w8a8(xq, sx, wq, sw, bias, out_dtype=torch.bfloat16)

    def kernel_resident(i):  # the same launch on ONE operand set: inputs served by the caches, not streamed
        xq, sx = pre[0]
        wq, sw = weights[0]
        ys[0] = ops.linear_w8a8(xq, sx, wq, sw, bias, out_dtype=torch.bfloat16)

    def quant_only(i):
        ys[0] = ops.quant_rowwise_i8(xs[i % nbuf])

    gamma = (1 + 0.1 * torch.randn(K, generator=g, device=dev)).to(torch.bfloat16)

    def norm_quant_only(i):  # RMSNorm fused with the same quantisation (what feeds q/k/v and up/gate)
        ys[0] = ops.rmsnorm_quant_rowwise_i8(xs[i % nbuf], gamma, 1e-5)

    ops_alg = 2.0 * M * N * K
    steps = max(10, min(args.steps, 100))
    d_step, d_k, cond = [], [], {}
    ms = graph_time_ms(torch, step, steps, args.warmup, d_step)
    ms_k = graph_time_ms(torch, kernel_only, steps, args.warmup, d_k, cond)
    clock_mhz = gemm_clock_mhz(torch, ops, kernel_only, steps)
    ms_kr = graph_time_ms(torch, kernel_resident, steps, args.warmup)
    ms_q = graph_time_ms(torch, quant_only, steps, args.warmup)
    ms_nq = graph_time_ms(torch, norm_quant_only, steps, args.warmup)
    tops = ops_alg / (ms * 1e-3) / 1e12
    tops_k = ops_alg / (ms_k * 1e-3) / 1e12
    traffic, traffic_src = measured_traffic("prefill") if (M, N, K) == (4096, 2048, 2048) else (None, "not measured for this shape")
    qbytes = 2 * M * K + M * K + 4 * M
    return {
        "workload": f"prefill_linear_w8a8 M={M} K={K} N={N} quantise + int8 MFMA GEMM + scale/bias epilogue, bf16 out",
        "value": tops, "unit": "TOPS", "ms_per_step": ms, "ms_per_step_p10_p50_p90": d_step, "ops_per_step": ops_alg,
        "dtype": "int8",
        "roofline": {"bound": "mfma", "kernel": "gemm_kernel<int8,bf16>", "achieved": tops_k, "peak": PEAK_INT8_TOPS,
                     "unit": "TOP/s", "frac": tops_k / PEAK_INT8_TOPS, "traffic": traffic, "traffic_source": traffic_src,
                     "kernel_us": ms_k * 1e3, "kernel_us_p10_p50_p90": [v * 1e3 for v in d_k],
                     "algorithmic_ops": ops_alg, **cond, **mfma_ceiling_fields(tops_k, False, clock_mhz),
                     # kernel_us streams 8 rotating operand sets (what a model's layers do); this is the same launch
                     # on one resident set: the difference is the box's memory path, not the kernel
                     "kernel_us_operands_resident": ms_kr * 1e3},
        "quantise_kernel": {"us": ms_q * 1e3, "gbs": qbytes / (ms_q * 1e-3) / 1e9, "frac_hbm": qbytes / (ms_q * 1e-3) / 1e9 / PEAK_HBM_GBS,
                            "algorithmic_bytes": qbytes},
        "rmsnorm_quantise_kernel": {"us": ms_nq * 1e3, "gbs": (qbytes + 2 * K) / (ms_nq * 1e-3) / 1e9,
                                    "algorithmic_bytes": qbytes + 2 * K},
        "shape": (M, N, K),
    }


def bench_few_dozen_rows(torch, ops, args, dev):
    """The same Linear (configuration 2's weight, N = 8192, K = 2048) at batch sizes between the reference's default
    decode batch (16) and a prefill: row quantiser + the Linear on codes, which runs up to 32 rows on the
    weight-streaming kernel and the rest on 128 x 32 or 128 x 64 tiles (128 x 128 tiles: 64 of them here, 9.4 us
    whatever M).  us per step, HIP-graph replay over 40 weights."""
    N, K, nbuf = 8192, 2048, 40
    weights = make_weights(torch, ops, N, K, nbuf, dev, seed=21, mode="int8")
    g = torch.Generator(device=dev).manual_seed(22)
    out = {"workload": f"linear_w8a8 K={K} N={N}, bf16 rows -> int8 per token, bf16 out; quantiser + Linear on codes"}
    for M in (32, 64, 128, 256):
        x = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)

        def step(i, x=x):
            xq, sx = ops.quant_rowwise_i8(x)
            wq, sw = weights[i % nbuf]
            return ops.linear_w8a8(xq, sx, wq, sw, out_dtype=torch.bfloat16)

        xq, sx = ops.quant_rowwise_i8(x)

        def kern(i, xq=xq, sx=sx):
            wq, sw = weights[i % nbuf]
            return ops.linear_w8a8(xq, sx, wq, sw, out_dtype=torch.bfloat16)

        t = graph_time_ms(torch, step, args.steps, args.warmup) * 1e3
        tk = graph_time_ms(torch, kern, args.steps, args.warmup) * 1e3
        nbytes = N * K + 4 * N + 2 * M * K + 2 * M * N
        out[f"M={M}"] = {"us_per_step": t, "linear_on_codes_us": tk, "gbs": nbytes / t / 1e3,
                         "frac_hbm_linear_on_codes": nbytes / tk / 1e3 / PEAK_HBM_GBS, "algorithmic_bytes": nbytes}
    return out


def bench_fp8(torch, ops, args, dev):
    M, K, N = 2048, 8192, 2048
    nbuf = 4
    if getattr(args, "mnk", None) and args.workload == "fp8":
        M, N, K = (int(v) for v in args.mnk.split(","))
        nbuf = 4 if M * K <= (1 << 25) else 2
    weights = make_weights(torch, ops, N, K, nbuf, dev, seed=5, mode="fp8")
    g = torch.Generator(device=dev).manual_seed(6)
    xs = [torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16) for _ in range(nbuf)]
    ys = [None]

    qstate = ops.fp8_onepass_state(dev)  # what Fp8Linear keeps per device and stream

    def step(i):
        xq, sx = ops.quant_tensor_fp8(xs[i % nbuf], state=qstate)  # 32 MiB: the one-launch form
        wq, sw = weights[i % nbuf]
        ys[0] = ops.linear_fp8(xq, sx, wq, sw, out_dtype=torch.bfloat16)

    pre = [ops.quant_tensor_fp8(x) for x in xs]

    def kernel_only(i):
        xq, sx = pre[i % nbuf]
        wq, sw = weights[i % nbuf]
        ys[0] = ops.linear_fp8(xq, sx, wq, sw, out_dtype=torch.bfloat16)

    flops = 2.0 * M * N * K
    steps = max(10, min(args.steps, 50))
    d_k, cond = [], {}
    ms = graph_time_ms(torch, step, steps, args.warmup)
    ms_k = graph_time_ms(torch, kernel_only, steps, args.warmup, d_k, cond)
    clock_mhz = gemm_clock_mhz(torch, ops, kernel_only, steps)
    # the activation quantiser alone, in its one-launch form (what the step uses) and its stateless two-launch form
    qbytes = 3 * M * K  # bf16 read once, codes written
    us_q1 = graph_time_ms(torch, lambda i: ops.quant_tensor_fp8(xs[i % nbuf], state=qstate), steps, args.warmup) * 1e3
    us_q2 = graph_time_ms(torch, lambda i: ops.quant_tensor_fp8(xs[i % nbuf]), steps, args.warmup) * 1e3
    # the same variant at decode sizes (configuration 2's shape): per-tensor cast inside the streaming GEMV
    dec = {}
    if not args.no_extra:
        Nd, Kd = 8192, 2048
        wd = make_weights(torch, ops, Nd, Kd, 40, dev, seed=15, mode="fp8")
        for Md in (1, 16):
            xd = torch.randn(Md, Kd, generator=g, device=dev).to(torch.bfloat16)
            wsd = torch.empty((ops._abi.load().aq_gemv_fp8_workspace_bytes(Md, Kd),), dtype=torch.uint8, device=dev)

            def dstep(i, xd=xd, wsd=wsd):
                wq, sw = wd[i % 40]
                ys[0] = ops.gemv_fp8_decode(xd, wq, sw, None, out_dtype=torch.bfloat16, workspace=wsd)

            t_us = graph_time_ms(torch, dstep, args.steps, args.warmup) * 1e3
            db = Nd * Kd + 2 * Md * Kd + 2 * Md * Nd
            dec[f"M={Md}"] = {"us_per_step": t_us, "gbs": db / t_us / 1e3, "frac_hbm": db / t_us / 1e3 / PEAK_HBM_GBS,
                              "algorithmic_bytes": db}
        del wd
    t = flops / (ms * 1e-3) / 1e12
    tk = flops / (ms_k * 1e-3) / 1e12
    traffic, traffic_src = measured_traffic("fp8") if (M, N, K) == (2048, 2048, 8192) else (None, "not measured for this shape")
    return {
        "workload": f"fp8_linear M={M} K={K} N={N} per-tensor e4m3 quantise + FP8 MFMA GEMM, bf16 out",
        "value": t, "unit": "TFLOP/s", "ms_per_step": ms, "flops_per_step": flops, "dtype": "fp8_e4m3",
        "roofline": {"bound": "mfma", "kernel": "gemm_kernel<fp8,bf16>", "achieved": tk, "peak": PEAK_FP8_TFLOPS,
                     "unit": "TFLOP/s", "frac": tk / PEAK_FP8_TFLOPS, "traffic": traffic, "traffic_source": traffic_src,
                     "kernel_us": ms_k * 1e3, "kernel_us_p10_p50_p90": [v * 1e3 for v in d_k], "algorithmic_flops": flops,
                     **cond, **mfma_ceiling_fields(tk, True, clock_mhz)},
        "quantise_kernel": {"us": us_q1, "gbs": qbytes / us_q1 / 1e3, "frac_hbm": qbytes / us_q1 / 1e3 / PEAK_HBM_GBS,
                            "algorithmic_bytes": qbytes, "two_launch_form_us": us_q2},
        "decode_gemv_fp8_N8192_K2048": dec,
        "shape": (M, N, K),
    }


def bench_block(torch, ops, args, dev):
    """benchmark configuration 4 of 5 (0-based): one int8-quantized 1B-class decoder block, 8 x 512 prefill then 64 decode steps."""
    from khaosz_amd.block import DecoderBlock, PagedKV, decode_mask, rotary_table
    from khaosz_amd.linear import fuse_shared_inputs, quantize_model

    dt = torch.bfloat16
    B, S, steps, dim = 8, 512, 64, 2048
    torch.manual_seed(7)
    blk = DecoderBlock(dim, 16, 5632, 4)
    blk.reset_parameters()
    blk = blk.to(dev).to(dt)
    quantize_model(blk)
    tab = rotary_table(128, S + steps, device=dev)
    x = torch.randn(B, S, dim, device=dev).to(dt)
    xs = torch.randn(steps, B, 1, dim, device=dev).to(dt)
    page = 64  # the serving scheduler's default page size (astrai/inference/core/scheduler.py:26)
    pages_per_seq = (S + steps + page - 1) // page
    cache = PagedKV(B * pages_per_seq, page, 4, 128, dev, dt)
    # physical pages dealt out in a fixed shuffled order, as after some allocation history
    table = torch.randperm(B * pages_per_seq, generator=torch.Generator().manual_seed(8)).view(B, pages_per_seq).to(dev)
    fr = lambda a, n: tab[a:a + n].unsqueeze(0).expand(B, -1, -1)
    # the reference passes an all-zero mask tensor to a step whose sequences sit at one position; the paged
    # kernels take no mask tensor (a tensor would send the step to the stock attention), so once they are
    # switched on the steps pass None
    zero_masks = [decode_mask(B, S + t + 1, dev, dt) for t in range(steps)]
    masks = list(zero_masks)

    def prefill(i=0):
        return blk(x, fr(0, S), None, cache.bind(table, S))

    def decode_all(i=0):
        for t in range(steps):
            blk(xs[t], fr(S + t, 1), masks[t], cache.bind(table, S + t + 1))

    # first with the seven projections launched one by one, as the reference's forward calls them,
    # then with q/k/v and up/gate fused into one projection each (bit-identical outputs)
    ms_pre_sep = graph_time_ms(torch, prefill, 10, 3)
    prefill()
    ms_dec_sep = graph_time_ms(torch, decode_all, 3, 2) / steps
    fuse_shared_inputs(blk)
    ms_pre_proj = graph_time_ms(torch, prefill, 10, 3)
    prefill()
    ms_dec_proj = graph_time_ms(torch, decode_all, 3, 2) / steps
    # and with RMSNorm + activation quantisation as one launch in front of each fused projection
    fuse_shared_inputs(blk, norms=True)
    ms_pre = graph_time_ms(torch, prefill, 10, 3)
    prefill()
    ms_dec_norms = graph_time_ms(torch, decode_all, 3, 2) / steps
    # and the paged-cache kernels: rotary + page writes in one launch at prefill, rotary + page
    # write + in-place attention in one launch for the single-token steps
    fuse_shared_inputs(blk, norms=True, decode_attention=True)
    masks[:] = [None] * steps
    ms_pre_att = graph_time_ms(torch, prefill, 10, 3)
    prefill()
    ms_dec_att = graph_time_ms(torch, decode_all, 3, 2) / steps
    # and the two residual adds inside the epilogues of o_proj and down (bit-identical)
    fuse_shared_inputs(blk, norms=True, decode_attention=True, residuals=True)
    ms_pre_norms, ms_pre = ms_pre, graph_time_ms(torch, prefill, 10, 3)
    prefill()
    ms_dec = graph_time_ms(torch, decode_all, 3, 2) / steps

    # The same steps over 8 distinct blocks in turn, each with its own KV cache: 8 x 45 MB of weights
    # do not stay in the 256 MB last-level cache between steps, as one block's do -- this is what a
    # layer of a whole model sees.
    nb = 8
    blks, caches = [blk], [cache]
    for j in range(1, nb):
        b2 = DecoderBlock(dim, 16, 5632, 4)
        b2.reset_parameters()
        b2 = b2.to(dev).to(dt)
        quantize_model(b2)
        fuse_shared_inputs(b2, norms=True, decode_attention=True, residuals=True)
        c2 = PagedKV(B * pages_per_seq, page, 4, 128, dev, dt)
        b2(x, fr(0, S), None, c2.bind(table, S))
        blks.append(b2)
        caches.append(c2)

    def decode_rotating(i=0):
        for t in range(steps):
            blks[t % nb](xs[t], fr(S + t, 1), masks[t], caches[t % nb].bind(table, S + t + 1))

    ms_dec_rot = graph_time_ms(torch, decode_rotating, 3, 2) / steps
    del blks[1:], caches[1:]

    # The Linears alone (q/k/v and up/gate fused), at the shapes and in the order the block calls them (same modules,
    # inputs of the right shape): what of the block's time is this library's, what is the stock
    # torch attention / RoPE / norm / KV work around it.
    att, mlp = blk.attention, blk.mlp
    lin_calls = [(att._qkv, dim), (att.o_proj, dim), (mlp._upgate, dim), (mlp.down, 5632)]

    def linears_only(rows):
        ins = {k: torch.randn(rows, k, device=dev).to(dt) for k in (dim, 5632)}

        def run(i=0):
            for mod, k in lin_calls:
                mod(ins[k])
        return run

    ms_lin_pre = graph_time_ms(torch, linears_only(B * S), 10, 3)
    ms_lin_dec = graph_time_ms(torch, linears_only(B), 50, 5)
    lin_ops = 2.0 * B * S * 45088768
    lin_bytes = 45088768
    return {
        "workload": "decoder_block hidden=2048 16q/4kv x128 ffn=5632, 7 Linears W8A8, bf16; 8x512 prefill through a paged KV cache (64-token pages) + 64 decode steps (M=8)",
        "value": ms_pre + steps * ms_dec, "unit": "ms", "prefill_ms": ms_pre, "decode_ms_per_step": ms_dec,
        "decode_ms_per_step_weights_from_hbm": ms_dec_rot,
        "separate_projections": {"prefill_ms": ms_pre_sep, "decode_ms_per_step": ms_dec_sep},
        "fused_projections_separate_norms": {"prefill_ms": ms_pre_proj, "decode_ms_per_step": ms_dec_proj},
        "fused_norms_torch_attention": {"prefill_ms": ms_pre_norms, "decode_ms_per_step": ms_dec_norms},
        "paged_attention_kernels_separate_adds": {"prefill_ms": ms_pre_att, "decode_ms_per_step": ms_dec_att},
        "linears_prefill_ms": ms_lin_pre, "linears_prefill_tops": lin_ops / (ms_lin_pre * 1e-3) / 1e12,
        "linears_decode_ms_per_step": ms_lin_dec, "linears_decode_gbs": lin_bytes / (ms_lin_dec * 1e-3) / 1e9,
        "non_linear_prefill_ms": ms_pre - ms_lin_pre, "non_linear_decode_ms_per_step": ms_dec - ms_lin_dec,
        "dtype": "int8", "ms_per_step": ms_pre + steps * ms_dec,
        # the Linear kernels of the block against the published peaks (algorithmic work: 2 * rows * 45 088 768
        # operations at prefill, 45 088 768 weight bytes per decode step), and what is left outside them
        "roofline": {"bound": "hbm", "kernel": "the block's four Linear launches of a decode step (q/k/v, o, up/gate + SwiGLU, down)",
                     "achieved": lin_bytes / (ms_lin_dec * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": lin_bytes / (ms_lin_dec * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": None,
                     "kernel_us": ms_lin_dec * 1e3, "algorithmic_bytes": lin_bytes,
                     "empty_kernel_in_graph_us": CEIL.get("empty_kernel_in_graph_us"),
                     "prefill_linears": {"bound": "mfma", "achieved": lin_ops / (ms_lin_pre * 1e-3) / 1e12,
                                         "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                                         "frac": lin_ops / (ms_lin_pre * 1e-3) / 1e12 / PEAK_INT8_TOPS,
                                         "kernel_us": ms_lin_pre * 1e3, "algorithmic_ops": lin_ops,
                                         **{k: v for k, v in mfma_ceiling_fields(lin_ops / (ms_lin_pre * 1e-3) / 1e12, False, None).items()
                                            if k != "shader_clock_mhz_during_kernel"}},
                     "non_linear_residue": {"prefill_ms": ms_pre - ms_lin_pre, "decode_ms_per_step": ms_dec - ms_lin_dec,
                                            "prefill_frac_of_block": (ms_pre - ms_lin_pre) / ms_pre,
                                            "decode_frac_of_step": (ms_dec - ms_lin_dec) / ms_dec}},
        "shape": (B * S, 0, 0),
    }


def bench_model(torch, ops, args, dev):
    """The reference's own generation benchmark (scripts/tools/benchmark.py:219-248): 24 layers of width 1536,
    24 query / 4 KV heads of 64, FFN 6912, vocabulary 10000, bf16, 128-token pages; prefill 4 x 512 tokens, then
    128 decode steps of 4 sequences.  The float model runs the reference's flow in stock torch; the quantized one
    has the 168 block projections and the vocabulary projection in W8A8 with every fusion this package offers."""
    from khaosz_amd import AutoRegressiveLM, LMConfig, fuse_shared_inputs, quantize_model

    dt = torch.bfloat16
    cfg = LMConfig(vocab_size=10000, dim=1536, n_layers=24, n_heads=24, n_kv_heads=4, dim_ffn=6912, max_len=2048)
    B, S, gen, page = 4, 512, 128, 128
    torch.manual_seed(11)
    model = AutoRegressiveLM(cfg).to(dev).to(dt).eval()
    P = (S + gen + page - 1) // page
    cache = model.new_cache(B * P, page)
    table = torch.arange(B * P, device=dev).view(B, P)  # pages handed out in order, as the benchmark's fresh pool does
    g = torch.Generator(device="cpu").manual_seed(12)
    prompt = torch.randint(0, cfg.vocab_size, (B, S), generator=g).to(dev)
    gen_ids = torch.randint(0, cfg.vocab_size, (B, gen), generator=g).to(dev)

    def prefill(i=0):
        return model(prompt, paged_cache=cache.bind(table, S), start_pos=0)["logits"]

    def decode_all(i=0):
        for t in range(gen):
            model(gen_ids[:, t:t + 1], paged_cache=cache.bind(table, S + t + 1), start_pos=S + t)

    def measure():
        pre_eager = eager_time_ms(torch, prefill, 5, 2)
        pre_spread = []
        pre_first = graph_time_ms(torch, prefill, 3, 1, dist=pre_spread)
        pre_graph = pre_spread[1]  # the median of 11 replays: a single replay of 3 prompts now and then catches a hiccup
        prefill()
        dec_eager = eager_time_ms(torch, decode_all, 2, 1) / gen
        dec_graph = graph_time_ms(torch, decode_all, 1, 1) / gen
        return {"prefill_ms": pre_graph, "prefill_ms_first_timed_replay": pre_first, "prefill_tok_s": B * S / (pre_graph * 1e-3),
                "prefill_eager_ms": pre_eager, "prefill_eager_tok_s": B * S / (pre_eager * 1e-3),
                "decode_ms_per_step": dec_graph, "decode_tok_s": B / (dec_graph * 1e-3),
                "decode_eager_ms_per_step": dec_eager, "decode_eager_tok_s": B / (dec_eager * 1e-3)}

    flt = measure()
    ref_logits = prefill().float()
    n = quantize_model(model, target_modules={"q_proj", "k_proj", "v_proj", "o_proj", "up", "gate", "down", "lm_head"})
    qsep = measure()  # quantized, every projection on its own and torch around them, as a drop-in gives
    fuse_shared_inputs(model, norms=True, decode_attention=True, residuals=True)
    q = measure()
    ql = prefill().float()
    err = ((ql - ref_logits).norm() / ref_logits.norm()).item()
    weight_bytes = sum(m.qweight.numel() for m in model.modules() if hasattr(m, "qweight"))
    return {
        "workload": "generation benchmark of the reference (24 x 1536, 24q/4kv x 64, ffn 6912, vocab 10000, bf16, "
                    "128-token pages): prefill 4 x 512, then 128 decode steps of 4 sequences; W8A8, all fusions, "
                    "HIP graph replay",
        "value": q["decode_tok_s"], "unit": "tok/s", "ms_per_step": q["decode_ms_per_step"], "dtype": "int8",
        "quantized_linears": n, "int8_weight_bytes": weight_bytes,
        "decode_weight_stream_gbs": weight_bytes / (q["decode_ms_per_step"] * 1e-3) / 1e9,
        "quantized_fused": q, "quantized_drop_in": qsep, "float_bf16_torch": flt,
        "prefill_logits_rel_err_vs_float": err,
        "speedup_decode_vs_float_graph": flt["decode_ms_per_step"] / q["decode_ms_per_step"],
        "speedup_prefill_vs_float_graph": flt["prefill_ms"] / q["prefill_ms"],
        "roofline": {}, "shape": (B, 0, 0),
    }


def measure_ceilings(torch, ops, dev, calibrate=True):
    """What this part delivers on trivial kernels (the lab library's probes, csrc/aq_lab.h):
      * an MFMA-only loop with constant operands (no bit toggling: the clock stays at its maximum) and with random
        operands that change every instruction (what a GEMM feeds the matrix cores), each with the shader clock
        the loop ran at: under matrix-core load with real data this part runs against its power limit;
      * a 1 GiB streaming read;
      * ONE launch reading 16 MiB (the size of the decode weight) from HBM, as a grid-stride loop and with every
        load of a lane issued before any is used (1 .. 16 loads of 16 bytes per lane, plain and streaming), over
        40 distinct buffers so that no launch finds its buffer in the last-level cache: no kernel of that size
        can beat the best of these;
      * an empty kernel: what a launch costs inside a replayed graph."""
    lab = ops._abi.load_lab()
    st = torch.cuda.current_stream().cuda_stream
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)

    def timed(fn, n):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(n):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / n

    def graph_us(launch, n=40):
        """n launches captured in one graph, replayed once untimed and once timed: us per launch."""
        for i in range(n):
            launch(i, st)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                for i in range(n):
                    launch(i, side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e3 / n
            best = t if best is None else min(best, t)
        return best

    out = {}
    iters = 20000  # a few ms per probe: long enough for the clock to settle under the load
    for kind, name, ops_per in ((0, "mfma_i8_32x32x32", 65536), (2, "mfma_fp8_32x32x64", 131072)):
        unit = "tops" if kind == 0 else "tflops"
        for data, tag in ((0, "constant_operands"), (1, "random_operands")):
            t = timed(lambda i=0: lab.aq_lab_probe_mfma(kind, data, 256, iters, sink.data_ptr(), clocks.data_ptr(), st), 2)
            c = clocks.tolist()
            out[f"{name}_{tag}_{unit}"] = 256 * 4 * iters * 8 * ops_per / t / 1e12
            out[f"{name}_{tag}_clock_mhz"] = c[0] / max(c[1], 1) * 100.0
    # fragment reads against the matrix pipe with one wavefront per SIMD, by placement (cycles per 32 MFMAs; 1024 = free)
    issue = {}
    for variant, label in ((0, "mfma_only"), (1, "one_read_behind_every_2nd_mfma"), (2, "eight_reads_first"),
                           (3, "pairs_behind_every_4th_mfma")):
        n_it = 2000
        lab.aq_lab_probe_mfma_lds_issue(variant, 256, 50, sink.data_ptr(), clocks.data_ptr(), st)
        lab.aq_lab_probe_mfma_lds_issue(variant, 256, n_it, sink.data_ptr(), clocks.data_ptr(), st)
        torch.cuda.synchronize()
        issue[label] = clocks.tolist()[0] / n_it
    out["cycles_per_32_mfma_with_16_ds_read_b128_one_wavefront_per_simd"] = issue
    big = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    t = timed(lambda i=0: lab.aq_lab_probe_read(big.data_ptr(), big.numel(), 0, 2048, 0, sink.data_ptr(), st), 3)
    out["hbm_stream_read_gbs"] = big.numel() / t / 1e9
    del big
    small = [torch.empty(16 << 20, dtype=torch.uint8, device=dev) for _ in range(40)]
    shots = {}
    for label, lpl, nt in (("grid_stride_2048_workgroups", 0, 0), ("upfront_1_load_per_lane", 1, 0),
                           ("upfront_4_loads_per_lane", 4, 0), ("upfront_8_loads_per_lane", 8, 0),
                           ("upfront_16_loads_per_lane", 16, 0), ("upfront_8_streaming_loads_per_lane", 8, 1),
                           ("upfront_16_streaming_loads_per_lane", 16, 1)):
        shots[label] = graph_us(lambda i, s, lpl=lpl, nt=nt: lab.aq_lab_probe_read(small[i % 40].data_ptr(), 16 << 20, lpl,
                                                                                   2048, nt, sink.data_ptr(), s))
    out["one_shot_16mib_read_us_by_variant"] = shots
    best = min(shots.values())
    out["one_shot_16mib_read_us"] = best
    out["one_shot_16mib_read_gbs"] = (16 << 20) / (best * 1e-6) / 1e9
    out["empty_kernel_in_graph_us"] = graph_us(lambda i, s: lab.aq_lab_probe_empty(sink.data_ptr(), s))
    del small
    if calibrate:  # launches GEMMs of other shapes: left out of single-workload (profiling) runs
        out["gemm_operand_data_and_stock_library"] = gemm_calibration(torch, ops, dev)
    return out


def gemm_calibration(torch, ops, dev):
    """Two calibrations of the GEMM figures, measured in the same run on the same box:
      * this library's int8 GEMM (fused epilogue, bf16 out) at 8192^3 on all-zero operands and on uniformly random
        codes: identical instruction streams; with zeros the shader clock stays near its maximum, with real data
        the part throttles to about 1.5 GHz (the MFMA-only probe above shows the same), so the first figure is the
        kernel's pipeline efficiency and the second what the power limit leaves of it;
      * the stock library behind torch (hipBLASLt) on the same operands: torch._int_mm (int8 -> int32, no epilogue)
        and torch._scaled_mm (e4m3 -> bf16) at 8192^3 and at the benchmark shapes of configurations 3 and 4.
    Eager launches timed with events (kernels of 20 us and more; the launch path is not the limit)."""
    def timed_us(fn, n):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    res = {}
    g = torch.Generator(device=dev).manual_seed(99)
    for (M, N, K, n) in ((8192, 8192, 8192, 5), (4096, 2048, 2048, 30)):
        ops_n = 2.0 * M * N * K
        tag = f"{M}x{N}x{K}"
        sx = torch.full((M,), 0.01, device=dev)
        sw = torch.full((N,), 0.001, device=dev)
        for name, lim in (("zero_operands", 0), ("random_operands", 127)):
            a = torch.randint(-lim, lim + 1, (M, K), generator=g, device=dev, dtype=torch.int8)
            b = torch.randint(-lim, lim + 1, (N, K), generator=g, device=dev, dtype=torch.int8)
            us = timed_us(lambda: ops.linear_w8a8(a, sx, b, sw, None, out_dtype=torch.bfloat16), n)
            res[f"this_library_int8_{tag}_{name}_tops"] = ops_n / us / 1e6
            try:
                us = timed_us(lambda: torch._int_mm(a, b.t()), n)
                res[f"stock_int_mm_{tag}_{name}_tops"] = ops_n / us / 1e6
            except Exception as e:  # the stock routine is a calibration only
                res[f"stock_int_mm_{tag}_{name}_tops"] = f"unavailable: {str(e)[:80]}"
            del a, b
    for (M, N, K, n) in ((8192, 8192, 8192, 5), (2048, 2048, 8192, 30)):
        flops = 2.0 * M * N * K
        tag = f"{M}x{N}x{K}"
        a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
        b = (torch.randn(N, K, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        aq_, sa = ops.quant_tensor_fp8(a)
        bq_, sb = ops.quant_tensor_fp8(b)
        us = timed_us(lambda: ops.linear_fp8(aq_, sa, bq_, sb, out_dtype=torch.bfloat16), n)
        res[f"this_library_fp8_{tag}_tflops"] = flops / us / 1e6
        try:
            a8, b8 = aq_.view(torch.float8_e4m3fn), bq_.view(torch.float8_e4m3fn)
            us = timed_us(lambda: torch._scaled_mm(a8, b8.t(), scale_a=sa.reshape(()), scale_b=sb.reshape(()),
                                                   out_dtype=torch.bfloat16), n)
            res[f"stock_scaled_mm_fp8_{tag}_tflops"] = flops / us / 1e6
        except Exception as e:
            res[f"stock_scaled_mm_fp8_{tag}_tflops"] = f"unavailable: {str(e)[:80]}"
        del a, b, aq_, bq_
    return res


def cpu_baseline(workload, shape, unit, per_step):
    """The C oracle on the same shape, on this host's cores.  Test infrastructure used as the
    reported baseline only: it never feeds the GPU path."""
    import numpy as np

    from oracle import oracle

    M, N, K = shape
    rng = np.random.default_rng(0)
    threads = oracle.c_num_threads()
    if workload == "fp8":
        Ms = 32  # bounded sample: 32 of the 2048 rows (scalar fp32 accumulation is slow)
        x = rng.standard_normal((Ms, K)).astype(np.float32)
        w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
        wq, sw = oracle.c_quant_tensor_fp8(w)
        t0 = time.perf_counter()
        xq, sx = oracle.c_quant_tensor_fp8(x)
        oracle.c_linear_fp8(xq, sx, wq, sw, bf16_out=True)
        dt = time.perf_counter() - t0
        val = 2.0 * Ms * N * K / dt / 1e12
        return {"value": val, "unit": unit, "cores": threads, "kind": "port",
                "sample": f"one pass over {Ms} of {M} rows (same N, K), {dt:.2f} s"}
    x = oracle.np_f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    wq, sw = oracle.c_quant_rowwise_i8(w)
    bias = None if workload == "decode" else (rng.standard_normal(N) * 0.01).astype(np.float32)
    oracle.c_linear_w8a8(x[: min(M, 64)], wq, sw, bias, x_bf16_bits=True, bf16_out=True)  # warm the threads
    reps, t_total = 0, 0.0
    budget = 10.0  # seconds of CPU work per leg
    while t_total < budget and reps < 20000:
        t0 = time.perf_counter()
        oracle.c_linear_w8a8(x, wq, sw, bias, x_bf16_bits=True, bf16_out=True)
        t_total += time.perf_counter() - t0
        reps += 1
    dt = t_total / reps
    scale = 1e9 if unit == "GB/s" else 1e12
    return {"value": per_step / dt / scale, "unit": unit, "cores": threads, "kind": "port",
            "sample": f"{reps} full passes of the same shape (quantise + int8 GEMM + epilogue), {dt * 1e3:.2f} ms each",
            "reference_float_path": float_linear_cpu(M, N, K, bias is not None)}


def float_linear_cpu(M, N, K, with_bias):
    """The reference's own arithmetic for this call, F.linear (astrai/model/components/linear.py:21),
    on the host in fp32 and bf16: a float GEMM by the vendor BLAS, not the quantized path."""
    import torch
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(0)
    x = torch.randn(M, K, generator=g)
    w = torch.randn(N, K, generator=g) * 0.02
    b = torch.randn(N, generator=g) * 0.01 if with_bias else None
    out = {"threads": torch.get_num_threads()}
    for name, dt in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        xx, ww, bb = x.to(dt), w.to(dt), (b.to(dt) if b is not None else None)
        with torch.inference_mode():
            F.linear(xx, ww, bb)
            reps, t_total = 0, 0.0
            while t_total < 2.0 and reps < 200:
                t0 = time.perf_counter()
                F.linear(xx, ww, bb)
                t_total += time.perf_counter() - t0
                reps += 1
        out[name + "_ms"] = t_total / reps * 1e3
    return out


def main():
    t_start = time.time()
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported in this build "
              "(no collectives or sharding are part of it)", file=sys.stderr)
        sys.exit(2)
    import torch

    from khaosz_amd import ops

    ops._abi.load()  # fails loudly when the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    fns = {"decode": bench_decode, "prefill": bench_prefill, "fp8": bench_fp8, "block": bench_block,
           "model": bench_model}
    with torch.inference_mode():
        # the part's own ceilings first: the roofline objects of the workloads quote them
        CEIL.update(measure_ceilings(torch, ops, dev, calibrate=False))
        main_res = fns[args.workload](torch, ops, args, dev)
        extra = {}
        if not args.no_extra:
            for name in ("decode", "prefill", "fp8", "block"):  # "model" only on request: it takes a minute
                if name != args.workload:
                    extra[name] = fns[name](torch, ops, args, dev)
            if args.workload == "decode":
                for m in (1, 4):
                    a2 = argparse.Namespace(**vars(args))
                    a2.m = m
                    r = bench_decode(torch, ops, a2, dev)
                    extra[f"decode_m{m}"] = r
                extra["batch_32_to_256"] = bench_few_dozen_rows(torch, ops, args, dev)
        ceilings = dict(CEIL)
        if not args.no_extra:  # launches GEMMs of other shapes: left out of single-workload (profiling) runs
            ceilings["gemm_operand_data_and_stock_library"] = gemm_calibration(torch, ops, dev)
        if not args.no_extra and args.workload != "model":
            # the reference's own generation benchmark: about a minute; skipped when this run is already long
            if time.time() - t_start < 150:
                m = bench_model(torch, ops, args, dev)
                extra["model"] = {k: m[k] for k in ("workload", "value", "unit", "ms_per_step", "dtype", "quantized_linears",
                                                     "int8_weight_bytes", "decode_weight_stream_gbs", "quantized_fused",
                                                     "quantized_drop_in", "float_bf16_torch", "prefill_logits_rel_err_vs_float",
                                                     "speedup_decode_vs_float_graph", "speedup_prefill_vs_float_graph")}
            else:
                extra["model"] = {"skipped": "time budget of the default run spent"}
    per_step = main_res.get("bytes_per_step") or main_res.get("ops_per_step") or main_res.get("flops_per_step")
    cpu = None
    if not args.no_cpu and args.workload not in ("block", "model"):
        cpu = cpu_baseline(args.workload, main_res["shape"], main_res["unit"], per_step)
        if not args.no_extra and "prefill" in extra:
            # one pass of the prefill shape as well, so both halves of the metric have a CPU figure
            extra["prefill"]["cpu_baseline"] = cpu_baseline("prefill", extra["prefill"]["shape"], "TOPS",
                                                            extra["prefill"]["ops_per_step"])
    for r in [main_res, *extra.values()]:
        r.pop("shape", None)
    top = ("workload", "value", "unit", "ms_per_step", "dtype", "roofline", "eager_ms_per_step")
    detail = {k: v for k, v in main_res.items() if k not in top} if args.workload in ("block", "model") else None
    line = {
        "metric": METRIC, "value": main_res["value"], "unit": main_res["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": main_res["unit"] != "ms", "scaling": "weak", "vs_baseline": None, "dtype": main_res["dtype"],
        "data": "synthetic", "config": {"workload": main_res["workload"], "timing": "HIP graph replay of the timed steps",
                                        "eager_ms_per_step": main_res.get("eager_ms_per_step"),
                                        "replay_ms_per_step_p10_p50_p90": main_res.get("ms_per_step_p10_p50_p90"),
                                        **({"detail": detail} if detail else {})},
        "roofline": main_res["roofline"], "cpu_baseline": cpu, "measured_ceilings": ceilings,
        "also": {k: {kk: vv for kk, vv in v.items()} for k, v in extra.items()},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the TW-Marlin W4A16 decode path on one MI355X.

Workload: the four M=1 GEMVs of a Qwen-7B-shaped layer
    qkv 3584->4608, o 3584->3584, gate_up 3584->37888, down 18944->3584
group-32 Q4 weights + FP16 scales, FP16 activations, FP32 outputs.  One "step" = one layer.
Several distinct layers (default 4, 525 MB of weights) are walked in turn so that the 256 MB
Infinity Cache cannot hold the working set and the rate is an HBM rate.  The layer sequence is
captured once as a hipGraph (the reference captures all layers of a decode step in one graph,
crates/kernels/src/generate.rs:2485-2536) and replayed; `config.us_per_layer_own_graph` is the
same measurement with one graph per layer, which pays the graph-launch cost once per layer.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--no-cpu] [--no-prefill] [--no-lm-head] [--extra]

`small_shapes_m1` holds the launch-bound configurations (4096->4096 and the Qwen-0.5B layer) per
projection and as a graph, `prefill` the W4A16 GEMM on the LLaMA-7B MLP shapes at M=512 and
2048 as TFLOP/s against the 2.5 PFLOP/s dense FP16 MFMA peak; it is not part of `value`.

Prints ONE JSON line. `value` = algorithmic bytes of a layer x K / time of K replays (inputs
resident in HBM). `roofline` is for the dominant kernel, the gate_up GEMV, timed with HIP events
on the stream it runs on. `cpu_baseline` is the CPU oracle (a port of the reference's CPU
semantics: TW-Marlin unpack to dense f32, then the naive cpu_gemm loop) on one layer, one thread.
"""
import argparse
import json
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense FP16 matrix, published

LAYER_7B = [("qkv", 3584, 4608), ("o", 3584, 3584), ("gate_up", 3584, 37888), ("down", 18944, 3584)]
LAYER_05B = [("qkv", 896, 1152), ("o", 896, 896), ("gate_up", 896, 9728), ("down", 4864, 896)]   # Qwen-0.5B layer
CFG0 = [("cfg0", 4096, 4096)]                                                                     # the single-GEMV configuration
# HBM bytes per gate_up launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by
# what the same counter reads for a 64 MiB copy (profiles/k_gemv4s_gate_up_m1_hbm_traffic.md).
GATE_UP_TRAFFIC_BYTES = 76647700


def algo_bytes(k, n, m=1):
    """K*N/2 nibbles + (K/32)*N*2 scales + M*K*2 FP16 activations + M*N*4 FP32 outputs"""
    return k * n // 2 + (k // 32) * n * 2 + m * k * 2 + m * n * 4


def make_layer(rng, shapes):
    host = {}
    for name, k, n in shapes:
        packed = rng.integers(0, 256, size=(k // 32) * n * 16, dtype=np.uint8)          # nibbles uniform 0..15
        scales = (np.abs(rng.standard_normal((k // 32) * n, dtype=np.float32)) * np.float32(0.02)).astype(np.float16)
        act = rng.standard_normal(k, dtype=np.float32).astype(np.float16)               # f16(N(0,1))
        host[name] = (packed, scales.view(np.uint16), act.view(np.uint16))
    return host


class VendorGemm:
    """rocBLAS gemm_ex (f16 x f16 -> f32, f32 accumulation) on the context's stream, through ctypes: a
    yardstick for the prefill kernel, not part of the product.  Row-major C[M,N] = A[M,K] W[K,N] is the
    column-major product C^T = W^T A^T, so W goes in as the first operand with leading dimension N."""
    OP_NONE, F16_R, F32_R, ALGO_STANDARD = 111, 150, 151, 0

    def __init__(self, dev):
        import ctypes as C
        self.C, self.dev, self.ok = C, dev, False
        try:
            self.lib = C.CDLL("librocblas.so")
            self.handle = C.c_void_p()
            if self.lib.rocblas_create_handle(C.byref(self.handle)) != 0:
                return
            if self.lib.rocblas_set_stream(self.handle, C.c_void_p(dev._l.twm_ctx_stream(dev.handle))) != 0:
                return
            self.lib.rocblas_gemm_ex.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                                 C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                                                 C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                                 C.c_int, C.c_int32, C.c_uint32]
            self.ok = True
        except OSError:
            pass

    def time(self, a, w16, c, m, n, k, reps):
        C = self.C
        alpha, beta = C.c_float(1.0), C.c_float(0.0)

        def call(i):
            return self.lib.rocblas_gemm_ex(self.handle, self.OP_NONE, self.OP_NONE, n, m, k, C.byref(alpha),
                                            w16.ptr, self.F16_R, n, a.ptr, self.F16_R, k, C.byref(beta),
                                            c.ptr, self.F32_R, n, c.ptr, self.F32_R, n, self.F32_R, self.ALGO_STANDARD, 0, 0)
        if call(0) != 0:
            return None
        for i in range(3):
            call(i)
        self.dev.synchronize()
        return time_launches(self.dev, call, reps)


def time_launches(dev, fn, reps, settle_ms=25.0):
    """average milliseconds per call of fn() over `reps` calls, HIP events on the context's stream.  The timed
    run follows about `settle_ms` of the same launches, untimed: after a section of short kernels the first
    few hundred launches of a long one run several per cent slower than its steady state."""
    def run(count):
        e0, e1 = dev.event(), dev.event()
        dev.record(e0)
        for i in range(count):
            fn(i)
        dev.record(e1)
        ms = dev.elapsed_ms(e0, e1)
        dev.event_destroy(e0)
        dev.event_destroy(e1)
        return ms
    if settle_ms > 0:
        first = run(reps)
        more = int(min(4000, max(0.0, settle_ms - first) / max(first / reps, 1e-4)))
        more -= more % 8            # keep the rotation over weight sets aligned
        if more:
            run(more)
    return run(reps) / reps


def trace_decode(T, dev, layers):
    """The layer's four GEMVs at M = 1, launched one after the other as in the layer, with every workgroup writing
    the GPU's 100 MHz clock at its start, when its first wave has its weights unpacked, and at its end
    (twm_debug_trace).  Prints, per projection: the gap since the previous kernel's last workgroup ended, when the
    first data was there, the span from first start to last end, and the bytes of finished workgroups per microsecond."""
    cap, slots = 4096, 48
    trace = T.GpuTensor.zeros(dev, (slots * cap * 4,), "i32")
    order = [name for name, _, _ in LAYER_7B]
    shape = {name: (k, n) for name, k, n in LAYER_7B}

    def launch(i, traced):
        name = order[i % 4]
        w, a, c = layers[(i // 4) % len(layers)][name]
        if traced:
            dev._l.twm_debug_trace(dev.handle, trace.ptr + (i % slots) * cap * 16, cap)
        T.gemm(dev, w, a, 1, c)
    for i in range(4000):
        launch(i, False)
    dev.synchronize()
    for i in range(slots):
        launch(i, True)
    dev.synchronize()
    dev._l.twm_debug_trace(dev.handle, None, 0)
    t = trace.to_host().view(np.uint32).reshape(slots, cap, 4)
    rows = {name: [] for name in order}
    prev_end = None
    for i in range(slots):
        x = t[i][t[i][:, 2] != 0]
        st, ld, en = x[:, 0].astype(np.int64), x[:, 1].astype(np.int64), x[:, 2].astype(np.int64)
        s0 = st.min()
        hw = x[:, 3]
        cus = len(np.unique(((hw >> 16) & 0xF) * 4096 + ((hw >> 8) & 0xFF)))   # XCD, then SE / SH / CU bits of HW_ID
        k, n = shape[order[i % 4]]
        per_wg = algo_bytes(k, n) / len(x)
        ends = np.sort((en - s0) / 100.0)
        span = ends[-1]
        # steady rate: between the moment 10 % and the moment 90 % of the workgroups have ended
        lo, hi = ends[int(0.1 * len(x))], ends[int(0.9 * len(x)) - 1]
        steady = 0.8 * len(x) * per_wg / max(hi - lo, 1e-9) / 1e6 if len(x) >= 512 else float("nan")
        if i >= 8:   # (the first launches after the switch to the traced kernels are left out)
            rows[order[i % 4]].append((len(x), cus, (s0 - prev_end) / 100.0 if prev_end is not None else float("nan"),
                                       (st.max() - s0) / 100.0, (ld[ld > 0].min() - s0) / 100.0, (ld[ld > 0] - st[ld > 0]).mean() / 100.0,
                                       ends[0], span, (en - st).mean() / 100.0, steady))
        prev_end = en.max()
    print("| projection | workgroups | CUs used | gap since the previous kernel's last end | last workgroup starts | first wave unpacked | "
          "start to unpacked (mean) | first workgroup ends | span (first start to last end) | workgroup lifetime (mean) | "
          "rate between 10 % and 90 % of the workgroups done |")
    print("|---|---|---|---|---|---|---|---|---|---|---|")
    for name in order:
        r = np.array(rows[name], dtype=np.float64)
        m = np.array([np.nanmean(r[:, j]) if np.isfinite(r[:, j]).any() else float("nan") for j in range(r.shape[1])])
        k, n = shape[name]
        print("| %s %d -> %d | %d | %d | %.2f us | %.2f us | %.2f us | %.2f us | %.2f us | %.2f us | %.2f us | %s |" % (
            name, k, n, m[0], m[1], m[2], m[3], m[4], m[5], m[6], m[7], m[8],
            ("%.2f TB/s" % m[9]) if np.isfinite(m[9]) else "-"))
    tot = sum(np.nanmean(np.array(rows[nm])[:, 2]) + np.nanmean(np.array(rows[nm])[:, 7]) for nm in order)
    print("\nsum of gaps and spans: %.2f us per layer (traced kernels, eager launches)" % tot)
    for name in order:
        k, n = shape[name]
        m = np.array(rows[name], dtype=np.float64).mean(axis=0)
        print("%s: %.1f MB in a span of %.2f us = %.2f TB/s inside the kernel" % (name, algo_bytes(k, n) / 1e6, m[7], algo_bytes(k, n) / m[7] / 1e6))


def mfma_mix(dev):
    """FP16 matrix throughput under the instruction mixes of a W4A16 prefill block (twm_debug_mfma_mix): the ceilings
    the prefill kernel's arrangement was chosen against.  Median of five timed launches per line."""
    import ctypes as C
    steps = 8192

    def run(form, parts, per_cu):
        vals = []
        for i in range(7):     # (the first two settle the clock)
            tf = C.c_float(0.0)
            rc = dev._l.twm_debug_mfma_mix(dev.handle, form, parts, per_cu, steps, C.byref(tf))
            assert rc == 0, dev._l.twm_last_error()
            if i >= 2:
                vals.append(tf.value)
        return sorted(vals)[2]
    rows = [
        (0, 0, "one wave per tile column: the 32 MFMAs of a step alone"),
        (0, 1, "... + the Q4 unpack of the next step's four B operands (52 vector instructions)"),
        (0, 3, "... + eight ds_read_b128 (the A operands)"),
        (0, 7, "... + four global_load_dwordx4 (nibbles, scales, the A tile's direct loads)"),
        (0, 15, "... + four ds_write_b128 (an A tile staged through registers)"),
    ]
    print("| instruction mix per 32-deep step and MFMA-issuing wave | one workgroup of four waves per CU | two per CU |")
    print("|---|---|---|")
    for form, parts, text in rows:
        one, two = run(form, parts, 1), run(form, parts, 2)
        print("| %s | %.0f TFLOP/s (%.1f %% of 2.5 PFLOP/s) | %.0f TFLOP/s (%.1f %%) |" % (text, one, one / 25.0, two, two / 25.0))
    print()
    print("| producers and consumers: eight waves per workgroup, one per CU, 64-deep intervals, one barrier each | TFLOP/s |")
    print("|---|---|")
    for parts, text in ((0, "four waves issue MFMAs on operands in registers; four waves only load nibbles"),
                        (2, "... the MFMA waves read their eight A operands per step from LDS"),
                        (18, "... and their four B operands per step too (twelve ds_read_b128 per 32 MFMAs)"),
                        (19, "... and the other four waves unpack the nibbles and write the f16 B tile to LDS")):
        v = run(1, parts, 1)
        print("| %s | %.0f (%.1f %% of 2.5 PFLOP/s) |" % (text, v, v / 25.0))


def profiler_attached():
    """True when a rocprofiler tool library is preloaded into this process (rocprofv3 does that).  Under it the
    bench issues every launch eagerly: rocprofv3 has crashed on the host inside hipGraphLaunch on this bench's
    longer graphs, and a kernel trace reads per-kernel durations, which do not need graphs."""
    import os
    if any("rocprof" in os.environ.get(key, "").lower() for key in ("LD_PRELOAD", "HSA_TOOLS_LIB", "ROCP_TOOL_LIB")):
        return True
    return any(key.startswith(("ROCPROF", "ROCPROFILER")) for key in os.environ)


class EagerGraph:
    """Stands in for a captured graph when graphs are off: replay() issues the launches one by one."""
    def __init__(self, fn):
        self.fn = fn

    def replay(self):
        self.fn()

    def destroy(self):
        pass


def sampled_prefill_rel_err(got, packed, scales, a16, m, k, n, rng):
    """max relative error (floor: 1e-3 of the largest compared output) of a prefill result against the f64 product on
    the FP16 Q4 unpack f16(f32(scale) * (q - 8)), restated here in numpy, on all rows of 256 sampled columns (the
    first and last among them).  Returns (error, number of columns)."""
    g = k // 32
    cols = np.unique(np.concatenate([rng.integers(0, n, 254), [0, n - 1]]))
    rec = packed.reshape(g, n, 16)[:, cols, :]                                # [G, C, 16]
    q = np.empty((g, len(cols), 32), np.float32)
    q[:, :, 0::2] = (rec & 0xF).astype(np.float32) - 8.0                      # low nibble = even k
    q[:, :, 1::2] = (rec >> 4).astype(np.float32) - 8.0
    sc = scales.view(np.float16).reshape(g, n)[:, cols].astype(np.float32)   # [G, C]
    w = (q * sc[:, :, None]).astype(np.float16)                               # f16_rne(scale * (q - 8))
    w = w.transpose(0, 2, 1).reshape(k, len(cols)).astype(np.float64)         # [K, C]
    t = a16.view(np.float16).reshape(m, k).astype(np.float64) @ w
    e = np.abs(got.reshape(m, n)[:, cols] - t) / np.maximum(np.abs(t), 1e-3 * np.abs(t).max())
    return float(e.max()), int(len(cols))


def time_short_launches(dev, T, fn, reps, keep, below_ms=8e-3):
    """As time_launches; a call that takes under `below_ms` is timed again as one captured graph of `reps`
    calls, because issuing launches one by one from Python (about 5 us each; a call with split-K is two)
    can be slower than the kernels run.  Returns (ms per call, "eager" | "graph")."""
    ms = time_launches(dev, fn, reps)
    if ms >= below_ms:
        return ms, "eager"

    def body():
        for i in range(reps):
            fn(i)
    if T is None:       # graphs are off (a profiler is attached): the eager figure stands
        return ms, "eager"
    g = T.GraphCapture.record_with_device(dev, body)
    keep.append(g)
    g.replay()
    dev.synchronize()
    return min(ms, time_launches(dev, lambda i: g.replay(), 4) / reps), "graph"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=8, help="distinct weight sets rotated through (8 x 131 MB: four times the 256 MB cache)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill GEMM timings")
    ap.add_argument("--no-lm-head", action="store_true", help="skip the LM-head GEMV + argmax timing")
    ap.add_argument("--no-swiglu", action="store_true", help="skip the fused gate_up + SwiGLU timing")
    ap.add_argument("--no-moe", action="store_true", help="skip the expert-bank (MoE decode) timing")
    ap.add_argument("--no-vendor-gemm", action="store_true",
                    help="skip timing rocBLAS' dense FP16 GEMM beside the prefill kernel")
    ap.add_argument("--no-batched", action="store_true", help="skip the batched-decode layer (M = 4 .. 32)")
    ap.add_argument("--no-tune", action="store_true", help="skip the layer with measured plans (twm_weight_tune)")
    ap.add_argument("--batched-eager", action="store_true",
                    help="batched-decode layer without graph capture (rocprofv3 has crashed in hipGraphLaunch of graphs this long)")
    ap.add_argument("--eager", action="store_true",
                    help="no graph capture anywhere: every launch is issued one by one (forced when a rocprofiler tool is preloaded)")
    ap.add_argument("--no-small", action="store_true", help="skip the small configurations (Qwen-0.5B layer, 4096 x 4096)")
    ap.add_argument("--sweep-splits", action="store_true",
                    help="also time every projection at M=1,4,8,16,32 with forced split-K factors next to the library's "
                         "own choice (batched decode configuration)")
    ap.add_argument("--sweep-prefill", action="store_true",
                    help="also time the prefill GEMM at M = 128 .. 2048 with the library's own block height and split-K "
                         "against forced ones")
    ap.add_argument("--sweep-models", action="store_true",
                    help="also time the projections of other model sizes (Llama-3-8B, 13B, 70B, Qwen-1.5B shapes) at "
                         "M = 1, 4, 8, 16 with the library's plan against the 64-column / streaming kernels alone")
    ap.add_argument("--pmc-copy", action="store_true",
                    help="also run four 64 MiB device-to-device copies: a kernel of known traffic to scale rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings by")
    ap.add_argument("--mfma-mix", action="store_true",
                    help="print what the matrix pipes deliver under the instruction mixes of a prefill block "
                         "(twm_debug_mfma_mix), as a markdown table, and exit")
    ap.add_argument("--trace-decode", action="store_true",
                    help="instead of the timings: run the four M = 1 GEMVs of the layer with the library's per-workgroup "
                         "clock trace (twm_debug_trace) and print where each launch's time goes, as a markdown table")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding)" % args.gpus)

    import tensorwarp_amd as T

    graphs_off = args.eager or profiler_attached()
    if graphs_off:
        print("[bench] graphs are off: every launch is issued eagerly%s" % (" (rocprofiler tool preloaded)" if not args.eager else ""),
              file=sys.stderr, flush=True)
    T_graphs = None if graphs_off else T     # what time_short_launches captures with

    def capture(fn):
        return EagerGraph(fn) if graphs_off else T.GraphCapture.record_with_device(dev, fn)

    dev = T.WarpDevice(0)
    rng = np.random.default_rng(20250101)
    graphs_done = []        # graphs stay alive until the end: nothing is destroyed between timed sections

    def log(section):       # progress on stderr: a run that dies names the section it died in
        print("[bench] " + section, file=sys.stderr, flush=True)
    layers_host = [make_layer(rng, LAYER_7B) for _ in range(args.layers)]
    layers = []
    for host in layers_host:
        entry = {}
        for name, k, n in LAYER_7B:
            packed, scales, act = host[name]
            entry[name] = (T.MarlinWeight.upload(dev, packed, scales, k, n),
                           T.GpuTensor.from_host(dev, act, "f16"),
                           T.GpuTensor.zeros(dev, (n,), "f32"))
        layers.append(entry)

    def run_layer(li):
        entry = layers[li]
        for name, k, n in LAYER_7B:
            w, a, c = entry[name]
            T.gemm(dev, w, a, 1, c)

    if args.trace_decode:
        trace_decode(T, dev, layers)
        return
    if args.mfma_mix:
        mfma_mix(dev)
        return

    if args.pmc_copy:
        # kernels of known traffic to scale counter readings by: a device-to-device copy of 64 MiB (a kernel only when
        # the runtime does not hand it to a copy engine), a fill kernel that writes 64 MiB, and an argmax over one row of
        # 16 Mi floats, which reads 64 MiB
        src = T.GpuTensor.zeros(dev, (64 << 20,), "u8")
        dst = T.GpuTensor.zeros(dev, (64 << 20,), "u8")
        row = T.GpuTensor.zeros(dev, (1, 16 << 20), "f32")
        idx = T.GpuTensor.zeros(dev, (1,), "i32")
        for _ in range(4):
            dev._l.twm_memcpy_d2d(dev.handle, dst.ptr, src.ptr, 64 << 20)
            dev._l.twm_memset_zero(dev.handle, dst.ptr, 64 << 20)
            T.argmax(dev, row, idx, 1, 16 << 20)
        dev.synchronize()

    log("decode layer: warm-up and graphs")
    # eager warm-up (also loads every code object before capture), then the graphs
    for li in range(args.layers):
        run_layer(li)
    dev.synchronize()
    L = args.layers
    steps, warmup = max(1, args.steps), max(0, args.warmup)

    def run_all():
        for li in range(L):
            run_layer(li)

    # one graph over all L distinct layers; K steps = K // L replays of it plus one replay of a graph over the
    # first K % L layers, so that exactly K steps are timed whatever K is
    graph_all = capture(run_all)
    graph_rest = {}

    def run_steps(count):
        for _ in range(count // L):
            graph_all.replay()
        rest = count % L
        if rest:
            if rest not in graph_rest:
                graph_rest[rest] = capture(lambda rest=rest: [run_layer(li) for li in range(rest)])
            graph_rest[rest].replay()

    def timed_window(count):
        e0, e1 = dev.event(), dev.event()
        dev.synchronize()
        dev.record(e0)
        run_steps(count)
        dev.record(e1)
        ms = dev.elapsed_ms(e0, e1)
        dev.synchronize()
        dev.event_destroy(e0)
        dev.event_destroy(e1)
        return ms / count

    run_steps(steps)                     # (captures the remainder graph outside any timed window)
    run_steps(warmup)
    dev.synchronize()
    t0 = time.perf_counter()
    # at least five windows of exactly K steps each, and at least ~800 steps in all; the headline is the median
    n_windows = max(5, min(50, (800 + steps - 1) // steps))
    windows = sorted(timed_window(steps) for _ in range(n_windows))
    ms_step = windows[len(windows) // 2]
    ms_step_min = windows[0]
    wall = time.perf_counter() - t0

    graphs = [capture(lambda li=li: run_layer(li)) for li in range(L)]
    for i in range(max(warmup, L)):
        graphs[i % L].replay()
    dev.synchronize()
    ms_step_own = time_launches(dev, lambda i: graphs[i % L].replay(), max(steps, 8 * L))
    dev.synchronize()

    layer_bytes = sum(algo_bytes(k, n) for _, k, n in LAYER_7B)
    value = layer_bytes / (ms_step * 1e-3) / 1e9

    log("per-projection timings")
    # per-projection timings, eager launches rotating over the distinct layers
    per_shape = {}
    for name, k, n in LAYER_7B:
        def one(i, name=name):
            w, a, c = layers[i % args.layers][name]
            T.gemm(dev, w, a, 1, c)
        for i in range(20):
            one(i)
        dev.synchronize()
        ms, how = time_short_launches(dev, T_graphs, one, 200, graphs_done)
        windows = [ms]
        if how == "eager":
            # five timed windows of 200 launches each, the median one counts (a single window scatters by 3 - 5 %)
            windows += [time_launches(dev, one, 200, settle_ms=0.0) for _ in range(4)]
            ms = sorted(windows)[len(windows) // 2]
        b = algo_bytes(k, n)
        per_shape[name] = {"k": k, "n": n, "us": round(ms * 1e3, 3), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                           "frac_hbm": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "timed": how,
                           "timed_windows": len(windows), "us_min": round(min(windows) * 1e3, 3),
                           "us_max": round(max(windows) * 1e3, 3), "plan": dev.plan(k, n, 1)}

    log("drop-in on the reference layout")
    # the literal drop-in: gemm_tw_marlin_m1 on the reference's arrays (no repack), f32 activations
    drop_in = {}
    for name, k, n in LAYER_7B:
        sets = []
        for li in range(args.layers):
            packed, scales, act = layers_host[li][name]
            sets.append((T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales, "f16")))
        a32 = T.GpuTensor.from_host(dev, layers_host[0][name][2].view(np.float16).astype(np.float32))
        c32 = T.GpuTensor.zeros(dev, (n,), "f32")

        def one(i, sets=sets, a32=a32, c32=c32, n=n, k=k):
            p_, s_ = sets[i % args.layers]
            T.gemm_tw_marlin_m1(dev, a32, p_, s_, c32, n, k)
        for i in range(8):
            one(i)
        dev.synchronize()
        ms, how = time_short_launches(dev, T_graphs, one, 104, graphs_done)
        b = k * n // 2 + (k // 32) * n * 2 + k * 4 + n * 4
        drop_in[name] = {"us": round(ms * 1e3, 2), "GBps": round(b / (ms * 1e-3) / 1e9, 1), "timed": how, "plan": dev.plan_m1(k, n)}
        one(0)                                             # layer 0 again, for the comparison
        w, a, c = layers[0][name]
        T.gemm(dev, w, a, 1, c)
        ref = c.to_host()
        assert np.abs(c32.to_host() - ref).max() <= 1e-4 * np.abs(ref).max(), "drop-in differs from the repacked path"
        for p_, s_ in sets:
            p_.free()
            s_.free()
    drop_in["layer_us"] = round(sum(v["us"] for v in drop_in.values()), 2)


    log("f32 activations on the repacked handles")
    # what a caller gets that keeps the reference's f32 activation buffers (twm_gemm with TWM_F32): per projection, and the
    # layer as one graph over the rotating layers
    f32_rows = {}
    a32s = {name: T.GpuTensor.from_host(dev, layers_host[0][name][2].view(np.float16).astype(np.float32)) for name, k, n in LAYER_7B}
    for name, k, n in LAYER_7B:
        def one(i, name=name):
            w, _, c = layers[i % args.layers][name]
            T.gemm(dev, w, a32s[name], 1, c)
        for i in range(8):
            one(i)
        dev.synchronize()
        ms, how = time_short_launches(dev, T_graphs, one, 104, graphs_done)
        b = k * n // 2 + (k // 32) * n * 2 + k * 4 + n * 4
        f32_rows[name] = {"us": round(ms * 1e3, 2), "GBps": round(b / (ms * 1e-3) / 1e9, 1), "timed": how}

    def run_all_f32():
        for li in range(L):
            for name, k, n in LAYER_7B:
                T.gemm(dev, layers[li][name][0], a32s[name], 1, layers[li][name][2])
    if not graphs_off:
        g32 = capture(run_all_f32)
        for _ in range(3):
            g32.replay()
        dev.synchronize()
        f32_rows["layer_us"] = round(time_launches(dev, lambda i: g32.replay(), max(8, steps // L)) / L * 1e3, 2)
        graphs_done.append(g32)
    else:
        f32_rows["layer_us"] = round(sum(v["us"] for v in f32_rows.values()), 2)

    gu = per_shape["gate_up"]
    gu_bytes = algo_bytes(3584, 37888)
    roofline = {"bound": "hbm", "kernel": "k_gemv4s (gate_up 3584->37888, M=1)",
                "achieved": gu["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gu["GBps"] / HBM_PEAK_GBS, 4),
                "bytes_per_launch": gu_bytes, "us_per_launch": gu["us"],
                "us_per_launch_is": "median of %d timed windows of 200 launches (min %.3f, max %.3f)" % (
                    gu["timed_windows"], gu["us_min"], gu["us_max"]),
                "traffic": GATE_UP_TRAFFIC_BYTES,
                "traffic_source": "not measured by this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel, "
                                  "profiles/k_gemv4s_gate_up_m1_hbm_traffic.md"}

    extra = {}
    if not args.no_batched:
        log("batched decode")
        # the same layer at M = 4 .. 32 f16 rows: one graph of the four projections over the rotating layers
        for m in (4, 8, 16, 32):
            bufs = {name: (T.GpuTensor.from_host(dev, rng.standard_normal((m, k), dtype=np.float32).astype(np.float16).view(np.uint16), "f16"),
                           T.GpuTensor.zeros(dev, (m, n), "f32")) for name, k, n in LAYER_7B}

            def run_rows(m=m, bufs=bufs):
                for li in range(L):
                    for name, k, n in LAYER_7B:
                        T.gemm(dev, layers[li][name][0], bufs[name][0], m, bufs[name][1])
            run_rows()
            dev.synchronize()
            if args.batched_eager:      # for a kernel trace: launches issued one by one (the host then sets the pace)
                ms = time_launches(dev, lambda i: run_rows(), max(4, steps // L // 4)) / L
            else:
                g_rows = capture(run_rows)
                ms = time_launches(dev, lambda i: g_rows.replay(), max(4, steps // L // 4)) / L
                graphs_done.append(g_rows)
            lb = sum(algo_bytes(k, n, m) for _, k, n in LAYER_7B)
            extra["layer_M%d" % m] = {"us": round(ms * 1e3, 2), "GBps": round(lb / (ms * 1e-3) / 1e9, 1),
                                      "frac_hbm": round(lb / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    # the same layer once more with measured plans: twm_weight_tune times the launch forms per weight and row count and
    # keeps what beats the planners' choice by more than 2 % (the role of the reference's autotune table)
    tuned = None
    if not args.no_batched and not args.no_tune:
        log("decode layer with measured plans")
        t0 = time.time()
        for li in range(L):
            for name, k, n in LAYER_7B:
                layers[li][name][0].tune([1, 4, 8, 16, 32])
        tuned = {"tune_seconds": round(time.time() - t0, 2),
                 "plans_layer0": {name: {"M%d" % m: layers[0][name][0].tuned_plan(m) for m in (1, 4, 8, 16, 32)} for name, _, _ in LAYER_7B}}
        for m in (1, 4, 8, 16, 32):
            bufs = {name: (T.GpuTensor.from_host(dev, rng.standard_normal((m, k), dtype=np.float32).astype(np.float16).view(np.uint16), "f16"),
                           T.GpuTensor.zeros(dev, (m, n), "f32")) for name, k, n in LAYER_7B}

            def run_rows(m=m, bufs=bufs):
                for li in range(L):
                    for name, k, n in LAYER_7B:
                        T.gemm(dev, layers[li][name][0], bufs[name][0], m, bufs[name][1])
            run_rows()
            dev.synchronize()
            g_rows = capture(run_rows)
            ms = time_launches(dev, lambda i: g_rows.replay(), max(4, steps // L // 4)) / L
            graphs_done.append(g_rows)
            lb = sum(algo_bytes(k, n, m) for _, k, n in LAYER_7B)
            tuned["layer_M%d" % m] = {"us": round(ms * 1e3, 2), "GBps": round(lb / (ms * 1e-3) / 1e9, 1),
                                      "frac_hbm": round(lb / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    log("small configurations")
    # the small configurations: launch- and latency-bound, reported per projection and as one graph per layer
    small = {}
    for label, shapes in (() if args.no_small else (("qwen05b", LAYER_05B), ("cfg0", CFG0))):
        sets = []
        for _ in range(8):                                   # 8 x 9.4 MB: still inside the 256 MB cache, as in a real
            host = make_layer(rng, shapes)                   # 0.5B model (all weights 250 MB) these shapes would be
            sets.append({name: (T.MarlinWeight.upload(dev, host[name][0], host[name][1], k, n),
                                T.GpuTensor.from_host(dev, host[name][2], "f16"),
                                T.GpuTensor.zeros(dev, (n,), "f32")) for name, k, n in shapes})
        entry = {}
        for name, k, n in shapes:
            def one(i, name=name, sets=sets):
                w, a, c = sets[i % len(sets)][name]
                T.gemm(dev, w, a, 1, c)
            for i in range(16):
                one(i)
            dev.synchronize()
            ms, how = time_short_launches(dev, T_graphs, one, 200, graphs_done)
            b = algo_bytes(k, n)
            entry[name] = {"k": k, "n": n, "us": round(ms * 1e3, 3), "GBps": round(b / (ms * 1e-3) / 1e9, 1), "timed": how}

        def run_sets(sets=sets, shapes=shapes):
            for st in sets:
                for name, k, n in shapes:
                    w, a, c = st[name]
                    T.gemm(dev, w, a, 1, c)
        g = capture(run_sets)
        for _ in range(5):
            g.replay()
        dev.synchronize()
        ms = time_launches(dev, lambda i: g.replay(), 50) / len(sets)
        lb = sum(algo_bytes(k, n) for _, k, n in shapes)
        entry["layer_graph"] = {"us": round(ms * 1e3, 3), "GBps": round(lb / (ms * 1e-3) / 1e9, 1), "bytes": lb}
        graphs_done.append(g)
        small[label] = entry
        for st in sets:
            for name in st:
                st[name][0].free(); st[name][1].free(); st[name][2].free()

    # The LM head of the same model class as a TW-Marlin GEMV with on-device argmax (the reference has
    # forward_lm_head_tw_marlin, generate.rs:1748-1761, and a GPU argmax buffer, :1417): 3584 -> 152064, the
    # largest GEMV of a decode step.  Two weight sets (616 MB) alternate so that the cache cannot hold them.
    log("LM head")
    lm = None
    if not args.no_lm_head:
        k, n = 3584, 152064
        sets = []
        for _ in range(2):
            packed = rng.integers(0, 256, size=(k // 32) * n * 16, dtype=np.uint8)
            scales = (np.abs(rng.standard_normal((k // 32) * n, dtype=np.float32)) * np.float32(0.02)).astype(np.float16)
            sets.append(T.MarlinWeight.upload(dev, packed, scales.view(np.uint16), k, n))
        a1 = T.GpuTensor.from_host(dev, rng.standard_normal(k, dtype=np.float32).astype(np.float16).view(np.uint16), "f16")
        logits = T.GpuTensor.zeros(dev, (n,), "f32")
        token = T.GpuTensor.from_host(dev, np.zeros(1, np.int32))

        def one_gemv(i):
            T.gemm(dev, sets[i % 2], a1, 1, logits)

        def one_argmax(i):
            T.argmax(dev, logits, token, 1, n)
        for i in range(6):
            one_gemv(i)
            one_argmax(i)
        dev.synchronize()
        ms_g = time_launches(dev, one_gemv, 100)
        ms_a = time_launches(dev, one_argmax, 100)
        picked = int(token.to_host()[0])
        assert picked == int(np.argmax(logits.to_host())), "argmax disagrees with the host"
        b = algo_bytes(k, n)
        lm = {"k": k, "n": n, "gemv_us": round(ms_g * 1e3, 2), "GBps": round(b / (ms_g * 1e-3) / 1e9, 1),
              "frac_hbm": round(b / (ms_g * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "argmax_us": round(ms_a * 1e3, 2),
              "bytes": b}
        for w in sets:
            w.free()
        logits.free()

    # MLP front half at M=1: the reference's three launches (GEMV, split_gate_up, fused_silu_mul) against the
    # single launch with the gate applied in the GEMV's store; graphs over distinct weight sets
    log("MLP front half")
    mlp_front = None
    if not args.no_swiglu:
        k, ffn = 3584, 18944
        plain, pairedw = [], []
        for _ in range(L):
            halves = []
            for _h in range(2):
                packed = rng.integers(0, 256, size=(k // 32) * ffn * 16, dtype=np.uint8)
                scales = (np.abs(rng.standard_normal((k // 32) * ffn, dtype=np.float32)) * np.float32(0.02)).astype(np.float16)
                halves.append((T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales.view(np.uint16), "f16")))
            fp, fs = T.fuse_tw_marlin_n(dev, halves, k, [ffn, ffn])
            plain.append(T.MarlinWeight.from_device(dev, fp, fs, k, 2 * ffn))
            pairedw.append(T.MarlinWeight.gate_up(dev, halves[0], halves[1], k, ffn))
            for t in (fp, fs, halves[0][0], halves[0][1], halves[1][0], halves[1][1]):
                t.free()
        a1 = T.GpuTensor.from_host(dev, rng.standard_normal(k, dtype=np.float32).astype(np.float16).view(np.uint16), "f16")
        gate_up = T.GpuTensor.zeros(dev, (2 * ffn,), "f32")
        g1, u1 = T.GpuTensor.zeros(dev, (ffn,), "f32"), T.GpuTensor.zeros(dev, (ffn,), "f32")
        act3, act2, act1 = (T.GpuTensor.zeros(dev, (ffn,), "f32") for _ in range(3))

        def three():
            for w in plain:
                T.gemm(dev, w, a1, 1, gate_up)
                T.split_gate_up(dev, gate_up, g1, u1, ffn, 1)
                T.fused_silu_mul(dev, g1, u1, act3)

        def two():
            for w in plain:
                T.gemm_split(dev, w, a1, 1, [g1, u1], [ffn, ffn])
                T.fused_silu_mul(dev, g1, u1, act2)

        def fused():
            for w in pairedw:
                T.gemm_swiglu(dev, w, a1, 1, act1)
        mlp_front = {"k": k, "ffn": ffn}
        for label, fn in (("gemv_split_silu_us", three), ("gemv_with_split_store_silu_us", two), ("fused_us", fused)):
            fn()
            dev.synchronize()
            gr = capture(fn)
            for _ in range(5):
                gr.replay()
            dev.synchronize()
            mlp_front[label] = round(time_launches(dev, lambda i: gr.replay(), 50) / L * 1e3, 2)
            graphs_done.append(gr)
        a1h, a3h = act1.to_host(), act3.to_host()     # same sums, possibly another split order per column
        assert np.abs(a1h - a3h).max() <= 1e-4 * np.abs(a3h).max(), "fused SwiGLU differs from the three-launch sequence"
        for w in plain + pairedw:
            w.free()

    # Mixture-of-experts decode (the reference's Gemma MoE shape: hidden 2816, expert dim 704, 128 experts, top 8):
    # gate+up of the eight routed experts, GEGLU, down + weighted sum; ids rotate so the experts come from HBM
    log("MoE decode")
    moe = None
    if not args.no_moe:
        k, dim, experts, top_k = 2816, 704, 128, 8
        g_gu, g_d = k // 32, dim // 32
        gu_p = T.GpuTensor.from_host(dev, rng.integers(0, 256, size=experts * g_gu * 2 * dim * 16, dtype=np.uint8))
        gu_s = T.GpuTensor.from_host(dev, (np.abs(rng.standard_normal(experts * g_gu * 2 * dim, dtype=np.float32)) * np.float32(0.02)).astype(np.float16).view(np.uint16), "f16")
        d_p = T.GpuTensor.from_host(dev, rng.integers(0, 256, size=experts * g_d * k * 16, dtype=np.uint8))
        d_s = T.GpuTensor.from_host(dev, (np.abs(rng.standard_normal(experts * g_d * k, dtype=np.float32)) * np.float32(0.02)).astype(np.float16).view(np.uint16), "f16")
        bank_gu = T.ExpertBank.from_device(dev, gu_p, gu_s, g_gu * 2 * dim * 16, g_gu * 2 * dim, k, 2 * dim, experts)
        bank_gu_paired = T.ExpertBank.from_device(dev, gu_p, gu_s, g_gu * 2 * dim * 16, g_gu * 2 * dim, k, 2 * dim, experts, pair_gate_up=True)
        bank_d = T.ExpertBank.from_device(dev, d_p, d_s, g_d * k * 16, g_d * k, dim, k, experts)
        id_sets = [T.GpuTensor.from_host(dev, ((np.arange(top_k) * 16 + r) % experts).astype(np.float32)) for r in range(16)]
        wts = T.GpuTensor.from_host(dev, np.full(top_k, 0.125, np.float32))
        x = T.GpuTensor.from_host(dev, rng.standard_normal(k, dtype=np.float32))
        gate_up_all = T.GpuTensor.zeros(dev, (top_k, 2 * dim), "f32")
        geglu_a, geglu_b = T.GpuTensor.zeros(dev, (top_k, dim), "f32"), T.GpuTensor.zeros(dev, (top_k, dim), "f32")
        acc_a, acc_b = T.GpuTensor.zeros(dev, (k,), "f32"), T.GpuTensor.zeros(dev, (k,), "f32")

        def three():
            for ids in id_sets:
                T.batched_marlin_gate_up(dev, x, bank_gu, ids, gate_up_all, top_k)
                T.batched_marlin_split_geglu(dev, gate_up_all, geglu_a, dim, top_k)
                T.batched_marlin_down_axpy(dev, geglu_a, bank_d, ids, wts, acc_a, top_k)

        def two():
            for ids in id_sets:
                T.batched_marlin_gate_up(dev, x, bank_gu_paired, ids, geglu_b, top_k, act=T.ACT_GEGLU)
                T.batched_marlin_down_axpy(dev, geglu_b, bank_d, ids, wts, acc_b, top_k)
        acc_c = T.GpuTensor.zeros(dev, (k,), "f32")

        def slabs():   # the reference's own arguments: raw slabs, nothing repacked
            for ids in id_sets:
                T.batched_marlin_gate_up_slabs(dev, x, gu_p, gu_s, ids, gate_up_all, g_gu * 2 * dim * 16, g_gu * 2 * dim, 2 * dim, k, top_k)
                T.batched_marlin_split_geglu(dev, gate_up_all, geglu_a, dim, top_k)
                T.batched_marlin_down_axpy_slabs(dev, geglu_a, d_p, d_s, ids, wts, acc_c, g_d * k * 16, g_d * k, k, dim, top_k)
        moe_bytes = top_k * (algo_bytes(k, 2 * dim) + algo_bytes(dim, k))
        moe = {"hidden": k, "expert_dim": dim, "experts": experts, "top_k": top_k, "bytes": moe_bytes}
        for label, fn in (("gate_up_geglu_down_us", three), ("fused_geglu_then_down_us", two), ("reference_slabs_us", slabs)):
            fn()
            dev.synchronize()
            gr = capture(fn)
            for _ in range(3):
                gr.replay()
            dev.synchronize()
            us = time_launches(dev, lambda i: gr.replay(), 30) / len(id_sets) * 1e3
            moe[label] = round(us, 2)
            moe[label.replace("_us", "_GBps")] = round(moe_bytes / (us * 1e-6) / 1e9, 1)
            graphs_done.append(gr)
        # (the down projection accumulates: compare one pass of each from zero)
        acc_a.copy_from_host(np.zeros(k, np.float32))
        acc_b.copy_from_host(np.zeros(k, np.float32))
        three()
        two()
        assert np.array_equal(acc_a.to_host(), acc_b.to_host()), "fused GEGLU differs from the three-launch sequence"
        for b_ in (bank_gu, bank_gu_paired, bank_d):
            b_.free()

    log("prefill")
    prefill = None
    if not args.no_prefill:
        prefill = {}
        vendor = None if args.no_vendor_gemm else VendorGemm(dev)
        for k, n in ((4096, 11008), (11008, 4096)):
            packed = rng.integers(0, 256, size=(k // 32) * n * 16, dtype=np.uint8)
            scales = (np.abs(rng.standard_normal((k // 32) * n, dtype=np.float32)) * np.float32(0.02)).astype(np.float16)
            w = T.MarlinWeight.upload(dev, packed, scales.view(np.uint16), k, n)
            for m in (512, 2048):
                a_host = rng.standard_normal((m, k), dtype=np.float32).astype(np.float16).view(np.uint16)
                a_m = T.GpuTensor.from_host(dev, a_host, "f16")
                c_m = T.GpuTensor.zeros(dev, (m, n), "f32")

                def one(i, w=w, a_m=a_m, c_m=c_m, m=m):
                    T.gemm(dev, w, a_m, m, c_m)
                for i in range(3):
                    one(i)
                dev.synchronize()
                # five timed windows of 20 launches each, the median one counts (as for the decode kernels)
                pf_windows = [time_launches(dev, one, 20)] + [time_launches(dev, one, 20, settle_ms=0.0) for _ in range(4)]
                ms = sorted(pf_windows)[len(pf_windows) // 2]
                tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
                err, ncols = sampled_prefill_rel_err(c_m.to_host(), packed, scales.view(np.uint16), a_host, m, k, n, rng)
                assert err < 1e-2, "prefill result outside the tolerance: %g" % err
                prefill["M%d_K%d_N%d" % (m, k, n)] = {"us": round(ms * 1e3, 1), "TFLOPs": round(tf, 1),
                                                      "frac_mfma_f16_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                                                      "timed_windows": len(pf_windows),
                                                      "us_min": round(min(pf_windows) * 1e3, 1), "us_max": round(max(pf_windows) * 1e3, 1),
                                                      "plan": dev.plan(k, n, m),
                                                      "max_rel_err": err,
                                                      "max_rel_err_over": "all %d rows x %d sampled columns, f64 product on the FP16 Q4 unpack" % (m, ncols)}
                if vendor is not None and vendor.ok:
                    # the vendor library's dense FP16 GEMM on the already unpacked weights (no Q4 unpack in the
                    # timed region): what the reference's dequant + library-GEMM prefill route would cost here
                    if m == 512:
                        w16 = w.dequant_f16()
                    ours = c_m.to_host() if m == 512 else None
                    v_ms = vendor.time(a_m, w16, c_m, m, n, k, 20)
                    if v_ms is not None and ours is not None:
                        theirs = c_m.to_host()
                        assert np.abs(theirs - ours).max() <= 2e-3 * np.abs(ours).max(), "rocBLAS result differs"
                    if v_ms is not None:
                        prefill["M%d_K%d_N%d" % (m, k, n)]["rocblas_dense_f16_us"] = round(v_ms * 1e3, 1)
                        prefill["M%d_K%d_N%d" % (m, k, n)]["rocblas_dense_f16_TFLOPs"] = round(2.0 * m * n * k / (v_ms * 1e-3) / 1e12, 1)
                    if m == 2048:
                        w16.free()
                a_m.free()
                c_m.free()
            w.free()

    # prefill MLP front half (LLaMA-7B: 4096 -> 2 x 11008, M = 2048): GEMM to [M, 2*ffn] + split/gate kernel
    # against the gate applied in the GEMM's store
    prefill_mlp = None
    if not args.no_prefill and not args.no_swiglu:
        log("prefill MLP front half")
        k, ffn, m = 4096, 11008, 2048
        halves = []
        for _h in range(2):
            packed = rng.integers(0, 256, size=(k // 32) * ffn * 16, dtype=np.uint8)
            scales = (np.abs(rng.standard_normal((k // 32) * ffn, dtype=np.float32)) * np.float32(0.02)).astype(np.float16)
            halves.append((T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales.view(np.uint16), "f16")))
        wp = T.MarlinWeight.gate_up(dev, halves[0], halves[1], k, ffn)
        a_m = T.GpuTensor.from_host(dev, rng.standard_normal((m, k), dtype=np.float32).astype(np.float16).view(np.uint16), "f16")
        tmp = T.GpuTensor.zeros(dev, (m, 2 * ffn), "f32")
        seq, fused_out = T.GpuTensor.zeros(dev, (m, ffn), "f32"), T.GpuTensor.zeros(dev, (m, ffn), "f32")

        def two_step(i):
            T.gemm(dev, wp, a_m, m, tmp)
            T.swiglu_rows(dev, tmp, seq, ffn, m, paired=True)

        def one_step(i):
            T.gemm_swiglu(dev, wp, a_m, m, fused_out)
        prefill_mlp = {"m": m, "k": k, "ffn": ffn}
        for label, fn in (("gemm_then_gate_us", two_step), ("fused_us", one_step)):
            for i in range(3):
                fn(i)
            dev.synchronize()
            ms = time_launches(dev, fn, 10)
            prefill_mlp[label] = round(ms * 1e3, 1)
            prefill_mlp[label.replace("_us", "_TFLOPs")] = round(2.0 * m * 2 * ffn * k / (ms * 1e-3) / 1e12, 1)
        assert np.array_equal(fused_out.to_host(), seq.to_host()), "fused prefill SwiGLU differs from GEMM + gate"
        for t in (tmp, seq, fused_out, a_m, halves[0][0], halves[0][1], halves[1][0], halves[1][1]):
            t.free()
        wp.free()

    sweep = None
    if args.sweep_splits:
        sweep = {}
        for name, k, n in LAYER_7B:
            for m in (1, 4, 8, 16, 32):
                a_m = T.GpuTensor.from_host(dev, rng.standard_normal((m, k), dtype=np.float32).astype(np.float16).view(np.uint16), "f16")
                c_m = T.GpuTensor.zeros(dev, (m, n), "f32")
                row = {}
                for sp in (1, 2, 3, 4, 6, 8, 12, 16, 0):      # the library's own plan last, after the forced ones
                    def one(i, a_m=a_m, c_m=c_m, m=m, sp=sp, name=name):
                        T.gemm(dev, layers[i % args.layers][name][0], a_m, m, c_m, sp)
                    for i in range(8):
                        one(i)
                    dev.synchronize()
                    row["auto" if sp == 0 else str(sp)] = round(time_short_launches(dev, T_graphs, one, 104, graphs_done, below_ms=16e-3)[0] * 1e3, 2)
                best = min((v, key) for key, v in row.items() if key != "auto")
                sweep["%s_M%d" % (name, m)] = {"us": row, "auto_over_best": round(row["auto"] / best[0], 3), "best_splits": int(best[1])}
                a_m.free()
                c_m.free()

    model_sweep = None
    if args.sweep_models:
        # the planner away from the shapes it was fitted on: option "sub" = 1 (and "kernel" = 3 from M = 5 on) keeps
        # the 64-column lane-per-column kernel / the streaming kernel, 0 is the library's plan
        model_sweep = {}
        other = [("llama3_8b_qkv", 4096, 6144), ("llama3_8b_o", 4096, 4096), ("llama3_8b_gate_up", 4096, 28672),
                 ("llama3_8b_down", 14336, 4096), ("13b_qkv", 5120, 15360), ("13b_down", 13824, 5120),
                 ("70b_qkv", 8192, 10240), ("70b_o", 8192, 8192), ("70b_gate_up", 8192, 57344), ("70b_down", 28672, 8192),
                 ("qwen15b_qkv", 1536, 2048), ("qwen15b_gate_up", 1536, 17920), ("qwen15b_down", 8960, 1536)]
        for name, k, n in other:
            sets = []
            for _ in range(max(3, min(12, int(600e6 // (k * n * 0.5625)) + 1))):
                packed = rng.integers(0, 256, size=(k // 32) * n * 16, dtype=np.uint8)
                scales = (np.abs(rng.standard_normal((k // 32) * n, dtype=np.float32)) * np.float32(0.02)).astype(np.float16)
                sets.append(T.MarlinWeight.upload(dev, packed, scales.view(np.uint16), k, n))
            for m, dt in ((1, "f16"), (1, "f32"), (4, "f16"), (8, "f16"), (16, "f16"), (32, "f16")):
                ah = rng.standard_normal((m, k), dtype=np.float32)
                a_m = (T.GpuTensor.from_host(dev, ah.astype(np.float16).view(np.uint16), "f16") if dt == "f16"
                       else T.GpuTensor.from_host(dev, ah))
                c_m = T.GpuTensor.zeros(dev, (m, n), "f32")

                def one(i, a_m=a_m, c_m=c_m, m=m, sets=sets):
                    T.gemm(dev, sets[i % len(sets)], a_m, m, c_m)
                row = {}
                for label in ("whole_tiles", "plan"):
                    dev.set_option("sub", 1 if label == "whole_tiles" else 0)
                    dev.set_option("kernel", 3 if (label == "whole_tiles" and m > 4) else 0)
                    for i in range(8):
                        one(i)
                    dev.synchronize()
                    row[label] = round(time_short_launches(dev, T_graphs, one, 96, graphs_done, below_ms=1.0)[0] * 1e3, 2)
                dev.set_option("sub", 0)
                dev.set_option("kernel", 0)
                row["plan_GBps"] = round(algo_bytes(k, n, m) / (row["plan"] * 1e-6) / 1e9, 1)
                model_sweep["%s_K%d_N%d_M%d_%s" % (name, k, n, m, dt)] = row
                a_m.free()
                c_m.free()
            for w in sets:
                w.free()

    prefill_sweep = None
    if args.sweep_prefill:
        # block form (64 x 256, 128 x 256, 128 rows x 192 columns per workgroup) x split-K forced against the library's plan; the plan is timed
        # after the forced cases, every case after ~200 untimed launches
        prefill_sweep = {}
        for k, n in ((4096, 11008), (11008, 4096), (3584, 37888), (18944, 3584), (3584, 4608)):
            packed = rng.integers(0, 256, size=(k // 32) * n * 16, dtype=np.uint8)
            scales = (np.abs(rng.standard_normal((k // 32) * n, dtype=np.float32)) * np.float32(0.02)).astype(np.float16)
            w = T.MarlinWeight.upload(dev, packed, scales.view(np.uint16), k, n)
            for m in (128, 256, 512, 1024, 2048):
                a_m = T.GpuTensor.from_host(dev, rng.standard_normal((m, k), dtype=np.float32).astype(np.float16).view(np.uint16), "f16")
                c_m = T.GpuTensor.zeros(dev, (m, n), "f32")
                row = {}
                for bm, sp in ((64, 1), (64, 2), (64, 4), (128, 1), (128, 2), (128, 4), (192, 1), (192, 2), (192, 4), (0, 0)):
                    dev.set_option("prefill_bm", bm)
                    for _ in range(200):
                        T.gemm(dev, w, a_m, m, c_m, sp)
                    dev.synchronize()
                    us = min(time_launches(dev, lambda i: T.gemm(dev, w, a_m, m, c_m, sp), 20, settle_ms=0) for _ in range(3)) * 1e3
                    row["auto" if bm == 0 else "%dx%d" % (bm, sp)] = round(us, 1)
                dev.set_option("prefill_bm", 0)
                best = min((v, key) for key, v in row.items() if key != "auto")
                prefill_sweep["K%d_N%d_M%d" % (k, n, m)] = {"us": row, "auto_over_best": round(row["auto"] / best[0], 3),
                                                            "auto_TFLOPs": round(2.0 * m * n * k / row["auto"] / 1e6, 1)}
                a_m.free()
                c_m.free()
            w.free()

    log("cpu baseline")
    cpu = None
    if not args.no_cpu:
        # the checker, timed: reference CPU semantics, one thread, whole layers (a different weight set each pass)
        # until about ten seconds of CPU work are done; the first pass also checks the GPU result
        from oracle import twm_oracle as O
        host = layers_host[0]
        t_cpu = 0.0
        worst = 0.0
        passes = 0
        while t_cpu < 10.0 and passes < 12:
            li = passes % args.layers
            for name, k, n in LAYER_7B:
                packed, scales, act = layers_host[li][name]
                a32 = act.view(np.float16).astype(np.float32).reshape(1, k)
                t1 = time.perf_counter()
                c_cpu = O.linear_dense(a32, packed, scales, 1, k, n)
                t_cpu += time.perf_counter() - t1
                if passes == 0:
                    w, a, c = layers[0][name]
                    T.gemm(dev, w, a, 1, c)
                    got = c.to_host().astype(np.float64)
                    truth = c_cpu[0].astype(np.float64)
                    denom = np.maximum(np.abs(truth), 1e-3 * np.abs(truth).max())
                    worst = max(worst, float((np.abs(got - truth) / denom).max()))
            passes += 1
        t_cpu /= passes
        # the same layer with the fused on-the-fly form (no dense copy), OpenMP over N on all host cores
        t_mt, cores_mt = 0.0, 1
        for name, k, n in LAYER_7B:
            packed, scales, act = host[name]
            a32 = act.view(np.float16).astype(np.float32).reshape(1, k)
            t1 = time.perf_counter()
            _, used = O.gemv_ref_order_mt(a32, packed, scales, 1, k, n)
            t_mt += time.perf_counter() - t1
            cores_mt = max(cores_mt, int(used))
        cpu = {"value": round(layer_bytes / t_cpu / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
               "sample": "%d Qwen-7B-shaped layers (4 GEMVs each, M=1, 131.3 MB algorithmic per layer), unpack to dense f32 + naive cpu_gemm" % passes,
               "seconds": round(t_cpu * passes, 3), "seconds_per_layer": round(t_cpu, 3), "gpu_over_cpu": round(value / (layer_bytes / t_cpu / 1e9), 1),
               "max_rel_err_gpu_vs_cpu": worst,
               "all_cores": {"value": round(layer_bytes / t_mt / 1e9, 4), "unit": "GB/s", "cores": cores_mt,
                             "sample": "same layer, on-the-fly unpack + dot per column (reference GEMV order), OpenMP over N",
                             "seconds": round(t_mt, 3)}}

    out = {
        "metric": "achieved HBM GB/s of the W4A16 GEMV set at M=1 (Qwen-7B layer shapes, hipGraph replay)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 x int4 -> f32", "data": "synthetic",
        "config": {"workload": "Qwen-7B decode linear set, M=1: qkv 3584->4608, o 3584->3584, gate_up 3584->37888, "
                               "down 18944->3584; group-32 Q4 + FP16 scales; %d distinct layers rotated" % args.layers,
                   "layer_bytes": layer_bytes, "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
                   "us_per_layer": round(ms_step * 1e3, 3), "us_per_layer_min": round(ms_step_min * 1e3, 3),
                   "timed_windows": n_windows, "steps_per_window": steps, "headline": "median over the windows",
                   "us_per_layer_own_graph": round(ms_step_own * 1e3, 3),
                   "graphs": "off (eager launches)" if graphs_off else "on", "wall_s": round(wall, 3)},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "per_projection": per_shape,
        "drop_in_reference_layout_m1": drop_in,
        "f32_activations_m1": f32_rows,
    }
    out["small_shapes_m1"] = small
    if lm:
        out["lm_head_m1"] = lm
    if mlp_front is not None:
        out["mlp_front_m1"] = mlp_front
    if moe is not None:
        out["moe_decode_m1"] = moe
    if prefill_mlp:
        out["prefill_mlp_front"] = prefill_mlp
    if prefill:
        out["prefill"] = prefill
        # the figure held against the 50 % target is the slower of the two M = 2048 shapes
        m2048 = {key: v for key, v in prefill.items() if key.startswith("M2048")}
        worst = min(m2048.items(), key=lambda kv: kv[1]["TFLOPs"])
        out["roofline_prefill"] = {"bound": "mfma", "kernel": "k_prefill (%s, the slower M = 2048 shape)" % worst[0],
                                   "achieved": worst[1]["TFLOPs"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                   "frac": worst[1]["frac_mfma_f16_peak"], "us_per_launch": worst[1]["us"],
                                   "us_min": worst[1]["us_min"], "us_max": worst[1]["us_max"],
                                   "timed_windows": worst[1]["timed_windows"],
                                   "all_m2048_shapes": {key: v["frac_mfma_f16_peak"] for key, v in m2048.items()}}
    if extra:
        out["batched_decode"] = extra
    if tuned is not None:
        out["decode_with_measured_plans"] = tuned
    if sweep:
        out["split_sweep"] = sweep
    if prefill_sweep is not None:
        out["prefill_sweep"] = prefill_sweep
    if model_sweep is not None:
        out["model_sweep"] = model_sweep
    print(json.dumps(out))
    for g in graphs + [graph_all] + list(graph_rest.values()) + graphs_done:
        g.destroy()
    dev.close()


if __name__ == "__main__":
    main()

// C ABI of libtwmarlin_hip.so (declared in include/twmarlin.h): contexts, device memory,
// weight upload with one-time repack, the quantized-GEMM dispatcher with its split-K choice,
// and hipGraph capture/replay.  Host-side counterpart of the reference's
// crates/kernels/src/{quantize.rs:1301-1360, device.rs, tensor.rs, cuda_graph.rs}.
#include "../../include/twmarlin.h"
#include "twm_internal.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <string>
#include <vector>

using namespace twm;

static thread_local std::string g_err;
twm::TraceBuf twm::g_trace = {nullptr, 0};

int twm::api_fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

#define HIP_TRY(expr, code, what)                                                      \
    do {                                                                               \
        hipError_t e__ = (expr);                                                       \
        if (e__ != hipSuccess) return api_fail(code, "%s: %s", what, hipGetErrorString(e__)); \
    } while (0)

struct twm_ctx {
    int ordinal;
    hipStream_t own_stream;
    hipStream_t stream;
    float *ws;            // split-K partial tiles
    size_t ws_bytes;
    float *sk_ws;         // parked partial tiles of the stream-K prefill GEMM
    size_t sk_ws_bytes;
    int prefill_sk;       // stream-K prefill: 0 = the planner's choice, 1 = off, 128 / 256 = on with that block height
    unsigned *counters;   // one arrival counter per tile group, zero between launches
    uint32_t n_counters;
    bool capturing;
    int force_nt;         // 0 = heuristic
    int force_waves;      // 0 = heuristic
    int force_sub_waves;  // sub-tile kernels with a forced width: waves per workgroup (1 .. 16), 0 = "waves" or eight
    int force_sub;        // M <= 4: 0 = heuristic, 1 = whole 64-column tiles per workgroup, 32 or 16 = the sub-tile kernel
    int force_kernel;     // 0 = heuristic, 2 = one-lane-per-column kernel on whole tiles (M <= 4), 3 = streaming kernel (M <= 32),
                          // 4 = batched-decode kernel with LDS-shared activations (M <= 32; "nt" = tiles per wave, "waves" 8 / 16 = 2 / 4 k-slices)
    int prefill_bm;       // prefill block form: 0 = choose, 64 = 64 rows x 256 columns, 128 = 128 x 256, 192 = 128 rows x 192 columns
    int prefill_min_m;    // M from which the LDS/MFMA prefill kernel runs instead of 16-row decode blocks
    int dequant_src;      // which copy twm_weight_dequant_f16 unpacks: 0 = 16-column tiles, 1 = column-lane
    int weight_copies;    // copies a new weight handle is given: 0 or 3 = both, 1 = 16-column tiles only, 2 = column-lane only
    int m1_exact;         // twm_gemm_tw_marlin_m1: 1 = f32 activations and f32 FMAs in the reference's order
    int m1_splits;        // twm_gemm_tw_marlin_m1: split-K factor of the MFMA kernel, 0 = heuristic
    int batch_rounded;    // M = 17 .. 32: 1 = weights rounded to f16 (the reference's dequant-then-FP16-GEMM arithmetic), 0 = exact
    hipDeviceProp_t prop;
};

// A launch form as the option knobs name it (twm_ctx_set_option), measured to be the fastest for one weight and one
// bucket of row counts by twm_weight_tune: the role of the per-shape table of crates/kernels/src/autotune.rs:254-396.
struct TunedPlan {
    uint8_t valid, kernel, nt, waves, sub, sub_waves, splits, prefill_bm;
};
static_assert(sizeof(TunedPlan) == 8, "a tuned plan is eight bytes of the weight blob");
constexpr int kTuneBuckets = 12;
// row counts 1, 2, 3-4, 5-8, 9-16, 17-32, 33-64, 65-128, 129-256, 257-512, 513-1024, above
static int tune_bucket(uint32_t m)
{
    if (m <= 2) return (int)m - 1;
    int b = 2;
    for (uint32_t top = 4; m > top && b < kTuneBuckets - 1; top *= 2) b++;
    return b;
}

// The two repacked copies are allocations of their own, each made when the handle is created (option
// "weight_copies") or at the first call that needs it (weight_ensure): a decode-only or prefill-only deployment holds
// one copy, 4.5 bits per weight.
enum { kCopyTile = 1, kCopyCol = 2 };
struct twm_weight {
    twm_ctx *ctx;
    void *qw;   // 16-column tile order: nibbles (qw) and scales (sc) in one allocation; nullptr while not built
    void *sc;
    void *cq;   // column-lane copy: 4608-byte blocks (nibbles + scales together); nullptr while not built
    uint32_t k, n, groups, n_tiles, k_chunks;
    size_t copy_bytes;  // one copy
    size_t bytes;       // device memory held now
    bool paired;  // gate_up weight whose columns are in the paired order (32 gate, 32 up, ...)
    TunedPlan tuned[kTuneBuckets];  // measured plans per row-count bucket (twm_weight_tune); valid = 0: the planners' choice
};

struct twm_bank {
    twm_ctx *ctx;
    void *cq;           // experts x column-lane copy
    size_t expert_bytes, bytes;
    uint32_t experts, k, n, n_pad, k_chunks;
    bool paired;
};

struct twm_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

static const size_t kWsBytes = 64ull << 20;
static const uint32_t kCounters = 1u << 16;

extern "C" {

const char *twm_version(void) { return "0.1.0"; }

int twm_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

const char *twm_last_error(void) { return g_err.c_str(); }

twm_ctx *twm_ctx_create(int ordinal)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || ordinal < 0 || ordinal >= count) {
        api_fail(TWM_DEVICE_ERROR, "twm_ctx_create: no HIP device %d (%s)", ordinal,
             e != hipSuccess ? hipGetErrorString(e) : "ordinal out of range");
        return nullptr;
    }
    twm_ctx *c = new (std::nothrow) twm_ctx();
    if (!c) { api_fail(TWM_MEMORY_ERROR, "twm_ctx_create: out of host memory"); return nullptr; }
    c->ordinal = ordinal;
    c->capturing = false;
    c->force_nt = 0;
    c->force_waves = 0;
    c->force_sub = 0;
    c->force_sub_waves = 0;
    c->force_kernel = 0;
    c->dequant_src = 0;
    c->weight_copies = 0;
    c->m1_exact = 0;
    c->m1_splits = 0;
    c->batch_rounded = 0;
    c->prefill_bm = 0;
    c->prefill_min_m = 33;  // M <= 32 is batched decode (exact f32 scales, weights streamed once)
    c->ws = nullptr;
    c->sk_ws = nullptr;
    c->sk_ws_bytes = 0;
    c->prefill_sk = 0;
    c->counters = nullptr;
    c->own_stream = nullptr;
    bool ok = hipSetDevice(ordinal) == hipSuccess && hipGetDeviceProperties(&c->prop, ordinal) == hipSuccess;
    if (ok && strncmp(c->prop.gcnArchName, "gfx950", 6) != 0) {
        api_fail(TWM_DEVICE_ERROR, "twm_ctx_create: device %d is %s; this library holds gfx950 code only", ordinal,
             c->prop.gcnArchName);
        delete c;
        return nullptr;
    }
    ok = ok && hipStreamCreateWithFlags(&c->own_stream, hipStreamNonBlocking) == hipSuccess;
    ok = ok && init_prefill() == hipSuccess && init_prefill_sk() == hipSuccess;
    ok = ok && noalloc_scratch_for_current_device("twm_ctx_create") != nullptr;
    c->stream = c->own_stream;
    c->ws_bytes = kWsBytes;
    c->n_counters = kCounters;
    ok = ok && hipMalloc((void **)&c->ws, c->ws_bytes) == hipSuccess;
    ok = ok && hipMalloc((void **)&c->counters, c->n_counters * sizeof(unsigned)) == hipSuccess;
    if (ok) {  // two 256-row partial tiles per CU
        c->sk_ws_bytes = prefill_sk_scratch_bytes(256, (uint32_t)c->prop.multiProcessorCount);
        ok = hipMalloc((void **)&c->sk_ws, c->sk_ws_bytes) == hipSuccess;
    }
    ok = ok && hipMemset(c->counters, 0, c->n_counters * sizeof(unsigned)) == hipSuccess;
    ok = ok && hipDeviceSynchronize() == hipSuccess;
    if (!ok) {
        api_fail(TWM_DEVICE_ERROR, "twm_ctx_create: %s", hipGetErrorString(hipGetLastError()));
        if (c->ws) (void)hipFree(c->ws);
        if (c->sk_ws) (void)hipFree(c->sk_ws);
        if (c->counters) (void)hipFree(c->counters);
        if (c->own_stream) (void)hipStreamDestroy(c->own_stream);
        delete c;
        return nullptr;
    }
    return c;
}

void twm_ctx_destroy(twm_ctx *ctx)
{
    if (!ctx) return;
    (void)hipSetDevice(ctx->ordinal);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(ctx->ws);
    (void)hipFree(ctx->sk_ws);
    (void)hipFree(ctx->counters);
    (void)hipStreamDestroy(ctx->own_stream);
    delete ctx;
}

int twm_ctx_sync(twm_ctx *ctx)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_ctx_sync: null context");
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        // A launch that died may have left arrival counters of the in-launch split-K above zero, which would make
        // every later split-K launch of this context finish its tiles early: put them back to zero if the device
        // still takes a call.
        (void)hipGetLastError();
        (void)hipMemset(ctx->counters, 0, ctx->n_counters * sizeof(unsigned));
        (void)hipGetLastError();
        return api_fail(TWM_DEVICE_ERROR, "twm_ctx_sync: %s", hipGetErrorString(e));
    }
    return TWM_OK;
}

int twm_debug_trace(twm_ctx *ctx, uint32_t *trace_dev, uint32_t capacity_workgroups)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_debug_trace: null context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_debug_trace: a graph capture is open");
    g_trace.ptr = capacity_workgroups ? trace_dev : nullptr;
    g_trace.capacity = trace_dev ? capacity_workgroups : 0;
    return TWM_OK;
}

int twm_ctx_set_stream(twm_ctx *ctx, void *hip_stream)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_ctx_set_stream: null context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_ctx_set_stream: a graph capture is open");
    ctx->stream = hip_stream ? (hipStream_t)hip_stream : ctx->own_stream;
    return TWM_OK;
}

void *twm_ctx_stream(twm_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int twm_ctx_info(twm_ctx *ctx, char *buf, size_t buf_len)
{
    if (!ctx || !buf || buf_len == 0) return api_fail(TWM_INVALID_HANDLE, "twm_ctx_info: null argument");
    snprintf(buf, buf_len, "%s (%s) | %d CUs | %.1f GiB", ctx->prop.name, ctx->prop.gcnArchName,
             ctx->prop.multiProcessorCount, (double)ctx->prop.totalGlobalMem / (1024.0 * 1024.0 * 1024.0));
    return TWM_OK;
}

/* Tuning knobs for sweeps (0 = heuristic): "nt" = tiles per workgroup (1, 2, 4); "waves" = waves per
 * workgroup; "kernel" = 2 the one-lane-per-column kernel (M <= 4), 3 the
 * streaming kernel, 4 the batched-decode kernel with LDS-shared activations;
 * "dequant_src" = which weight copy twm_weight_dequant_f16 unpacks; "prefill_min_m" = smallest M that
 * runs the prefill kernel. */
int twm_ctx_set_option(twm_ctx *ctx, const char *key, int value)
{
    if (!ctx || !key) return api_fail(TWM_INVALID_HANDLE, "twm_ctx_set_option: null argument");
    if (strcmp(key, "nt") == 0) {
        if (value < 0 || value > 4) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: nt must be 0 .. 4");
        ctx->force_nt = value;
        return TWM_OK;
    }
    if (strcmp(key, "waves") == 0) {
        if (value != 0 && value != 1 && value != 2 && value != 4 && value != 8 && value != 16)
            return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: waves must be 0, 1, 2, 4, 8 or 16");
        ctx->force_waves = value;
        return TWM_OK;
    }
    if (strcmp(key, "sub_waves") == 0) {
        if (value < 0 || value > 16) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: sub_waves must be 0 .. 16");
        ctx->force_sub_waves = value;
        return TWM_OK;
    }
    if (strcmp(key, "sub") == 0) {
        if (value != 0 && value != 1 && value != 16 && value != 32)
            return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: sub must be 0, 1, 16 or 32");
        ctx->force_sub = value;
        return TWM_OK;
    }
    if (strcmp(key, "prefill_bm") == 0) {
        if (value != 0 && value != 64 && value != 128 && value != 192)
            return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: prefill_bm must be 0, 64, 128 or 192");
        ctx->prefill_bm = value;
        return TWM_OK;
    }
    if (strcmp(key, "prefill_sk") == 0) {
        if (value != 0 && value != 1 && value != 128 && value != 256)
            return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: prefill_sk must be 0, 1, 128 or 256");
        ctx->prefill_sk = value;
        return TWM_OK;
    }
    if (strcmp(key, "prefill_min_m") == 0) {
        if (value < 1) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: prefill_min_m must be >= 1");
        ctx->prefill_min_m = value;
        return TWM_OK;
    }
    if (strcmp(key, "weight_copies") == 0) {
        if (value < 0 || value > 3) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: weight_copies must be 0 .. 3");
        ctx->weight_copies = value;
        return TWM_OK;
    }
    if (strcmp(key, "dequant_src") == 0) {
        if (value != 0 && value != 1) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: dequant_src must be 0 or 1");
        ctx->dequant_src = value;
        return TWM_OK;
    }
    if (strcmp(key, "m1_exact") == 0) {
        if (value != 0 && value != 1) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: m1_exact must be 0 or 1");
        ctx->m1_exact = value;
        return TWM_OK;
    }
    if (strcmp(key, "m1_splits") == 0) {
        if (value < 0 || value > 64) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: m1_splits must be 0 .. 64");
        ctx->m1_splits = value;
        return TWM_OK;
    }
    if (strcmp(key, "batch_rounded") == 0) {
        if (value != 0 && value != 1) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: batch_rounded must be 0 or 1");
        ctx->batch_rounded = value;
        return TWM_OK;
    }
    if (strcmp(key, "kernel") == 0) {
        if (value < 0 || value > 4 || value == 1) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: kernel must be 0, 2, 3 or 4");
        ctx->force_kernel = value;
        return TWM_OK;
    }
    return api_fail(TWM_UNSUPPORTED_OP, "twm_ctx_set_option: unknown key %s", key);
}

/* ---- memory ---------------------------------------------------------------------------- */

void *twm_malloc(twm_ctx *ctx, size_t bytes)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_malloc: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_malloc: not allowed inside a graph capture"); return nullptr; }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes ? bytes : 4);
    if (e != hipSuccess) { api_fail(TWM_MEMORY_ERROR, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e)); return nullptr; }
    return p;
}

int twm_free(twm_ctx *ctx, void *ptr_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_free: null context");
    if (!ptr_dev) return TWM_OK;
    HIP_TRY(hipFree(ptr_dev), TWM_MEMORY_ERROR, "hipFree");
    return TWM_OK;
}

int twm_memcpy_h2d(twm_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_memcpy_h2d: null context");
    if (bytes == 0) return TWM_OK;
    if (!dst_dev || !src_host) return api_fail(TWM_INVALID_HANDLE, "twm_memcpy_h2d: null pointer");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_memcpy_h2d: not allowed inside a graph capture");
    HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream), TWM_MEMORY_ERROR, "memcpy h2d");
    HIP_TRY(hipStreamSynchronize(ctx->stream), TWM_DEVICE_ERROR, "memcpy h2d sync");
    return TWM_OK;
}

int twm_memcpy_d2h(twm_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_memcpy_d2h: null context");
    if (bytes == 0) return TWM_OK;
    if (!dst_host || !src_dev) return api_fail(TWM_INVALID_HANDLE, "twm_memcpy_d2h: null pointer");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_memcpy_d2h: not allowed inside a graph capture");
    HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream), TWM_MEMORY_ERROR, "memcpy d2h");
    HIP_TRY(hipStreamSynchronize(ctx->stream), TWM_DEVICE_ERROR, "memcpy d2h sync");
    return TWM_OK;
}

int twm_memcpy_d2d(twm_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_memcpy_d2d: null context");
    if (bytes == 0) return TWM_OK;
    if (!dst_dev || !src_dev) return api_fail(TWM_INVALID_HANDLE, "twm_memcpy_d2d: null pointer");
    HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream), TWM_MEMORY_ERROR, "memcpy d2d");
    return TWM_OK;
}

int twm_memset_zero(twm_ctx *ctx, void *ptr_dev, size_t bytes)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_memset_zero: null context");
    if (bytes == 0) return TWM_OK;
    if (!ptr_dev) return api_fail(TWM_INVALID_HANDLE, "twm_memset_zero: null pointer");
    if (bytes % 4 != 0 || ((uintptr_t)ptr_dev & 3) != 0)
        return api_fail(TWM_SHAPE_ERROR, "twm_memset_zero: pointer and size must be multiples of 4 bytes");
    HIP_TRY(launch_fill_zero(ctx->stream, ptr_dev, bytes), TWM_DEVICE_ERROR, "fill kernel launch");
    return TWM_OK;
}

/* ---- events ------------------------------------------------------------------------------ */

void *twm_event_create(twm_ctx *ctx)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_event_create: null context"); return nullptr; }
    hipEvent_t ev = nullptr;
    hipError_t e = hipEventCreate(&ev);
    if (e != hipSuccess) { api_fail(TWM_DEVICE_ERROR, "hipEventCreate: %s", hipGetErrorString(e)); return nullptr; }
    return (void *)ev;
}

int twm_event_destroy(twm_ctx *ctx, void *event)
{
    if (!ctx || !event) return api_fail(TWM_INVALID_HANDLE, "twm_event_destroy: null argument");
    HIP_TRY(hipEventDestroy((hipEvent_t)event), TWM_DEVICE_ERROR, "hipEventDestroy");
    return TWM_OK;
}

int twm_event_record(twm_ctx *ctx, void *event)
{
    if (!ctx || !event) return api_fail(TWM_INVALID_HANDLE, "twm_event_record: null argument");
    HIP_TRY(hipEventRecord((hipEvent_t)event, ctx->stream), TWM_DEVICE_ERROR, "hipEventRecord");
    return TWM_OK;
}

int twm_event_elapsed_ms(twm_ctx *ctx, void *start, void *stop, float *ms_out)
{
    if (!ctx || !start || !stop || !ms_out) return api_fail(TWM_INVALID_HANDLE, "twm_event_elapsed_ms: null argument");
    HIP_TRY(hipEventSynchronize((hipEvent_t)stop), TWM_DEVICE_ERROR, "hipEventSynchronize");
    HIP_TRY(hipEventElapsedTime(ms_out, (hipEvent_t)start, (hipEvent_t)stop), TWM_DEVICE_ERROR, "hipEventElapsedTime");
    return TWM_OK;
}

/* ---- format operations -------------------------------------------------------------------- */

extern "C++" int twm::check_kn(const char *who, uint32_t k, uint32_t n)
{
    if (k % 32 != 0) return api_fail(TWM_SHAPE_ERROR, "%s: K (%u) must be divisible by 32", who, k);
    if ((uint64_t)(k / 32) * n * 16 > (1ull << 40)) return api_fail(TWM_SHAPE_ERROR, "%s: K x N too large", who);
    return TWM_OK;
}

int twm_quantize_weights_q4_0(twm_ctx *ctx, const float *w_kn_dev, uint32_t k, uint32_t n, uint8_t *q4_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_quantize_weights_q4_0: null context");
    if (int rc = check_kn("twm_quantize_weights_q4_0", k, n)) return rc;
    if (k == 0 || n == 0) return TWM_OK;
    if (!w_kn_dev || !q4_dev) return api_fail(TWM_INVALID_HANDLE, "twm_quantize_weights_q4_0: null pointer");
    HIP_TRY(launch_quantize_q4_0(ctx->stream, w_kn_dev, k, n, q4_dev), TWM_DEVICE_ERROR, "quantize launch");
    return TWM_OK;
}

int twm_reorder_to_tw_marlin(twm_ctx *ctx, const uint8_t *q4_dev, uint32_t k, uint32_t n, uint8_t *packed_dev,
                             uint16_t *scales_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_reorder_to_tw_marlin: null context");
    if (int rc = check_kn("twm_reorder_to_tw_marlin", k, n)) return rc;
    if (k == 0 || n == 0) return TWM_OK;
    if (!q4_dev || !packed_dev || !scales_dev) return api_fail(TWM_INVALID_HANDLE, "twm_reorder_to_tw_marlin: null pointer");
    HIP_TRY(launch_reorder(ctx->stream, q4_dev, k, n, packed_dev, scales_dev), TWM_DEVICE_ERROR, "reorder launch");
    return TWM_OK;
}

int twm_quantize_f32_to_tw_marlin(twm_ctx *ctx, const float *w_dev, int w_is_nk, uint32_t k, uint32_t n,
                                  uint8_t *packed_dev, uint16_t *scales_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_quantize_f32_to_tw_marlin: null context");
    if (int rc = check_kn("twm_quantize_f32_to_tw_marlin", k, n)) return rc;
    if (k == 0 || n == 0) return TWM_OK;
    if (!w_dev || !packed_dev || !scales_dev)
        return api_fail(TWM_INVALID_HANDLE, "twm_quantize_f32_to_tw_marlin: null pointer");
    HIP_TRY(launch_quantize_twm(ctx->stream, w_dev, w_is_nk, k, n, packed_dev, scales_dev), TWM_DEVICE_ERROR,
            "quantize launch");
    return TWM_OK;
}

int twm_fuse_tw_marlin_n(twm_ctx *ctx, const uint8_t *const *packed_devs, const uint16_t *const *scales_devs, uint32_t k,
                         const uint32_t *ns, uint32_t count, uint8_t *packed_out_dev, uint16_t *scales_out_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_fuse_tw_marlin_n: null context");
    if (!packed_devs || !scales_devs || !ns) return api_fail(TWM_INVALID_HANDLE, "twm_fuse_tw_marlin_n: null array");
    uint64_t total = 0;
    for (uint32_t i = 0; i < count; i++) total += ns[i];
    if (total > 0xFFFFFFFFull) return api_fail(TWM_SHAPE_ERROR, "twm_fuse_tw_marlin_n: fused N overflows u32");
    if (int rc = check_kn("twm_fuse_tw_marlin_n", k, (uint32_t)total)) return rc;
    if (total == 0 || k == 0) return TWM_OK;
    if (!packed_out_dev || !scales_out_dev) return api_fail(TWM_INVALID_HANDLE, "twm_fuse_tw_marlin_n: null output");
    uint32_t off = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (ns[i] == 0) continue;
        if (!packed_devs[i] || !scales_devs[i]) return api_fail(TWM_INVALID_HANDLE, "twm_fuse_tw_marlin_n: null input %u", i);
        HIP_TRY(launch_fuse_one(ctx->stream, packed_devs[i], scales_devs[i], k / 32, ns[i], (uint32_t)total, off,
                                packed_out_dev, scales_out_dev),
                TWM_DEVICE_ERROR, "fuse launch");
        off += ns[i];
    }
    return TWM_OK;
}

static int dequant_common(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev, uint32_t k, uint32_t n,
                          void *out, bool f16)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_dequant: null context");
    if (int rc = check_kn("twm_dequant", k, n)) return rc;
    if (k == 0 || n == 0) return TWM_OK;
    if (!packed_dev || !scales_dev || !out) return api_fail(TWM_INVALID_HANDLE, "twm_dequant: null pointer");
    HIP_TRY(launch_dequant(ctx->stream, packed_dev, scales_dev, k, n, out, f16), TWM_DEVICE_ERROR, "dequant launch");
    return TWM_OK;
}

int twm_dequant_to_f16(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev, uint32_t k, uint32_t n,
                       uint16_t *out_kn_dev)
{
    return dequant_common(ctx, packed_dev, scales_dev, k, n, out_kn_dev, true);
}

int twm_dequant_to_f32(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev, uint32_t k, uint32_t n,
                       float *out_kn_dev)
{
    return dequant_common(ctx, packed_dev, scales_dev, k, n, out_kn_dev, false);
}

int twm_split_qkv(twm_ctx *ctx, const float *qkv_dev, float *q_dev, float *k_dev, float *v_dev, uint32_t h,
                  uint32_t kv_dim, uint32_t batch)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_split_qkv: null context");
    if ((uint64_t)batch * ((uint64_t)h + 2ull * kv_dim) == 0) return TWM_OK;
    if (!qkv_dev || !q_dev || !k_dev || !v_dev) return api_fail(TWM_INVALID_HANDLE, "twm_split_qkv: null pointer");
    HIP_TRY(launch_split_qkv(ctx->stream, qkv_dev, q_dev, k_dev, v_dev, h, kv_dim, batch), TWM_DEVICE_ERROR,
            "split_qkv launch");
    return TWM_OK;
}

int twm_argmax_f32(twm_ctx *ctx, const float *input_dev, uint32_t rows, uint32_t cols, int32_t *out_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_argmax_f32: null context");
    if (rows == 0) return TWM_OK;
    if (!out_dev || (cols != 0 && !input_dev)) return api_fail(TWM_INVALID_HANDLE, "twm_argmax_f32: null pointer");
    HIP_TRY(launch_argmax(ctx->stream, input_dev, rows, cols, out_dev, ctx->ws, ctx->ws_bytes), TWM_DEVICE_ERROR, "argmax launch");
    return TWM_OK;
}

int twm_split_gate_up(twm_ctx *ctx, const float *gate_up_dev, float *gate_dev, float *up_dev, uint32_t ffn_dim,
                      uint32_t batch)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_split_gate_up: null context");
    if ((uint64_t)batch * ffn_dim == 0) return TWM_OK;
    if (!gate_up_dev || !gate_dev || !up_dev) return api_fail(TWM_INVALID_HANDLE, "twm_split_gate_up: null pointer");
    HIP_TRY(launch_split_gate_up(ctx->stream, gate_up_dev, gate_dev, up_dev, ffn_dim, batch), TWM_DEVICE_ERROR,
            "split_gate_up launch");
    return TWM_OK;
}

int twm_silu_mul(twm_ctx *ctx, const float *gate_dev, const float *up_dev, float *out_dev, size_t count)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_silu_mul: null context");
    if (count == 0) return TWM_OK;
    if (!gate_dev || !up_dev || !out_dev) return api_fail(TWM_INVALID_HANDLE, "twm_silu_mul: null pointer");
    HIP_TRY(launch_silu_mul(ctx->stream, gate_dev, up_dev, out_dev, count), TWM_DEVICE_ERROR, "silu_mul launch");
    return TWM_OK;
}

int twm_swiglu_rows(twm_ctx *ctx, const float *gate_up_dev, uint32_t batch, uint32_t ffn_dim, int paired, float *out_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_swiglu_rows: null context");
    if (paired && ffn_dim % kPairWidth != 0)
        return api_fail(TWM_SHAPE_ERROR, "twm_swiglu_rows: the paired order needs ffn_dim %% %u == 0, got %u", kPairWidth, ffn_dim);
    if ((uint64_t)ffn_dim * 2 > 0xFFFFFFFFull) return api_fail(TWM_SHAPE_ERROR, "twm_swiglu_rows: 2 * ffn_dim overflows u32");
    if ((uint64_t)batch * ffn_dim == 0) return TWM_OK;
    if (!gate_up_dev || !out_dev) return api_fail(TWM_INVALID_HANDLE, "twm_swiglu_rows: null pointer");
    HIP_TRY(launch_swiglu_rows(ctx->stream, gate_up_dev, out_dev, ffn_dim, batch, paired != 0), TWM_DEVICE_ERROR,
            "swiglu_rows launch");
    return TWM_OK;
}

static int check_pair_args(const char *who, uint32_t k, uint32_t ffn_dim)
{
    if (ffn_dim % kPairWidth != 0) return api_fail(TWM_SHAPE_ERROR, "%s: ffn_dim must be a multiple of %u, got %u", who, kPairWidth, ffn_dim);
    if ((uint64_t)ffn_dim * 2 > 0xFFFFFFFFull) return api_fail(TWM_SHAPE_ERROR, "%s: 2 * ffn_dim overflows u32", who);
    return check_kn(who, k, ffn_dim * 2);
}

int twm_pair_gate_up(twm_ctx *ctx, const uint8_t *gate_packed_dev, const uint16_t *gate_scales_dev,
                     const uint8_t *up_packed_dev, const uint16_t *up_scales_dev, uint32_t k, uint32_t ffn_dim,
                     uint8_t *packed_out_dev, uint16_t *scales_out_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_pair_gate_up: null context");
    if (int rc = check_pair_args("twm_pair_gate_up", k, ffn_dim)) return rc;
    if (k == 0 || ffn_dim == 0) return TWM_OK;
    if (!gate_packed_dev || !gate_scales_dev || !up_packed_dev || !up_scales_dev || !packed_out_dev || !scales_out_dev)
        return api_fail(TWM_INVALID_HANDLE, "twm_pair_gate_up: null pointer");
    HIP_TRY(launch_pair_gate_up(ctx->stream, gate_packed_dev, gate_scales_dev, up_packed_dev, up_scales_dev, k / 32,
                                ffn_dim, packed_out_dev, scales_out_dev),
            TWM_DEVICE_ERROR, "pair_gate_up launch");
    return TWM_OK;
}

/* ---- GEMV on the reference layout ------------------------------------------------------- */

void twm_pick_splits_reference(uint32_t k, uint32_t n, uint32_t *n_blocks, uint32_t *splits, uint32_t *groups_per_split)
{
    uint32_t groups = k / 32u;
    uint32_t nb = (n + 255u) / 256u;
    uint32_t sp;
    if (k < 2048u || nb >= 128u) {
        sp = 1;
    } else {
        uint32_t max_splits = groups / 8u;
        if (max_splits < 1u) max_splits = 1u;
        sp = (256u + nb - 1u) / nb;
        if (sp < 1u) sp = 1u;
        if (sp > max_splits) sp = max_splits;
    }
    if (n_blocks) *n_blocks = nb;
    if (splits) *splits = sp;
    if (groups_per_split) *groups_per_split = (groups + sp - 1u) / sp;
}

extern "C++" int twm::m1_dispatch(const M1Env &env, const char *who, const float *a_dev, const uint8_t *packed_dev,
                       const uint16_t *scales_dev, float *c_dev, uint32_t n, uint32_t k)
{
    if (int rc = check_kn(who, k, n)) return rc;
    if (n == 0) return TWM_OK;
    if (!c_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null output", who);
    if (k == 0) {
        HIP_TRY(launch_fill_zero(env.stream, c_dev, (size_t)n * 4), TWM_DEVICE_ERROR, "fill kernel launch");
        return TWM_OK;
    }
    if (!a_dev || !packed_dev || !scales_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null input", who);
    // the reference kernel reads a record as four 32-bit words (quantize.rs:1227-1228): 4-byte alignment is its own limit
    if (((uintptr_t)packed_dev & 3) != 0) return api_fail(TWM_SHAPE_ERROR, "%s: packed must be 4-byte aligned", who);
    if (env.exact || ((uintptr_t)a_dev & 15) != 0 || ((uintptr_t)packed_dev & 15) != 0) {
        // f32 activations, f32 FMAs, the reference kernel's order and its own split-K rule (float atomics)
        uint32_t nb, sp, gps;
        twm_pick_splits_reference(k, n, &nb, &sp, &gps);
        HIP_TRY(launch_ref_gemv(env.stream, a_dev, packed_dev, scales_dev, c_dev, n, k, sp, gps), TWM_DEVICE_ERROR, "gemv launch");
        return TWM_OK;
    }
    // the M <= 4 MFMA kernels reading the reference's arrays as they are (f32 activations as two f16 terms)
    uint32_t n_pad = ((n + 63) / 64) * 64, k_chunks = (k / 32 + kChunkGroups - 1) / kChunkGroups;
    // On the reference's arrays a wave's four group rows of a chunk are N x 16 bytes apart, and many waves in flight
    // with one pass each pay better than on the contiguous copy: the sub-tile kernel with sixteen waves on 32
    // columns as long as every wave gets a single pass (K <= 4096), or with 16 columns when 64-column tiles number no
    // more than 64.  Deeper wide matrices keep the 64-column kernel and its split-K (8192 -> 57344: 46.6 against
    // 63.7 us).  Fitted to sweeps over the
    // Qwen2.5-7B, Llama-3-8B, 13B and 70B projections; option "sub" = 1 keeps the 64-column kernel.
    const uint32_t tiles64 = n_pad / 64, passes16 = (k_chunks + 3) / 4, passes32 = (k_chunks + 1) / 2;
    uint32_t sub = tiles64 <= 64 ? 16 : 32, sub_waves = (sub == 16 && passes16 <= 8) ? 8 : 16;
    // (on 16 columns a deeper K runs the pipelined pass loop on sixteen waves: 18944 -> 3584 12.5 against 12.8 us,
    // 14336 -> 4096 10.8 against 11.7)
    bool use_sub = env.force_sub != 1 && (sub == 16 || passes32 <= 16);
    if (env.force_sub >= 16) {
        sub = (uint32_t)env.force_sub;
        sub_waves = 8;
        use_sub = true;
    }
    if (use_sub) {
        uint32_t sp = env.splits ? (uint32_t)env.splits : 1;
        if (env.force_waves) sub_waves = (uint32_t)env.force_waves;
        if (sp > k_chunks) sp = k_chunks;
        while (sp > 1 && (size_t)sp * n_pad * 4 > env.ws_bytes) sp--;
        if (n_pad / sub > env.n_counters) sp = 1;
        if (sp > 1 && env.clear_counters)
            HIP_TRY(launch_fill_zero(env.stream, env.counters, (size_t)(n_pad / sub) * 4), TWM_DEVICE_ERROR, "fill kernel launch");
        HIP_TRY(launch_gemv4s_ref(env.stream, packed_dev, scales_dev, k, n, a_dev, c_dev, env.ws, env.counters, sub, sub_waves, sp),
                TWM_DEVICE_ERROR, "sub-tile gemv launch");
        return TWM_OK;
    }
    DecodePlan plan;
    plan.lane_col = 1;
    plan.nt = 1;
    plan.waves = 8;
    plan.splits = 1;
    if (tiles64 < 256) {
        plan.waves = 16;
        while (tiles64 * plan.splits * 2 <= 256 && k_chunks >= plan.splits * 2 * 8) plan.splits *= 2;
    }
    if (env.force_waves) plan.waves = (uint32_t)env.force_waves;
    if (env.splits) plan.splits = (uint32_t)env.splits;
    if (plan.splits > k_chunks) plan.splits = k_chunks;
    while (plan.splits > 1 && (size_t)plan.splits * n_pad * 4 > env.ws_bytes) plan.splits--;
    if (tiles64 > env.n_counters) plan.splits = 1;
    if (plan.splits > 1 && env.clear_counters)
        HIP_TRY(launch_fill_zero(env.stream, env.counters, (size_t)tiles64 * 4), TWM_DEVICE_ERROR, "fill kernel launch");
    HIP_TRY(launch_gemv4_ref(env.stream, packed_dev, scales_dev, k, n, a_dev, c_dev, env.ws, env.counters, plan.waves,
                             plan.splits),
            TWM_DEVICE_ERROR, "gemv launch");
    return TWM_OK;
}

int twm_gemm_tw_marlin_m1(twm_ctx *ctx, const float *a_dev, const uint8_t *packed_dev, const uint16_t *scales_dev,
                          float *c_dev, uint32_t n, uint32_t k)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_tw_marlin_m1: null context");
    const M1Env env = {ctx->stream, ctx->m1_exact, ctx->m1_splits, ctx->force_sub, ctx->force_waves,
                       ctx->ws, ctx->ws_bytes, ctx->counters, ctx->n_counters, false};
    return m1_dispatch(env, "twm_gemm_tw_marlin_m1", a_dev, packed_dev, scales_dev, c_dev, n, k);
}

int twm_gemm_tw_marlin_m1_from_buffer(twm_ctx *ctx, const float *a_dev, const uint8_t *packed_buf_dev,
                                      size_t packed_offset, const uint16_t *scales_buf_dev, size_t scales_offset,
                                      float *c_dev, uint32_t n, uint32_t k)
{
    if (!packed_buf_dev || !scales_buf_dev)
        return api_fail(TWM_INVALID_HANDLE, "twm_gemm_tw_marlin_m1_from_buffer: null slab");
    return twm_gemm_tw_marlin_m1(ctx, a_dev, packed_buf_dev + packed_offset, scales_buf_dev + scales_offset, c_dev, n, k);
}

/* ---- repacked weights ----------------------------------------------------------------------- */

static twm_weight *weight_alloc(twm_ctx *ctx, uint32_t k, uint32_t n)
{
    twm_weight *w = new (std::nothrow) twm_weight();
    if (!w) { api_fail(TWM_MEMORY_ERROR, "twm_weight: out of host memory"); return nullptr; }
    w->ctx = ctx;
    w->k = k;
    w->n = n;
    w->groups = k / 32;
    uint32_t n_pad = ((n + kNPadTo - 1) / kNPadTo) * kNPadTo;
    w->n_tiles = n_pad / kTileN;
    w->k_chunks = (w->groups + kChunkGroups - 1) / kChunkGroups;
    size_t tiles = (size_t)w->n_tiles * w->k_chunks;
    w->copy_bytes = tiles * (1024 + 128);  // nibbles + scales: the same in either order
    w->bytes = 0;
    w->qw = w->sc = w->cq = nullptr;
    w->paired = false;
    memset(w->tuned, 0, sizeof w->tuned);
    return w;
}

// device memory for the copies in `mask` that the handle does not hold yet (contents undefined)
static int weight_alloc_copies(twm_weight *w, int mask, const char *who)
{
    if (w->copy_bytes == 0) return TWM_OK;
    if ((mask & kCopyTile) && !w->qw) {
        hipError_t e = hipMalloc(&w->qw, w->copy_bytes);
        if (e != hipSuccess) { w->qw = nullptr; return api_fail(TWM_MEMORY_ERROR, "%s: hipMalloc(%zu): %s", who, w->copy_bytes, hipGetErrorString(e)); }
        w->sc = (char *)w->qw + (size_t)w->n_tiles * w->k_chunks * 1024;
        w->bytes += w->copy_bytes;
    }
    if ((mask & kCopyCol) && !w->cq) {
        hipError_t e = hipMalloc(&w->cq, w->copy_bytes);
        if (e != hipSuccess) { w->cq = nullptr; return api_fail(TWM_MEMORY_ERROR, "%s: hipMalloc(%zu): %s", who, w->copy_bytes, hipGetErrorString(e)); }
        w->bytes += w->copy_bytes;
    }
    return TWM_OK;
}

static void weight_release(twm_weight *w)
{
    if (w->qw) (void)hipFree(w->qw);
    if (w->cq) (void)hipFree(w->cq);
    delete w;
}

static int copies_of(const twm_weight *w) { return (w->qw ? kCopyTile : 0) | (w->cq ? kCopyCol : 0); }

// Makes sure the handle holds the copies in `mask`, building a missing one from the other on the context's stream.
// Allocates, so not inside a graph capture: a caller that captures its launches asks for the copies before
// (twm_weight_ensure, or option "weight_copies" when the handle is made).
static int weight_ensure(twm_ctx *ctx, const twm_weight *cw, int mask, const char *who)
{
    twm_weight *w = const_cast<twm_weight *>(cw);  // (the handle is the library's own object; callers see it opaque)
    const int have = copies_of(w), missing = mask & ~have;
    if (!missing || w->copy_bytes == 0) return TWM_OK;
    if (ctx->capturing)
        return api_fail(TWM_UNSUPPORTED_OP, "%s: this call needs the weight's %s copy, which the handle does not hold, and building it "
                        "allocates: call twm_weight_ensure before the capture", who, (missing & kCopyTile) ? "16-column tile" : "column-lane");
    if (!have) return api_fail(TWM_INVALID_HANDLE, "%s: the weight holds no copy at all", who);
    if (int rc = weight_alloc_copies(w, missing, who)) return rc;
    hipError_t e = (missing & kCopyTile) ? launch_col_to_tile(ctx->stream, w->cq, w->n_tiles, w->k_chunks, w->qw, w->sc)
                                         : launch_tile_to_col(ctx->stream, w->qw, w->sc, w->n_tiles, w->k_chunks, w->cq);
    if (e != hipSuccess) return api_fail(TWM_DEVICE_ERROR, "%s: building the second weight copy: %s", who, hipGetErrorString(e));
    return TWM_OK;
}

int twm_weight_ensure(twm_ctx *ctx, twm_weight *w, int copies)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_ensure: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_weight_ensure: weight belongs to another context");
    if (copies < 1 || copies > 3) return api_fail(TWM_SHAPE_ERROR, "twm_weight_ensure: copies is 1 (16-column tiles), 2 (column-lane) or 3 (both)");
    return weight_ensure(ctx, w, copies, "twm_weight_ensure");
}

int twm_weight_drop(twm_ctx *ctx, twm_weight *w, int copies)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_drop: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_weight_drop: weight belongs to another context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_weight_drop: not allowed inside a graph capture");
    if (copies != kCopyTile && copies != kCopyCol) return api_fail(TWM_SHAPE_ERROR, "twm_weight_drop: copies is 1 (16-column tiles) or 2 (column-lane)");
    if (w->copy_bytes == 0 || !(copies_of(w) & copies)) return TWM_OK;
    if (copies_of(w) == copies) return api_fail(TWM_SHAPE_ERROR, "twm_weight_drop: that is the only copy the handle holds");
    HIP_TRY(hipStreamSynchronize(ctx->stream), TWM_DEVICE_ERROR, "twm_weight_drop: sync");
    if (copies == kCopyTile) { (void)hipFree(w->qw); w->qw = w->sc = nullptr; }
    else { (void)hipFree(w->cq); w->cq = nullptr; }
    w->bytes -= w->copy_bytes;
    return TWM_OK;
}

int twm_weight_copies(const twm_weight *w) { return w ? copies_of(w) : 0; }

twm_weight *twm_weight_from_device(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev, uint32_t k,
                                   uint32_t n)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_weight_from_device: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_weight_from_device: not allowed inside a graph capture"); return nullptr; }
    if (check_kn("twm_weight_from_device", k, n)) return nullptr;
    if ((uint64_t)k * n != 0 && (!packed_dev || !scales_dev)) {
        api_fail(TWM_INVALID_HANDLE, "twm_weight_from_device: null pointer");
        return nullptr;
    }
    if (((uintptr_t)packed_dev & 3) != 0) { api_fail(TWM_SHAPE_ERROR, "twm_weight_from_device: packed must be 4-byte aligned"); return nullptr; }
    twm_weight *w = weight_alloc(ctx, k, n);
    if (!w) return nullptr;
    const int mask = ctx->weight_copies ? ctx->weight_copies : (kCopyTile | kCopyCol);
    if (weight_alloc_copies(w, mask, "twm_weight_from_device")) { weight_release(w); return nullptr; }
    if (w->copy_bytes) {
        hipError_t e = hipSuccess;
        if (w->qw) e = launch_repack(ctx->stream, packed_dev, scales_dev, k, n, w->qw, w->sc, w->n_tiles, w->k_chunks);
        if (e == hipSuccess && w->cq)
            e = launch_repack_col(ctx->stream, packed_dev, scales_dev, k, n, w->cq, w->n_tiles * kTileN, w->k_chunks);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) {
            api_fail(TWM_DEVICE_ERROR, "twm_weight_from_device: repack: %s", hipGetErrorString(e));
            weight_release(w);
            return nullptr;
        }
    }
    return w;
}

// Fusing along N on the repacked copies is block copying: the column-lane copy is tile-major (one contiguous run per
// input), the 16-column tile copy chunk-major (one 2-D copy per input: k_chunks rows of the input's tiles).
twm_weight *twm_weight_fuse_n(twm_ctx *ctx, const twm_weight *const *parts, uint32_t count)
{
    const char *who = "twm_weight_fuse_n";
    if (!ctx || !parts || count == 0) { api_fail(TWM_INVALID_HANDLE, "%s: null argument", who); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "%s: not allowed inside a graph capture", who); return nullptr; }
    uint64_t total = 0;
    for (uint32_t i = 0; i < count; i++) {
        const twm_weight *p = parts[i];
        if (!p) { api_fail(TWM_INVALID_HANDLE, "%s: part %u is null", who, i); return nullptr; }
        if (p->ctx != ctx) { api_fail(TWM_INVALID_HANDLE, "%s: part %u belongs to another context", who, i); return nullptr; }
        if (p->k != parts[0]->k) { api_fail(TWM_SHAPE_ERROR, "%s: part %u has K = %u, part 0 has %u", who, i, p->k, parts[0]->k); return nullptr; }
        if (p->paired) { api_fail(TWM_UNSUPPORTED_OP, "%s: part %u is a paired gate/up weight", who, i); return nullptr; }
        if (i + 1 < count && p->n % kNPadTo != 0) {
            api_fail(TWM_SHAPE_ERROR, "%s: part %u has N = %u; every part but the last must be a multiple of %u columns "
                     "(fuse the arrays with twm_fuse_tw_marlin_n instead)", who, i, p->n, kNPadTo);
            return nullptr;
        }
        total += p->n;
    }
    if (total > 0xFFFFFFFFull) { api_fail(TWM_SHAPE_ERROR, "%s: fused N overflows u32", who); return nullptr; }
    if (check_kn(who, parts[0]->k, (uint32_t)total)) return nullptr;
    twm_weight *w = weight_alloc(ctx, parts[0]->k, (uint32_t)total);
    if (!w) return nullptr;
    const int mask = ctx->weight_copies ? ctx->weight_copies : (kCopyTile | kCopyCol);
    for (uint32_t i = 0; i < count; i++)
        if (weight_ensure(ctx, parts[i], mask, who)) { weight_release(w); return nullptr; }
    if (weight_alloc_copies(w, mask, who)) { weight_release(w); return nullptr; }
    hipError_t e = hipSuccess;
    uint32_t t16 = 0;  // 16-column tiles before this part
    for (uint32_t i = 0; i < count && e == hipSuccess && w->copy_bytes; i++) {
        const twm_weight *p = parts[i];
        if (p->n_tiles == 0) continue;
        if (w->cq)
            e = hipMemcpyAsync((char *)w->cq + (size_t)(t16 / 4) * w->k_chunks * kColBlockBytes, p->cq,
                               (size_t)(p->n_tiles / 4) * p->k_chunks * kColBlockBytes, hipMemcpyDeviceToDevice, ctx->stream);
        if (e == hipSuccess && w->qw)
            e = hipMemcpy2DAsync((char *)w->qw + (size_t)t16 * 1024, (size_t)w->n_tiles * 1024, p->qw, (size_t)p->n_tiles * 1024,
                                 (size_t)p->n_tiles * 1024, w->k_chunks, hipMemcpyDeviceToDevice, ctx->stream);
        if (e == hipSuccess && w->qw)
            e = hipMemcpy2DAsync((char *)w->sc + (size_t)t16 * 128, (size_t)w->n_tiles * 128, p->sc, (size_t)p->n_tiles * 128,
                                 (size_t)p->n_tiles * 128, w->k_chunks, hipMemcpyDeviceToDevice, ctx->stream);
        t16 += p->n_tiles;
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        api_fail(TWM_DEVICE_ERROR, "%s: copy: %s", who, hipGetErrorString(e));
        weight_release(w);
        return nullptr;
    }
    return w;
}

twm_weight *twm_weight_upload(twm_ctx *ctx, const uint8_t *packed_host, const uint16_t *scales_host, uint32_t k,
                              uint32_t n)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_weight_upload: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_weight_upload: not allowed inside a graph capture"); return nullptr; }
    if (check_kn("twm_weight_upload", k, n)) return nullptr;
    size_t pbytes = (size_t)(k / 32) * n * 16, sbytes = (size_t)(k / 32) * n * 2;
    if (pbytes == 0) return twm_weight_from_device(ctx, nullptr, nullptr, k, n);
    if (!packed_host || !scales_host) { api_fail(TWM_INVALID_HANDLE, "twm_weight_upload: null pointer"); return nullptr; }
    void *stage = nullptr;
    hipError_t e = hipMalloc(&stage, pbytes + sbytes);
    if (e != hipSuccess) { api_fail(TWM_MEMORY_ERROR, "twm_weight_upload: staging hipMalloc: %s", hipGetErrorString(e)); return nullptr; }
    uint8_t *p = (uint8_t *)stage;
    uint16_t *s = (uint16_t *)(p + pbytes);
    twm_weight *w = nullptr;
    if (twm_memcpy_h2d(ctx, p, packed_host, pbytes) == TWM_OK && twm_memcpy_h2d(ctx, s, scales_host, sbytes) == TWM_OK)
        w = twm_weight_from_device(ctx, p, s, k, n);
    (void)hipFree(stage);
    return w;
}

twm_weight *twm_weight_gate_up(twm_ctx *ctx, const uint8_t *gate_packed_dev, const uint16_t *gate_scales_dev,
                               const uint8_t *up_packed_dev, const uint16_t *up_scales_dev, uint32_t k, uint32_t ffn_dim)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_weight_gate_up: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_weight_gate_up: not allowed inside a graph capture"); return nullptr; }
    if (check_pair_args("twm_weight_gate_up", k, ffn_dim)) return nullptr;
    uint32_t n = ffn_dim * 2;
    size_t pbytes = (size_t)(k / 32) * n * 16, sbytes = (size_t)(k / 32) * n * 2;
    twm_weight *w = nullptr;
    if (pbytes == 0) {
        w = twm_weight_from_device(ctx, nullptr, nullptr, k, n);
    } else {
        void *stage = nullptr;
        hipError_t e = hipMalloc(&stage, pbytes + sbytes);
        if (e != hipSuccess) { api_fail(TWM_MEMORY_ERROR, "twm_weight_gate_up: staging hipMalloc: %s", hipGetErrorString(e)); return nullptr; }
        uint8_t *p = (uint8_t *)stage;
        uint16_t *sc = (uint16_t *)(p + pbytes);
        if (twm_pair_gate_up(ctx, gate_packed_dev, gate_scales_dev, up_packed_dev, up_scales_dev, k, ffn_dim, p, sc) == TWM_OK)
            w = twm_weight_from_device(ctx, p, sc, k, n);  // synchronises the stream before returning
        else
            (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(stage);
    }
    if (w) w->paired = true;
    return w;
}

int twm_weight_is_paired(const twm_weight *w) { return w && w->paired ? 1 : 0; }

void twm_weight_destroy(twm_weight *w)
{
    if (!w) return;
    if (w->qw || w->cq) (void)hipStreamSynchronize(w->ctx->stream);
    weight_release(w);
}

int twm_weight_dims(const twm_weight *w, uint32_t *k, uint32_t *n)
{
    if (!w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_dims: null weight");
    if (k) *k = w->k;
    if (n) *n = w->n;
    return TWM_OK;
}

size_t twm_weight_bytes(const twm_weight *w) { return w ? w->bytes : 0; }

/* ---- repacked weights as a byte blob (for an on-disk cache) -------------------------------- */

// 64-byte little-endian header followed by the device allocation as it is.
struct WeightBlobHeader {
    char magic[8];          // "TWMWGT01"
    uint32_t layout;        // changes whenever the repacked byte order does
    uint32_t k, n, n_tiles, k_chunks;
    uint32_t paired;
    uint64_t payload_bytes;
    uint64_t checksum;      // of the payload
    uint8_t copies;         // payload: the 16-column tile copy (bit 0) and / or the column-lane copy (bit 1), in this order
    uint8_t reserved[15];
};
static_assert(sizeof(WeightBlobHeader) == 64, "blob header is 64 bytes");
static const char kBlobMagic[8] = {'T', 'W', 'M', 'W', 'G', 'T', '0', '1'};
static const uint32_t kBlobLayout = 5;
static const size_t kBlobTrailer = sizeof(TunedPlan) * kTuneBuckets;  // the measured plans (twm_weight_tune), after the payload

// Four independent multiply-rotate lanes over 64-bit words (memory-bound on the host), folded at the end.
static uint64_t blob_checksum(const uint8_t *p, size_t bytes)
{
    uint64_t h[4] = {0x9E3779B97F4A7C15ull, 0xC2B2AE3D27D4EB4Full, 0x165667B19E3779F9ull, 0x27D4EB2F165667C5ull};
    size_t words = bytes / 8, i = 0;
    for (; i + 4 <= words; i += 4) {
        for (int l = 0; l < 4; l++) {
            uint64_t v;
            memcpy(&v, p + (i + l) * 8, 8);
            h[l] = (h[l] ^ v) * 0x100000001B3ull;
            h[l] = (h[l] << 29) | (h[l] >> 35);
        }
    }
    uint64_t tail = 0;
    for (size_t b = i * 8; b < bytes; b++) tail = tail * 257 + p[b];
    uint64_t r = tail ^ (uint64_t)bytes;
    for (int l = 0; l < 4; l++) r = (r ^ h[l]) * 0xFF51AFD7ED558CCDull + (r >> 31);
    return r;
}

size_t twm_weight_blob_bytes(const twm_weight *w) { return w ? sizeof(WeightBlobHeader) + w->bytes + kBlobTrailer : 0; }

int twm_weight_export(twm_ctx *ctx, const twm_weight *w, void *blob_host, size_t blob_bytes)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_export: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_weight_export: weight belongs to another context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_weight_export: not allowed inside a graph capture");
    if (!blob_host) return api_fail(TWM_INVALID_HANDLE, "twm_weight_export: null buffer");
    if (blob_bytes != twm_weight_blob_bytes(w))
        return api_fail(TWM_SHAPE_ERROR, "twm_weight_export: the buffer must hold %zu bytes, got %zu", twm_weight_blob_bytes(w), blob_bytes);
    uint8_t *payload = (uint8_t *)blob_host + sizeof(WeightBlobHeader);
    size_t at = 0;
    if (w->qw) {
        if (int rc = twm_memcpy_d2h(ctx, payload + at, w->qw, w->copy_bytes)) return rc;
        at += w->copy_bytes;
    }
    if (w->cq) {
        if (int rc = twm_memcpy_d2h(ctx, payload + at, w->cq, w->copy_bytes)) return rc;
        at += w->copy_bytes;
    }
    WeightBlobHeader hd;
    memset(&hd, 0, sizeof hd);
    memcpy(hd.magic, kBlobMagic, 8);
    hd.layout = kBlobLayout;
    hd.k = w->k;
    hd.n = w->n;
    hd.n_tiles = w->n_tiles;
    hd.k_chunks = w->k_chunks;
    hd.paired = w->paired ? 1u : 0u;
    hd.payload_bytes = at;
    hd.checksum = blob_checksum(payload, at);
    hd.copies = (uint8_t)copies_of(w);
    memcpy(blob_host, &hd, sizeof hd);
    memcpy(payload + at, w->tuned, kBlobTrailer);
    return TWM_OK;
}

twm_weight *twm_weight_import(twm_ctx *ctx, const void *blob_host, size_t blob_bytes)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_weight_import: null context"); return nullptr; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_weight_import: not allowed inside a graph capture"); return nullptr; }
    if (!blob_host || blob_bytes < sizeof(WeightBlobHeader)) { api_fail(TWM_SHAPE_ERROR, "twm_weight_import: blob shorter than its header"); return nullptr; }
    WeightBlobHeader hd;
    memcpy(&hd, blob_host, sizeof hd);
    if (memcmp(hd.magic, kBlobMagic, 8) != 0) { api_fail(TWM_SHAPE_ERROR, "twm_weight_import: not a repacked-weight blob (bad magic)"); return nullptr; }
    if (hd.layout != kBlobLayout) {
        api_fail(TWM_UNSUPPORTED_OP, "twm_weight_import: blob has layout %u, this library writes %u: repack from the TW-Marlin arrays", hd.layout, kBlobLayout);
        return nullptr;
    }
    if (check_kn("twm_weight_import", hd.k, hd.n)) return nullptr;
    twm_weight *w = weight_alloc(ctx, hd.k, hd.n);
    if (!w) return nullptr;
    const uint8_t *payload = (const uint8_t *)blob_host + sizeof(WeightBlobHeader);
    const int held = hd.copies & 3, n_held = (held & 1) + (held >> 1);
    bool ok = w->n_tiles == hd.n_tiles && w->k_chunks == hd.k_chunks && hd.copies <= 3 &&
              (w->copy_bytes == 0 ? hd.payload_bytes == 0 : (n_held >= 1 && hd.payload_bytes == (uint64_t)n_held * w->copy_bytes)) &&
              blob_bytes == sizeof(WeightBlobHeader) + hd.payload_bytes + kBlobTrailer && hd.paired <= 1 &&
              (!hd.paired || hd.n % (2 * kPairWidth) == 0);
    if (!ok) api_fail(TWM_SHAPE_ERROR, "twm_weight_import: header does not describe a %u x %u weight of %zu bytes", hd.k, hd.n, blob_bytes);
    if (ok && blob_checksum(payload, (size_t)hd.payload_bytes) != hd.checksum) {
        ok = false;
        api_fail(TWM_SHAPE_ERROR, "twm_weight_import: checksum mismatch (corrupt or truncated blob)");
    }
    if (ok && w->copy_bytes) {
        ok = weight_alloc_copies(w, held, "twm_weight_import") == TWM_OK;
        size_t at = 0;
        if (ok && w->qw) { ok = twm_memcpy_h2d(ctx, w->qw, payload + at, w->copy_bytes) == TWM_OK; at += w->copy_bytes; }
        if (ok && w->cq) ok = twm_memcpy_h2d(ctx, w->cq, payload + at, w->copy_bytes) == TWM_OK;
    }
    if (!ok) {
        weight_release(w);
        return nullptr;
    }
    w->paired = hd.paired != 0;
    memcpy(w->tuned, payload + hd.payload_bytes, kBlobTrailer);
    for (TunedPlan &p : w->tuned)   // (a plan is a set of option values: anything outside their ranges is dropped)
        if (p.valid > 1 || p.kernel > 4 || p.kernel == 1 || p.nt > 4 || p.waves > 16 || p.sub_waves > 16 ||
            (p.sub != 0 && p.sub != 1 && p.sub != 16 && p.sub != 32) || (p.prefill_bm != 0 && p.prefill_bm != 64 && p.prefill_bm != 128 && p.prefill_bm != 192))
            memset(&p, 0, sizeof p);
    return w;
}

static WeightView view_of(const twm_weight *w)
{
    WeightView v;
    v.qw = w->qw;
    v.sc = w->sc;
    v.cq = w->cq;
    v.k = w->k;
    v.n = w->n;
    v.groups = w->groups;
    v.n_tiles = w->n_tiles;
    v.k_chunks = w->k_chunks;
    return v;
}

int twm_weight_dequant_f16(twm_ctx *ctx, const twm_weight *w, uint16_t *out_kn_dev)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_dequant_f16: null handle");
    if ((uint64_t)w->k * w->n == 0) return TWM_OK;
    if (!out_kn_dev) return api_fail(TWM_INVALID_HANDLE, "twm_weight_dequant_f16: null output");
    // "dequant_src" = 1 reads the column-lane copy instead of the 16-column tile order (each builds its copy if need be)
    if (int rc = weight_ensure(ctx, w, ctx->dequant_src == 1 ? kCopyCol : kCopyTile, "twm_weight_dequant_f16")) return rc;
    if (ctx->dequant_src == 1)
        HIP_TRY(launch_weight_dequant_f16_col(ctx->stream, view_of(w), out_kn_dev), TWM_DEVICE_ERROR, "dequant launch");
    else
        HIP_TRY(launch_weight_dequant_f16(ctx->stream, view_of(w), out_kn_dev), TWM_DEVICE_ERROR, "dequant launch");
    return TWM_OK;
}

/* ---- dispatcher --------------------------------------------------------------------------- */

// M <= 4 kernel (one lane per column): a workgroup of `waves` waves shares nt tiles of 64 columns
// and splits its k-chunks among the waves; workgroups split K further when 64-column tiles alone
// leave CUs idle.  Aim for about 16 waves per CU with at least two chunks per wave.
static DecodePlan plan_gemv4(uint32_t n_tiles, uint32_t k_chunks, int force_nt, int force_waves, uint32_t force_splits)
{
    DecodePlan p;
    p.lane_col = 1;
    uint32_t tiles64 = n_tiles * kTileN / 64;
    p.nt = 1;
    if (force_nt == 2 && tiles64 % 2 == 0) p.nt = 2;
    uint32_t tg = tiles64 / p.nt;
    // eight waves unless half of them would find no chunk: with a shallow K one chunk per wave puts every load
    // in flight at once (896-deep: 3.6 us with eight waves, 4.2 us with two)
    p.waves = 8;
    while (p.waves > 1 && k_chunks <= p.waves / 2) p.waves /= 2;
    // 64 .. 127 tiles with a deep K (4096 -> 4096 is the case): sixteen waves per tile put as many waves in flight
    // as a two-way split-K of eight-wave workgroups would, without its partial sums (5.9 against 6.5 us)
    if (p.waves == 8 && tg >= 64 && tg < 128 && k_chunks >= 32) p.waves = 16;
    if (force_waves) p.waves = (uint32_t)force_waves;
    uint32_t sp = 1;  // splitting across workgroups costs a synchronisation: only for matrices with few tiles
    while (tg * p.waves * sp < 1024 && k_chunks / (sp * 2) >= p.waves * 2) sp *= 2;
    if (force_splits) sp = force_splits;
    if (sp > k_chunks) sp = k_chunks ? k_chunks : 1;
    p.splits = sp;
    return p;
}

// Sub-tile variant of the M <= 4 kernel: 16 or 32 columns per workgroup, each wave one pass (4 or 2 chunks) of
// them, so that narrow matrices fill the CUs without a cross-workgroup split-K and wide ones run as many
// short-lived workgroups.  sub = 0: keep the 64-column plan.  Fitted to sweeps over the Qwen2.5-7B, Llama-7B and
// Qwen2.5-0.5B projections (M = 1, 2, 4; f16 and f32 activations); what it loses on are the activations, which
// every lane reads 64 / sub times per chunk: four distinct rows, or f32 rows cut into two terms, shift the
// balance back to wider workgroups.
struct SubPlan {
    uint32_t sub, waves;
};
static SubPlan plan_gemv4_sub(uint32_t tiles64, uint32_t k_chunks, uint32_t m, bool a_f32)
{
    const SubPlan none = {0, 0};
    if (k_chunks < 16) return none;  // shallow K: nothing to gain over one chunk per wave of the 64-column plan
    const bool two_pass = a_f32 && m > 2;
    const uint32_t passes16 = (k_chunks + 3) / 4;
    // waves per workgroup on 16 columns: one pass each while eight or sixteen cover K; deeper, the pipelined pass loop
    // on eight waves for one row and on four from two rows on (18944 -> 3584: M = 1 8.96 / 9.01 / 9.05 us on 8 / 4 / 16
    // waves, M = 2 9.5 / 9.2 / 9.7, M = 4 11.2 / 10.75 / 11.75)
    // (one row of f32 activations, which a lane takes as one shared piece: 9.3 / 9.6 us on 4 / 8 waves)
    const SubPlan narrow16 = {16, passes16 <= 8 ? 8u : passes16 <= 16 ? 16u : ((m >= 2 && !a_f32) || (m == 1 && a_f32)) ? 4u : 8u};
    if (tiles64 > 128) {
        // wide matrices: only the cheapest activations (f16, up to two rows) leave the sub-tiles ahead
        // (3584 -> 37888: 15.8 against 17.0 us at M = 1, 18.3 against 17.3 at M = 4, 19.9 against 17.9 with f32 rows)
        // and only while every wave gets exactly one pass (K <= 4096): beyond that the 64-column kernel is ahead
        // again (5120 -> 15360: 9.2 against 12.5 us; 8192 -> 57344: 42.3 against 49.7)
        // and where whole tiles would leave their last round of 256 workgroups under 80 % full, which is the loss the
        // finer workgroups remove (4096 -> 22016, 344 tiles = 1.34 rounds: 10.6 against 12.1 us; 3584 -> 37888, 2.31
        // rounds: 14.8 against 15.5; but 4096 -> 28672, 1.75 rounds: 13.2 against 12.7, and 3584 -> 152064, 9.3
        // rounds: 49.3 against 47.8)
        const uint32_t rounds = (tiles64 + 255) / 256;
        const bool poor_fill = tiles64 * 5 < rounds * 256 * 4;
        // (several workgroups per CU: no idle eighth wave, 3584 -> 37888 at M = 1 14.8 against 15.3 us; with one workgroup
        // per CU the eight-wave form is the faster one, 3584 -> 3584 3.9 against 4.05)
        if (!a_f32 && m <= 2 && passes16 <= 8 && poor_fill) return SubPlan{16, passes16};
        // one row of f32 activations: the shared-piece form in the pipelined loop on four waves (3584 -> 37888: 15.75 us
        // against 17.0 with one pass per wave and 16.8 on whole tiles)
        if (a_f32 && m == 1 && passes16 <= 8 && poor_fill) return SubPlan{16, 4};
        if (a_f32 && m <= 2 && tiles64 < 256 && k_chunks <= 32) return SubPlan{32, 16};
        return none;
    }
    if (two_pass && passes16 > 16) return k_chunks <= 100 ? SubPlan{32, 8} : none;  // (the looping 16-column variant spills)
    // very deep K, three or four rows: with f32 rows the 64-column split-K plan is level or ahead; with f16 rows the
    // pipelined pass loop is (18944 -> 3584 at M = 3 / 4: 9.96 / 10.75 against 11.75 / 11.84 us)
    if (m > 2 && passes16 > 32 && a_f32) return none;
    if (tiles64 > 64) return SubPlan{32, 16};  // 16 columns would leave a second, quarter-full round of workgroups
    return narrow16;
}

// M = 5 .. 16 (f16 rows): the same kernel repeats its MFMA chain per group of four rows on the unpacked weights.
// It pays where the streaming kernel's 64-column workgroups leave most CUs idle, i.e. on narrow matrices, and
// only in the one-pass form (the looping form runs out of registers): 3584 -> 3584 at M = 8 / 16: 4.8 / 6.5 us
// against 6.9 / 8.2; 3584 -> 4608: 5.5 / 7.4 against 6.9 / 8.2; 3584 -> 37888: 21.7 / 35 against 19.5 / 23.2.
static SubPlan plan_gemv4_sub_rows(uint32_t tiles64, uint32_t k_chunks)
{
    const SubPlan none = {0, 0};
    if (k_chunks < 16 || tiles64 > 128) return none;
    const uint32_t passes16 = (k_chunks + 3) / 4, passes32 = (k_chunks + 1) / 2;
    if (tiles64 <= 64 && passes16 <= 16) return SubPlan{16, passes16 <= 8 ? 8u : 16u};
    if (passes32 <= 16) return SubPlan{32, 16};
    return none;
}

// Batched-decode streaming kernel (M = 5 .. 32): one workgroup of eight waves per 64 columns and k-range.  K is
// cut when the column quads alone leave CUs idle, up to about one workgroup per CU, keeping two chunks per
// wave (one for the 32-row variant, whose chunks cost twice the arithmetic); the partial sums cost a second
// kernel.  Fitted to the per-shape sweep (bench.py --sweep-splits).
static uint32_t plan_stream(uint32_t n_tiles, uint32_t k_chunks, uint32_t m)
{
    uint32_t quads = n_tiles / 4;
    if (quads == 0 || quads >= 256) return 1;
    uint32_t sp = 256 / quads;
    uint32_t cap = k_chunks / (m > 16 ? 7 : 16);  // (3584 -> 3584 at M = 32: four splits of seven chunks 9.2 us, three 10.6)
    if (sp > cap) sp = cap;
    return sp < 2 ? 1 : sp;
}

// Waves per workgroup of the streaming kernel: eight, except that the 32-row variant (158 registers) fits
// only one eight-wave workgroup per CU, so with many column quads four-wave workgroups fill the CUs better.
static uint32_t stream_waves(uint32_t n_tiles, uint32_t m, int force_waves)
{
    if (force_waves == 4 || force_waves == 8) return (uint32_t)force_waves;
    return (m > 16 && n_tiles / 4 >= 256) ? 4 : 8;
}

// Batched-decode kernel with LDS-shared activations: split-K factor over workgroups, k-slices inside a workgroup and
// the columns that share one activation tile (one, two or three 64-column quads per workgroup with one tile per
// wave, or two quads with two tiles per wave) by a small cost model fitted to forced sweeps on fifteen projection
// shapes of 1.5B .. 70B models (microseconds).  A CU works through quad steps (one 128-deep chunk of one 64-column
// quad) at up to 3.5 per us with two row blocks (4.9 with one) when it holds enough waves.  The activation tile
// comes from L2 once per workgroup and chunk, and those requests compete with the weight stream for the CU's memory
// requests in flight: with two or three quads per workgroup the rate is 4.3 (5.2), with two tiles per wave 3.95
// (5.1).  A single slice alone advances at 1.9 (2.5) steps per us, 1.8 (2.4) with eight or twelve waves, 1.7 (2.2)
// with two tiles per wave: the latency of its barrier-and-load chain.  The busiest CU holds ceil(workgroups / 256)
// workgroups of `slices` slices, each with chunks / (splits * slices) steps (the time is the larger of the two
// bounds plus 15 % of the smaller: 8192 -> 10240 at M = 16 on 160 workgroups of two slices, both bounds 13, read 17.5 us
// with the launch, with four slices 15.4); a K-split over workgroups costs the
// second kernel (2.5) and, per split, 0.2 plus the partial sums written and read back at 2.7 TB/s
// (18944 -> 3584 at M = 32 read 19.0 us on nine splits against 17.2 on four).  A more elaborate plan has to win by
// 3 %; a slice keeps two chunks or more (eight with two tiles per wave).
// (3584 -> 37888, 592 quads x 28 chunks, M = 32: one quad per workgroup 26.1 us, two 26.0 -- 296 workgroups put four
// quads on some CUs instead of three --, three 22.4, two k-slices 27.3, two K-splits 30.3; 4096 -> 22016, 344 x 32:
// one quad 20.5, two quads x two slices 16.8; 8192 -> 57344, 896 x 64: one quad 72.4, two 63.2, two tiles per wave
// 61.9; 18944 -> 3584, 56 x 148: 4 splits x 2 slices 17.1, 4 x 1 20.7; 8192 -> 10240, 160 x 64: 3 splits, two quads x
// two slices 17.0, one quad 18.5.)
struct BatchPlan {
    uint32_t splits, slices, tiles_per_wave, quads_per_group;
};
static BatchPlan plan_batch(uint32_t n_tiles, uint32_t k_chunks, uint32_t m, bool rows_f32, uint32_t force_splits = 0)
{
    const uint32_t quads = n_tiles / 4;
    const bool two_blocks = m > 16;
    const double partial_us = (double)m * n_tiles * 16.0 * 4.0 * 2.0 / 4.0e6;  // one split's partial sums, written and read
    BatchPlan best = {force_splits ? (force_splits < k_chunks ? force_splits : k_chunks) : 1u, 1u, 1u, 1u};
    double best_us = 1e30;
    static const struct { uint32_t tpw, qpg, max_slices; double full2, full1, lone2, lone1; } kForms[] = {
        {1, 1, 4, 3.5, 4.9, 1.9, 2.5}, {1, 2, 2, 4.3, 5.2, 1.8, 2.4}, {1, 3, 1, 4.3, 5.2, 1.8, 2.4}, {2, 1, 2, 3.95, 5.1, 1.7, 2.2}};
    for (const auto &f : kForms) {
        const double full_rate = two_blocks ? f.full2 : f.full1, lone_rate = two_blocks ? f.lone2 : f.lone1;
        const uint32_t share = f.tpw * f.qpg;  // quads per workgroup
        const uint64_t groups = (quads + share - 1) / share;
        // (the 32-row two-term variant has LDS for one slice of eight waves, two of four)
        const uint32_t max_slices = two_blocks && rows_f32 ? (f.qpg == 2 ? 1u : f.max_slices < 2 ? f.max_slices : 2u) : f.max_slices;
        for (uint32_t sp = 1; sp <= 16 && sp <= k_chunks; sp++) {
            if (force_splits && sp != best.splits) continue;
            const uint32_t cps = (k_chunks + sp - 1) / sp;
            if (!force_splits && (k_chunks + cps - 1) / cps != sp) continue;  // same work as a smaller factor
            const double wgs_on_cu = (double)((groups * sp + 255) / 256);
            for (uint32_t ks = 1; ks <= max_slices; ks *= 2) {
                if (ks > 1 && cps < (f.tpw == 1 ? 2 : 8) * ks) continue;
                const double steps = (double)((cps + ks - 1) / ks);
                const double busy = wgs_on_cu * share * ks * steps / full_rate, chain = steps / lone_rate;
                double t = busy > chain ? busy + 0.15 * chain : chain + 0.15 * busy;  // (neither hides the other entirely)
                if (ks > 1) t += 0.3 * ks;  // the slices' sums through LDS, the wider barriers
                if (sp > 1) t += 2.5 + sp * (0.2 + 1.5 * partial_us);
                if (t < best_us * 0.97) {
                    best_us = t;
                    best.splits = sp;
                    best.slices = ks;
                    best.tiles_per_wave = f.tpw;
                    best.quads_per_group = f.qpg;
                }
            }
        }
    }
    return best;
}

// ---- the launch form of a GEMM: chosen in one place, launched in another ---------------------------------
// What twm_gemm will run for a weight's shape, a row count and the context's knobs.  Nothing here touches the device.
enum FormKind { kFormPrefill = 0, kFormSubTile = 1, kFormWholeTile = 2, kFormBatch = 3, kFormStream = 4, kFormNone = 5 };
struct LaunchForm {
    int kind;
    int copy;                 // the repacked order it reads (kCopyTile / kCopyCol)
    uint32_t sub, waves;      // sub-tile kernel: columns per workgroup, waves; whole tiles / streaming: waves
    uint32_t nt;              // whole tiles: 64-column tiles per workgroup
    uint32_t splits;          // K-splits over workgroups (prefill: the forced factor, 0 = plan_prefill's choice)
    bool batch_auto;          // LDS-shared batched decode: plan_batch per 32-row block, else `batch` as forced
    bool rounded;             //   ... on f16-rounded weights (option "batch_rounded")
    BatchPlan batch;
};
struct FormEnv {              // the knobs and limits of a context
    int kernel, nt, waves, sub, sub_waves, prefill_min_m, batch_rounded;
    size_t ws_bytes;          // split-K scratch
    uint32_t n_counters;      // arrival counters
};
static FormEnv form_env(const twm_ctx *c)
{
    return FormEnv{c->force_kernel, c->force_nt, c->force_waves, c->force_sub, c->force_sub_waves, c->prefill_min_m,
                   c->batch_rounded, c->ws_bytes, c->n_counters};
}

// n_tiles: 16-column tiles of the padded weight; gated: the gated store of a paired weight
static LaunchForm choose_form(const FormEnv &e, uint32_t n_tiles, uint32_t k_chunks, uint32_t m, bool a_f32, uint32_t splits, bool gated)
{
    LaunchForm f = {};
    const uint32_t n_ld = n_tiles * kTileN, tiles64 = n_ld / 64;
    f.splits = splits;
    if (m >= (uint32_t)e.prefill_min_m) {
        f.kind = kFormPrefill;
        f.copy = kCopyTile;
        return f;
    }
    // the sub-tile kernel's K-split fits the scratch and the counters
    auto fit_sub_splits = [&](uint32_t sub) {
        uint32_t ssp = splits ? splits : 1;
        if (ssp > k_chunks) ssp = k_chunks;
        while (ssp > 1 && (size_t)ssp * m * n_ld * 4 > e.ws_bytes) ssp--;
        if (n_ld / sub > e.n_counters) ssp = 1;
        return ssp;
    };
    auto fit_whole_splits = [&](DecodePlan &plan) {
        while (plan.splits > 1 && (size_t)plan.splits * m * n_ld * 4 > e.ws_bytes) plan.splits--;
        if (n_tiles / plan.nt > e.n_counters) plan.splits = 1;
    };
    if (e.kernel == 0 && m > 4 && m <= 16 && !a_f32 && e.sub != 1) {
        // M = 5 .. 16 on narrow matrices: the lane-per-column sub-tile kernel with two to four row groups
        SubPlan sub = {0, 0};
        if (e.sub >= 16) sub = SubPlan{(uint32_t)e.sub, e.sub_waves ? (uint32_t)e.sub_waves : e.waves ? (uint32_t)e.waves : 8};
        else if (!e.nt && !e.waves && !splits) sub = plan_gemv4_sub_rows(tiles64, k_chunks);
        if (sub.sub) {
            f.kind = kFormSubTile;
            f.copy = kCopyCol;
            f.sub = sub.sub;
            f.waves = sub.waves;
            f.splits = fit_sub_splits(sub.sub);
            return f;
        }
        if (m <= 8 && tiles64 > 128 && !e.nt && !splits) {
            // M = 5 .. 8 on wide matrices: the 64-column lane-per-column kernel with two row groups, which unpacks with
            // fewer vector instructions than the streaming kernel (3584 -> 37888 at M = 8: 18.0 against 19.2 us,
            // 3584 -> 152064: 54.8 against 60.0; with four row groups, M = 9 .. 16, it needs 127 registers and loses;
            // on 128 tiles or fewer the streaming kernel's split-K is ahead: 14336 -> 4096 11.4 against 19.8 us)
            DecodePlan plan = plan_gemv4(n_tiles, k_chunks, 1, e.waves, 0);
            fit_whole_splits(plan);
            f.kind = kFormWholeTile;
            f.copy = kCopyCol;
            f.nt = 1;
            f.waves = plan.waves;
            f.splits = plan.splits;
            return f;
        }
    }
    const bool batch_auto = e.kernel == 0 && !e.nt && !e.waves &&
                            (m > 16 || (!splits && ((m > 8 && (tiles64 > 128 || a_f32)) || (a_f32 && m > 4 && k_chunks <= 64))));
    if (e.kernel == 4 || batch_auto) {
        // batched decode with the activations shared through LDS, in 32-row blocks: from 17 rows on (the same exact
        // arithmetic as below 17 rows; option "batch_rounded" runs the f16-rounded weights of the prefill kernel
        // there), and from 9 rows on wide
        // matrices (3584 -> 37888: M = 16 19.8 against 22.8 us of the streaming kernel, M = 32 26.7 against
        // 33.3; 18944 -> 3584 at M = 32 17.3 against 21.8; at M = 9 .. 16 on narrow matrices the two are within 3 %
        // with f16 rows).  f32 rows, which the streaming kernel holds twice in registers: from 9 rows on everywhere
        // (3584 -> 4608 at M = 16 10.9 against 15.1 us, 18944 -> 3584 20.6 against 23.3), from 5 rows on up to 64
        // chunks deep (3584 -> 4608 at M = 8 10.5 against 11.4; 13824 -> 5120 would lose 18.6 against 18.5)
        f.kind = kFormBatch;
        f.copy = kCopyTile;
        f.batch_auto = batch_auto;
        f.rounded = e.batch_rounded && m > 16;
        // forced: "nt" 2 = two tiles per wave, 4 = two quads per workgroup, 3 = three; "waves" 8 / 16 = 2 / 4 k-slices
        f.batch = BatchPlan{splits ? splits : 1, e.waves == 8 ? 2u : e.waves == 16 ? 4u : 1u, e.nt == 2 ? 2u : 1u,
                            e.nt == 4 ? 2u : e.nt == 3 ? 3u : 1u};
        return f;
    }
    if (e.kernel == 3 || (e.kernel == 0 && m > 4)) {
        f.kind = kFormStream;   // batched decode: 32-row blocks of the streaming kernel
        f.copy = kCopyTile;
        return f;
    }
    // M <= 4: one lane per column (whole 64-column tiles, or the sub-tile kernel where the planner takes it)
    if (m > 4) {
        f.kind = kFormNone;
        return f;
    }
    f.copy = kCopyCol;
    SubPlan sub = {0, 0};
    if (e.sub >= 16) {
        sub.sub = (uint32_t)e.sub;
        sub.waves = e.sub_waves ? (uint32_t)e.sub_waves : e.waves ? (uint32_t)e.waves : 8;
    } else if (e.sub == 0 && !e.nt && !e.waves && !splits) {
        // (an explicit nt, waves or split factor asks for the 64-column kernel's plan)
        sub = plan_gemv4_sub(tiles64, k_chunks, m, a_f32);
        // the gated store splits a sub-tile into a gate and an up half: 16 columns would read 128-byte runs
        // (3584 -> 2 x 18944 at M = 1: 17.0 us on 16 columns, 16.3 on 32, 17.1 on whole tiles)
        if (gated && sub.sub == 16) sub = SubPlan{32, 8};
    }
    if (sub.sub) {
        f.kind = kFormSubTile;
        f.sub = sub.sub;
        f.waves = sub.waves;
        f.splits = fit_sub_splits(sub.sub);
        return f;
    }
    DecodePlan plan = plan_gemv4(n_tiles, k_chunks, e.nt, e.waves, splits);
    fit_whole_splits(plan);  // the scratch must hold splits x m x n_ld partials and one counter per tile group
    f.kind = kFormWholeTile;
    f.nt = plan.nt;
    f.waves = plan.waves;
    f.splits = plan.splits;
    return f;
}

static void tiles_of(uint32_t k, uint32_t n, uint32_t &n_tiles, uint32_t &k_chunks)
{
    n_tiles = ((n + kNPadTo - 1) / kNPadTo) * kNPadTo / kTileN;
    k_chunks = (k / 32 + kChunkGroups - 1) / kChunkGroups;
}
static FormEnv default_env()
{
    return FormEnv{0, 0, 0, 0, 0, 33, 0, kWsBytes, kCounters};
}

uint32_t twm_pick_splits(uint32_t k, uint32_t n, uint32_t m)
{
    uint32_t n_tiles, k_chunks;
    tiles_of(k, n, n_tiles, k_chunks);
    if (m == 0 || n_tiles == 0 || k_chunks == 0) return 1;
    // (f16 activations, nothing forced, the default scratch)
    const LaunchForm f = choose_form(default_env(), n_tiles, k_chunks, m, false, 0, false);
    switch (f.kind) {
    case kFormSubTile:
    case kFormWholeTile: return f.splits;
    case kFormBatch: return plan_batch(n_tiles, k_chunks, m < 32 ? m : 32, false).splits;
    case kFormStream: return plan_stream(n_tiles, k_chunks, m < 32 ? m : 32);
    default: return 1;  // prefill: see twm_plan_describe
    }
}

int twm_plan_describe(const twm_ctx *ctx, uint32_t k, uint32_t n, uint32_t m, int a_dtype, int gated, char *text, size_t bytes)
{
    if (!text || bytes == 0) return api_fail(TWM_INVALID_HANDLE, "twm_plan_describe: null buffer");
    if (a_dtype != TWM_F16 && a_dtype != TWM_F32) return api_fail(TWM_UNSUPPORTED_OP, "twm_plan_describe: activations must be f16 or f32");
    if (int rc = check_kn("twm_plan_describe", k, n)) return rc;
    uint32_t n_tiles, k_chunks;
    tiles_of(k, n, n_tiles, k_chunks);
    if (m == 0 || n == 0 || k == 0) {
        snprintf(text, bytes, "nothing to launch");
        return TWM_OK;
    }
    const bool a_f32 = a_dtype == TWM_F32;
    const FormEnv e = ctx ? form_env(ctx) : default_env();
    const LaunchForm f = choose_form(e, n_tiles, k_chunks, m, a_f32, 0, gated != 0);
    const uint32_t mb = m < (uint32_t)kMaxStreamM ? m : (uint32_t)kMaxStreamM;
    switch (f.kind) {
    case kFormPrefill: {
        uint32_t bm = 0, sp = 0;
        prefill_plan_of(m, 0, 0, n_tiles, k_chunks, e.ws_bytes, gated != 0, &bm, &sp);
        snprintf(text, bytes, "k_prefill: %u-row x %u-column blocks, %u K-split%s%s; 16-column tile copy", bm == 64 ? 64u : 128u,
                 bm == 192 ? 192u : 256u, sp, sp == 1 ? "" : "s", sp > 1 ? " + k_splitk_reduce" : "");
        break;
    }
    case kFormSubTile:
        snprintf(text, bytes, "k_gemv4s: %u-column sub-tiles, %u waves, %u K-split%s; column-lane copy", f.sub, f.waves, f.splits,
                 f.splits == 1 ? "" : "s");
        break;
    case kFormWholeTile:
        snprintf(text, bytes, "k_gemv4: %u x 64-column tiles per workgroup, %u waves, %u K-split%s; column-lane copy", f.nt, f.waves,
                 f.splits, f.splits == 1 ? "" : "s");
        break;
    case kFormBatch: {
        const BatchPlan bp = f.batch_auto ? plan_batch(n_tiles, k_chunks, f.rounded ? 32 : mb, a_f32, 0) : f.batch;
        snprintf(text, bytes, "k_batch: %u quad%s per workgroup, %u tile%s per wave, %u k-slice%s, %u K-split%s%s; 16-column tile copy",
                 bp.quads_per_group, bp.quads_per_group == 1 ? "" : "s", bp.tiles_per_wave, bp.tiles_per_wave == 1 ? "" : "s", bp.slices,
                 bp.slices == 1 ? "" : "s", bp.splits, bp.splits == 1 ? "" : "s", bp.splits > 1 ? " + k_splitk_reduce" : "");
        break;
    }
    case kFormStream: {
        const uint32_t sp = plan_stream(n_tiles, k_chunks, mb);
        snprintf(text, bytes, "k_stream: %u waves, %u K-split%s%s; 16-column tile copy", stream_waves(n_tiles, mb, e.waves), sp,
                 sp == 1 ? "" : "s", sp > 1 ? " + k_splitk_reduce" : "");
        break;
    }
    default: snprintf(text, bytes, "no kernel takes this case with the knobs set"); break;
    }
    return TWM_OK;
}

// swiglu_out (paired weight): the launch writes silu(gate) * up to swiglu_out[m][n/2] instead of the columns
// to `out`.
static int gemm_dispatch(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, const OutSpec &out,
                         uint32_t splits, const char *who, float *swiglu_out = nullptr, uint32_t gate_act = 2)
{
    if (a_dtype != TWM_F16 && a_dtype != TWM_F32) return api_fail(TWM_UNSUPPORTED_OP, "%s: activations must be f16 or f32", who);
    if (m == 0 || w->n == 0) return TWM_OK;
    if (w->k == 0) {
        for (uint32_t s = 0; s < out.count; s++) {
            if (!out.seg[s].bias) {
                if (int rc = twm_memset_zero(ctx, out.seg[s].ptr, (size_t)m * out.seg[s].width * 4)) return rc;
                continue;
            }
            for (uint32_t r = 0; r < m; r++)  // an empty sum plus the bias
                if (int rc = twm_memcpy_d2d(ctx, out.seg[s].ptr + (size_t)r * out.seg[s].width, out.seg[s].bias,
                                            (size_t)out.seg[s].width * 4))
                    return rc;
        }
        return TWM_OK;
    }
    if (!a_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null activations", who);
    if (((uintptr_t)a_dev & 15) != 0) return api_fail(TWM_SHAPE_ERROR, "%s: activations must be 16-byte aligned", who);
    const bool a_f32 = a_dtype == TWM_F32;
    const size_t a_row_bytes = (size_t)w->k * (a_f32 ? 4 : 2);
    OutSpec gated = out;
    gated.swiglu = swiglu_out;
    gated.gate_act = gate_act;
    const LaunchForm f = choose_form(form_env(ctx), w->n_tiles, w->k_chunks, m, a_f32, splits, swiglu_out != nullptr);
    if (f.kind == kFormNone) return api_fail(TWM_UNSUPPORTED_OP, "%s: the one-lane-per-column kernel takes M <= 4", who);
    // the copy the launch reads is built here if the handle does not hold it yet
    if (int rc = weight_ensure(ctx, w, f.copy, who)) return rc;
    const WeightView v = view_of(w);
    // rows beyond 32: blocks of 32 rows, each a launch of its own
    auto row_blocks = [&](auto &&launch_block) -> int {
        for (uint32_t m0 = 0; m0 < m; m0 += kMaxStreamM) {
            const uint32_t mb = m - m0 < (uint32_t)kMaxStreamM ? m - m0 : (uint32_t)kMaxStreamM;
            OutSpec o = gated;
            for (uint32_t s = 0; s < o.count; s++) o.seg[s].ptr += (size_t)m0 * o.seg[s].width;
            if (o.swiglu) o.swiglu += (size_t)m0 * (w->n / 2);
            if (int rc = launch_block((const char *)a_dev + (size_t)m0 * a_row_bytes, mb, o)) return rc;
        }
        return TWM_OK;
    };
    switch (f.kind) {
    case kFormPrefill: {
        const PrefillSk sk = {ctx->sk_ws, ctx->sk_ws_bytes, ctx->counters, ctx->n_counters, (uint32_t)ctx->prop.multiProcessorCount,
                              ctx->prefill_sk};
        HIP_TRY(launch_prefill(ctx->stream, v, a_dev, a_f32, m, gated, (uint32_t)ctx->prefill_bm, splits, ctx->ws, ctx->ws_bytes, &sk),
                TWM_DEVICE_ERROR, "prefill launch");
        return TWM_OK;
    }
    case kFormSubTile:
        HIP_TRY(launch_gemv4s(ctx->stream, v, a_dev, a_f32, m, gated, ctx->ws, ctx->counters, f.sub, f.waves, f.splits), TWM_DEVICE_ERROR,
                "sub-tile gemv launch");
        return TWM_OK;
    case kFormWholeTile:
        HIP_TRY(launch_gemv4(ctx->stream, v, a_dev, a_f32, m, gated, ctx->ws, ctx->counters, f.nt, f.waves, f.splits, swiglu_out),
                TWM_DEVICE_ERROR, "gemv launch");
        return TWM_OK;
    case kFormBatch:
        return row_blocks([&](const char *a_blk, uint32_t mb, const OutSpec &o) -> int {
            const BatchPlan bp = f.batch_auto ? plan_batch(w->n_tiles, w->k_chunks, f.rounded ? 32 : mb, a_f32, splits) : f.batch;
            HIP_TRY(launch_batch(ctx->stream, v, a_blk, a_f32, mb, o, bp.splits, bp.tiles_per_wave, bp.slices, bp.quads_per_group, f.rounded,
                                 ctx->ws, ctx->ws_bytes),
                    TWM_DEVICE_ERROR, "batched decode launch");
            return TWM_OK;
        });
    default:  // kFormStream
        return row_blocks([&](const char *a_blk, uint32_t mb, const OutSpec &o) -> int {
            HIP_TRY(launch_stream(ctx->stream, v, a_blk, a_f32, mb, o, splits ? splits : plan_stream(w->n_tiles, w->k_chunks, mb),
                                  stream_waves(w->n_tiles, mb, ctx->force_waves), ctx->ws, ctx->ws_bytes),
                    TWM_DEVICE_ERROR, "batched decode launch");
            return TWM_OK;
        });
    }
}

// The knobs of a launch form, saved and set as one
struct Knobs {
    int kernel, nt, waves, sub, sub_waves, prefill_bm;
};
static Knobs knobs_of(const twm_ctx *c) { return Knobs{c->force_kernel, c->force_nt, c->force_waves, c->force_sub, c->force_sub_waves, c->prefill_bm}; }
static void set_knobs(twm_ctx *c, const Knobs &k)
{
    c->force_kernel = k.kernel;
    c->force_nt = k.nt;
    c->force_waves = k.waves;
    c->force_sub = k.sub;
    c->force_sub_waves = k.sub_waves;
    c->prefill_bm = k.prefill_bm;
}

// With nothing forced by the caller, a plan that twm_weight_tune measured for this weight and row count is what runs.
static int gemm_common(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, const OutSpec &out,
                       uint32_t splits, const char *who, float *swiglu_out = nullptr, uint32_t gate_act = 2)
{
    const Knobs user = knobs_of(ctx);
    const bool free_choice = !splits && !user.kernel && !user.nt && !user.waves && !user.sub && !user.sub_waves && !user.prefill_bm;
    const TunedPlan *tp = (m >= 1 && free_choice && !swiglu_out && a_dtype == TWM_F16) ? &w->tuned[tune_bucket(m)] : nullptr;
    if (!tp || !tp->valid) return gemm_dispatch(ctx, w, a_dev, a_dtype, m, out, splits, who, swiglu_out, gate_act);
    set_knobs(ctx, Knobs{tp->kernel, tp->nt, tp->waves, tp->sub, tp->sub_waves, tp->prefill_bm});
    const int rc = gemm_dispatch(ctx, w, a_dev, a_dtype, m, out, tp->splits, who, swiglu_out, gate_act);
    set_knobs(ctx, user);
    return rc;
}

// Candidate launch forms for `m` rows: what the option knobs can ask for.  The first entry is the planners' own choice.
static void tune_candidates(uint32_t m, uint32_t k_chunks, std::vector<TunedPlan> &out)
{
    auto add = [&](int kernel, int nt, int waves, int sub, int sub_waves, int splits, int bm) {
        out.push_back(TunedPlan{1, (uint8_t)kernel, (uint8_t)nt, (uint8_t)waves, (uint8_t)sub, (uint8_t)sub_waves, (uint8_t)splits, (uint8_t)bm});
    };
    add(0, 0, 0, 0, 0, 0, 0);
    const uint32_t passes16 = (k_chunks + 3) / 4, passes32 = (k_chunks + 1) / 2;
    if (m <= 16) {
        // sub-tile kernel: one pass per wave where sixteen waves cover K, else the pass loop on 4, 8 or 16 waves
        for (int sub : {16, 32}) {
            const uint32_t passes = sub == 16 ? passes16 : passes32;
            if (passes <= 16) add(0, 0, 0, sub, (int)passes, 0, 0);
            for (int wv : {4, 8, 16})
                if ((uint32_t)wv < passes || (passes <= 16 && (uint32_t)wv != passes)) add(0, 0, 0, sub, wv, 0, 0);
        }
    }
    if (m <= 4) {
        for (int wv : {8, 16})
            for (int sp : {1, 2, 4, 8}) add(2, 1, wv, 0, 0, sp, 0);   // whole 64-column tiles, K split over workgroups
        add(2, 2, 8, 0, 0, 1, 0);
    } else if (m <= 32) {
        for (int sp : {1, 2, 3, 4, 6, 8}) add(3, 0, 0, 0, 0, sp, 0);  // streaming kernel
        for (int nt : {1, 2, 3, 4})                                     // LDS-shared kernel: tiles per wave / quads per workgroup
            for (int wv : {0, 8, 16})                                   // k-slices
                for (int sp : {1, 2, 3, 4, 6})
                    if (!(wv == 16 && nt != 1) && !(wv == 8 && nt == 3)) add(4, nt, wv, 0, 0, sp, 0);
    } else {
        for (int bm : {64, 128, 192})
            for (int sp : {1, 2, 3, 4, 6, 8}) add(0, 0, 0, 0, 0, sp, bm);
    }
}

int twm_weight_tune(twm_ctx *ctx, twm_weight *w, const uint32_t *ms, uint32_t count)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_tune: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_weight_tune: weight belongs to another context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_weight_tune: not allowed inside a graph capture");
    if (count != 0 && !ms) return api_fail(TWM_INVALID_HANDLE, "twm_weight_tune: null row counts");
    if (w->copy_bytes == 0 || w->k == 0 || w->n == 0) return TWM_OK;
    uint32_t m_max = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (ms[i] == 0 || ms[i] > 65536u) return api_fail(TWM_SHAPE_ERROR, "twm_weight_tune: row counts are 1 .. 65536");
        if (ms[i] > m_max) m_max = ms[i];
    }
    if (m_max == 0) return TWM_OK;
    // synthetic f16 activations (a fixed pattern of small values) and an output, both released at the end
    void *a_dev = nullptr, *c_dev = nullptr;
    const size_t a_bytes = (size_t)m_max * w->k * 2, c_bytes = (size_t)m_max * w->n * 4;
    if (hipMalloc(&a_dev, a_bytes) != hipSuccess || hipMalloc(&c_dev, c_bytes) != hipSuccess) {
        if (a_dev) (void)hipFree(a_dev);
        return api_fail(TWM_MEMORY_ERROR, "twm_weight_tune: hipMalloc of the trial buffers");
    }
    int rc = TWM_OK;
    {
        std::vector<uint16_t> host(a_bytes / 2);
        uint32_t x = 2463534242u;
        for (auto &h : host) {
            x ^= x << 13; x ^= x >> 17; x ^= x << 5;
            h = (uint16_t)(0x3000u + (x & 0x0FFFu)) | (uint16_t)((x >> 16) & 0x8000u);  // +-[0.125, 0.5)
        }
        rc = twm_memcpy_h2d(ctx, a_dev, host.data(), a_bytes);
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (rc == TWM_OK && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess))
        rc = api_fail(TWM_DEVICE_ERROR, "twm_weight_tune: hipEventCreate");
    // The trials rotate over copies of the weight that together exceed the 256 MB cache in front of HBM, as the layers
    // of a model do: timed on one resident copy, the forms that are best from the caches would win.
    if (rc == TWM_OK) rc = weight_ensure(ctx, w, kCopyTile | kCopyCol, "twm_weight_tune");
    std::vector<twm_weight> clones;
    if (rc == TWM_OK) {
        size_t want = ((size_t)320 << 20) / (2 * w->copy_bytes) + 1;
        if (want > 32) want = 32;
        for (size_t c = 0; c + 1 < want && rc == TWM_OK; c++) {
            twm_weight cl = *w;
            cl.qw = cl.sc = cl.cq = nullptr;
            if (hipMalloc(&cl.qw, w->copy_bytes) != hipSuccess || hipMalloc(&cl.cq, w->copy_bytes) != hipSuccess) {
                if (cl.qw) (void)hipFree(cl.qw);
                (void)hipGetLastError();
                break;   // (fewer copies: the trials are warmer than a model's layers would be, but still fair among themselves)
            }
            cl.sc = (char *)cl.qw + (size_t)w->n_tiles * w->k_chunks * 1024;
            if (hipMemcpyAsync(cl.qw, w->qw, w->copy_bytes, hipMemcpyDeviceToDevice, ctx->stream) != hipSuccess ||
                hipMemcpyAsync(cl.cq, w->cq, w->copy_bytes, hipMemcpyDeviceToDevice, ctx->stream) != hipSuccess)
                rc = api_fail(TWM_DEVICE_ERROR, "twm_weight_tune: copying the weight");
            clones.push_back(cl);
        }
    }
    uint32_t turn = 0;
    auto next_weight = [&]() -> const twm_weight * {
        const size_t n = clones.size() + 1;
        const size_t at = turn++ % n;
        return at == 0 ? w : &clones[at - 1];
    };
    const Knobs user = knobs_of(ctx);
    OutSpec out;
    memset(&out, 0, sizeof out);
    out.count = 1;
    out.seg[0].ptr = (float *)c_dev;
    out.seg[0].width = w->n;
    for (uint32_t i = 0; i < count && rc == TWM_OK; i++) {
        const uint32_t m = ms[i];
        std::vector<TunedPlan> cands;
        tune_candidates(m, w->k_chunks, cands);
        const int reps = m <= 32 ? 24 : 6;
        float best_ms = 0.f, own_ms = 0.f;
        TunedPlan best = cands[0];
        for (size_t c = 0; c < cands.size(); c++) {
            const TunedPlan &p = cands[c];
            set_knobs(ctx, Knobs{p.kernel, p.nt, p.waves, p.sub, p.sub_waves, p.prefill_bm});
            bool ok = true;
            for (int r = 0; r < 2 && ok; r++) ok = gemm_dispatch(ctx, next_weight(), a_dev, TWM_F16, m, out, p.splits, "twm_weight_tune") == TWM_OK;
            float ms_taken = 0.f;
            // timed as the decode loop runs it: a captured graph of `reps` launches over the rotating copies, replayed
            hipGraph_t graph = nullptr;
            hipGraphExec_t exec = nullptr;
            if (ok) {
                ok = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed) == hipSuccess;
                bool launched = ok;
                for (int r = 0; r < reps && launched; r++)
                    launched = gemm_dispatch(ctx, next_weight(), a_dev, TWM_F16, m, out, p.splits, "twm_weight_tune") == TWM_OK;
                if (ok) ok = hipStreamEndCapture(ctx->stream, &graph) == hipSuccess && launched;
                ok = ok && graph && hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess;
            }
            for (int run = 0; run < 3 && ok; run++) {   // one untimed replay, then the faster of two timed ones
                float t = 0.f;
                (void)hipEventRecord(e0, ctx->stream);
                ok = hipGraphLaunch(exec, ctx->stream) == hipSuccess;
                (void)hipEventRecord(e1, ctx->stream);
                ok = ok && hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&t, e0, e1) == hipSuccess;
                if (run == 1 || (run == 2 && t < ms_taken)) ms_taken = t;
            }
            if (exec) (void)hipGraphExecDestroy(exec);
            if (graph) (void)hipGraphDestroy(graph);
            if (!ok) {   // a form this shape does not take: skipped
                (void)hipGetLastError();
                continue;
            }
            if (c == 0) own_ms = ms_taken;
            if (best_ms == 0.f || ms_taken < best_ms) {
                best_ms = ms_taken;
                best = p;
            }
        }
        // the planners' choice stays unless a forced form beats it by more than 2 % (timing noise)
        TunedPlan &slot = w->tuned[tune_bucket(m)];
        if (own_ms > 0.f && best_ms < 0.98f * own_ms && (best.kernel || best.nt || best.waves || best.sub || best.sub_waves || best.splits || best.prefill_bm))
            slot = best;
        else
            memset(&slot, 0, sizeof slot);
    }
    set_knobs(ctx, user);
    (void)hipStreamSynchronize(ctx->stream);
    for (twm_weight &cl : clones) {
        (void)hipFree(cl.qw);
        (void)hipFree(cl.cq);
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(a_dev);
    (void)hipFree(c_dev);
    return rc;
}

int twm_weight_tuned_plan(const twm_weight *w, uint32_t m, int *knobs8)
{
    if (!w || !knobs8 || m == 0) return api_fail(TWM_INVALID_HANDLE, "twm_weight_tuned_plan: null argument");
    const TunedPlan &p = w->tuned[tune_bucket(m)];
    const int v[8] = {p.valid, p.kernel, p.nt, p.waves, p.sub, p.sub_waves, p.splits, p.prefill_bm};
    for (int i = 0; i < 8; i++) knobs8[i] = v[i];
    return TWM_OK;
}

int twm_gemm(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *c_dev, uint32_t splits)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_gemm: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_gemm: weight belongs to another context");
    if (m != 0 && w->n != 0 && !c_dev) return api_fail(TWM_INVALID_HANDLE, "twm_gemm: null output");
    OutSpec out;
    memset(&out, 0, sizeof out);
    out.count = 1;
    out.seg[0].ptr = c_dev;
    out.seg[0].start = 0;
    out.seg[0].width = w->n;
    return gemm_common(ctx, w, a_dev, a_dtype, m, out, splits, "twm_gemm");
}

int twm_gemm_split_bias(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m,
                        float *const *outs_dev, const float *const *biases_dev, const uint32_t *ns, uint32_t count,
                        uint32_t splits)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_split_bias: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_split_bias: weight belongs to another context");
    if (!outs_dev || !ns) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_split_bias: null array");
    if (count == 0 || count > (uint32_t)kMaxSegs)
        return api_fail(TWM_SHAPE_ERROR, "twm_gemm_split_bias: between 1 and %d outputs are supported", kMaxSegs);
    OutSpec out;
    memset(&out, 0, sizeof out);
    uint64_t total = 0;
    uint32_t used = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (ns[i] == 0) continue;
        if (m != 0 && !outs_dev[i]) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_split_bias: null output %u", i);
        out.seg[used].ptr = outs_dev[i];
        out.seg[used].start = (uint32_t)total;
        out.seg[used].width = ns[i];
        out.seg[used].bias = biases_dev ? biases_dev[i] : nullptr;
        used++;
        total += ns[i];
    }
    out.count = used;
    if (total != w->n) return api_fail(TWM_SHAPE_ERROR, "twm_gemm_split_bias: outputs cover %llu columns, weight has %u",
                                   (unsigned long long)total, w->n);
    return gemm_common(ctx, w, a_dev, a_dtype, m, out, splits, "twm_gemm_split_bias");
}

int twm_gemm_split(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *const *outs_dev,
                   const uint32_t *ns, uint32_t count, uint32_t splits)
{
    return twm_gemm_split_bias(ctx, w, a_dev, a_dtype, m, outs_dev, nullptr, ns, count, splits);
}

static int gemm_gated(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *out_dev,
                      uint32_t splits, uint32_t act, const char *who)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "%s: null handle", who);
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "%s: weight belongs to another context", who);
    if (!w->paired) return api_fail(TWM_UNSUPPORTED_OP, "%s: the weight was not built by twm_weight_gate_up", who);
    uint32_t ffn = w->n / 2;
    if (m == 0 || ffn == 0) return TWM_OK;
    if (!out_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null output", who);
    if (((uintptr_t)out_dev & 15) != 0) return api_fail(TWM_SHAPE_ERROR, "%s: the output must be 16-byte aligned", who);
    if (w->k == 0) return twm_memset_zero(ctx, out_dev, (size_t)m * ffn * 4);  // gate(0) * 0
    OutSpec out;
    memset(&out, 0, sizeof out);
    return gemm_common(ctx, w, a_dev, a_dtype, m, out, splits, who, out_dev, act);
}

int twm_gemm_swiglu(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *out_dev,
                    uint32_t splits)
{
    return gemm_gated(ctx, w, a_dev, a_dtype, m, out_dev, splits, 2, "twm_gemm_swiglu");
}

int twm_gemm_geglu(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *out_dev,
                   uint32_t splits)
{
    return gemm_gated(ctx, w, a_dev, a_dtype, m, out_dev, splits, 1, "twm_gemm_geglu");
}

/* ---- expert banks (mixture-of-experts decode) ------------------------------------------------ */

// The bank of both constructors: expert x lies at packed_base + packed_off[x] (bytes) and scales_base + scales_off[x]
// (f16 elements); the offsets have been checked by the caller.
static twm_bank *bank_build(twm_ctx *ctx, const char *who, const uint8_t *packed_base_dev, const uint16_t *scales_base_dev,
                            const std::vector<size_t> &packed_off, const std::vector<size_t> &scales_off, uint32_t k, uint32_t n,
                            uint32_t num_experts, int pair_gate_up)
{
    const size_t groups = k / 32;
    twm_bank *b = new (std::nothrow) twm_bank();
    if (!b) { api_fail(TWM_MEMORY_ERROR, "twm_bank: out of host memory"); return nullptr; }
    b->ctx = ctx;
    b->k = k;
    b->n = n;
    b->experts = num_experts;
    b->paired = pair_gate_up != 0;
    b->n_pad = ((n + 63) / 64) * 64;
    b->k_chunks = (uint32_t)((groups + kChunkGroups - 1) / kChunkGroups);
    b->expert_bytes = (size_t)(b->n_pad / 64) * b->k_chunks * kColBlockBytes;
    b->bytes = b->expert_bytes * num_experts;
    b->cq = nullptr;
    if ((uint64_t)k * n * num_experts == 0 || b->bytes == 0) return b;
    hipError_t e = hipMalloc(&b->cq, b->bytes);
    if (e != hipSuccess) {
        api_fail(TWM_MEMORY_ERROR, "twm_bank: hipMalloc(%zu): %s", b->bytes, hipGetErrorString(e));
        delete b;
        return nullptr;
    }
    for (uint32_t x = 0; x < num_experts && e == hipSuccess; x++)
        e = launch_repack_col(ctx->stream, packed_base_dev + packed_off[x], scales_base_dev + scales_off[x], k, n,
                              (char *)b->cq + (size_t)x * b->expert_bytes, b->n_pad, b->k_chunks, pair_gate_up ? n / 2 : 0);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        api_fail(TWM_DEVICE_ERROR, "%s: repack: %s", who, hipGetErrorString(e));
        (void)hipFree(b->cq);
        delete b;
        return nullptr;
    }
    return b;
}

static bool bank_args_ok(twm_ctx *ctx, const char *who, const uint8_t *packed_base_dev, const uint16_t *scales_base_dev, uint32_t k,
                         uint32_t n, uint32_t num_experts, int pair_gate_up)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "%s: null context", who); return false; }
    if (ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "%s: not allowed inside a graph capture", who); return false; }
    if (check_kn(who, k, n)) return false;
    if (pair_gate_up && n % (2 * kPairWidth) != 0) {
        api_fail(TWM_SHAPE_ERROR, "%s: a paired gate/up bank needs N %% %u == 0, got %u", who, 2 * kPairWidth, n);
        return false;
    }
    const bool empty = (uint64_t)k * n * num_experts == 0;
    if (!empty && (!packed_base_dev || !scales_base_dev)) { api_fail(TWM_INVALID_HANDLE, "%s: null pointer", who); return false; }
    if (((uintptr_t)packed_base_dev & 3) != 0) { api_fail(TWM_SHAPE_ERROR, "%s: packed must be 4-byte aligned", who); return false; }
    return true;
}

twm_bank *twm_bank_from_device(twm_ctx *ctx, const uint8_t *packed_base_dev, const uint16_t *scales_base_dev,
                               size_t packed_bytes_per_expert, size_t scales_per_expert, uint32_t k, uint32_t n,
                               uint32_t num_experts, int pair_gate_up)
{
    if (!bank_args_ok(ctx, "twm_bank_from_device", packed_base_dev, scales_base_dev, k, n, num_experts, pair_gate_up)) return nullptr;
    size_t groups = k / 32;
    if (packed_bytes_per_expert < groups * n * 16 || scales_per_expert < groups * n || packed_bytes_per_expert % 4 != 0) {
        api_fail(TWM_SHAPE_ERROR, "twm_bank_from_device: per-expert strides (%zu bytes, %zu scales) do not hold a %u x %u matrix",
             packed_bytes_per_expert, scales_per_expert, k, n);
        return nullptr;
    }
    std::vector<size_t> po(num_experts), so(num_experts);
    for (uint32_t x = 0; x < num_experts; x++) {
        po[x] = (size_t)x * packed_bytes_per_expert;
        so[x] = (size_t)x * scales_per_expert;
    }
    return bank_build(ctx, "twm_bank_from_device", packed_base_dev, scales_base_dev, po, so, k, n, num_experts, pair_gate_up);
}

twm_bank *twm_bank_from_device_offsets(twm_ctx *ctx, const uint8_t *packed_base_dev, const uint16_t *scales_base_dev,
                                       const uint32_t *packed_offsets_dev, const uint32_t *scales_offsets_dev, uint32_t k,
                                       uint32_t n, uint32_t num_experts, int pair_gate_up)
{
    const char *who = "twm_bank_from_device_offsets";
    if (!bank_args_ok(ctx, who, packed_base_dev, scales_base_dev, k, n, num_experts, pair_gate_up)) return nullptr;
    if (num_experts != 0 && (!packed_offsets_dev || !scales_offsets_dev)) { api_fail(TWM_INVALID_HANDLE, "%s: null offset table", who); return nullptr; }
    // the tables are read once, here: the bank holds its own copy of every expert
    std::vector<uint32_t> po32(num_experts), so32(num_experts);
    if (num_experts != 0) {
        hipError_t e = hipStreamSynchronize(ctx->stream);
        if (e == hipSuccess) e = hipMemcpy(po32.data(), packed_offsets_dev, (size_t)num_experts * 4, hipMemcpyDeviceToHost);
        if (e == hipSuccess) e = hipMemcpy(so32.data(), scales_offsets_dev, (size_t)num_experts * 4, hipMemcpyDeviceToHost);
        if (e != hipSuccess) { api_fail(TWM_DEVICE_ERROR, "%s: reading the offset tables: %s", who, hipGetErrorString(e)); return nullptr; }
    }
    std::vector<size_t> po(num_experts), so(num_experts);
    for (uint32_t x = 0; x < num_experts; x++) {
        // the reference's kernel reads a record as four 32-bit words (quantize_indirect.rs:216-218): 4-byte alignment
        if (po32[x] % 4 != 0) { api_fail(TWM_SHAPE_ERROR, "%s: packed offset of expert %u (%u) is not 4-byte aligned", who, x, po32[x]); return nullptr; }
        po[x] = po32[x];
        so[x] = so32[x];
    }
    return bank_build(ctx, who, packed_base_dev, scales_base_dev, po, so, k, n, num_experts, pair_gate_up);
}

void twm_bank_destroy(twm_bank *b)
{
    if (!b) return;
    if (b->cq) {
        (void)hipStreamSynchronize(b->ctx->stream);
        (void)hipFree(b->cq);
    }
    delete b;
}

size_t twm_bank_bytes(const twm_bank *b) { return b ? b->bytes : 0; }

static BankView bank_view(const twm_bank *b)
{
    BankView v;
    v.cq = b->cq;
    v.expert_bytes = b->expert_bytes;
    v.experts = b->experts;
    v.k = b->k;
    v.n = b->n;
    v.n_pad = b->n_pad;
    v.k_chunks = b->k_chunks;
    return v;
}

static int bank_common_checks(const char *who, twm_ctx *ctx, const twm_bank *b, const void *a_dev, int a_dtype)
{
    if (!ctx || !b) return api_fail(TWM_INVALID_HANDLE, "%s: null handle", who);
    if (b->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "%s: bank belongs to another context", who);
    if (a_dtype != TWM_F16 && a_dtype != TWM_F32) return api_fail(TWM_UNSUPPORTED_OP, "%s: activations must be f16 or f32", who);
    if (b->k != 0 && b->n != 0) {
        if (!a_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null activations", who);
        if (((uintptr_t)a_dev & 15) != 0) return api_fail(TWM_SHAPE_ERROR, "%s: activations must be 16-byte aligned", who);
    }
    return TWM_OK;
}

int twm_bank_gemv(twm_ctx *ctx, const twm_bank *b, const void *a_dev, int a_dtype, uint32_t a_slot_stride,
                  const float *topk_ids_dev, uint32_t top_k, int act, float *out_dev)
{
    if (int rc = bank_common_checks("twm_bank_gemv", ctx, b, a_dev, a_dtype)) return rc;
    if (act < 0 || act > 2) return api_fail(TWM_UNSUPPORTED_OP, "twm_bank_gemv: act must be 0 (none), 1 (GEGLU) or 2 (SwiGLU)");
    if (act != 0 && !b->paired) return api_fail(TWM_UNSUPPORTED_OP, "twm_bank_gemv: a fused gate needs a bank built with pair_gate_up");
    if (top_k == 0 || b->n == 0) return TWM_OK;
    if (top_k > 65535u) return api_fail(TWM_SHAPE_ERROR, "twm_bank_gemv: at most 65535 slots per call");
    if (!topk_ids_dev || !out_dev) return api_fail(TWM_INVALID_HANDLE, "twm_bank_gemv: null pointer");
    uint32_t width = act ? b->n / 2 : b->n;
    if (b->k == 0 || b->experts == 0) return twm_memset_zero(ctx, out_dev, (size_t)top_k * width * 4);  // gate(0) * 0 = 0
    // every slot's row must keep the 16-byte alignment of the loads
    if ((a_slot_stride * (a_dtype == TWM_F32 ? 4u : 2u)) % 16u != 0)
        return api_fail(TWM_SHAPE_ERROR, "twm_bank_gemv: the activation stride must keep rows 16-byte aligned");
    HIP_TRY(launch_bank_gemv(ctx->stream, bank_view(b), a_dev, a_dtype == TWM_F32, a_slot_stride, topk_ids_dev, top_k, act, out_dev,
                             ctx->force_sub, ctx->force_waves),
            TWM_DEVICE_ERROR, "bank gemv launch");
    return TWM_OK;
}

int twm_bank_down_axpy(twm_ctx *ctx, const twm_bank *b, const void *a_all_dev, int a_dtype, const float *topk_ids_dev,
                       const float *topk_weights_dev, uint32_t top_k, float *acc_dev)
{
    if (int rc = bank_common_checks("twm_bank_down_axpy", ctx, b, a_all_dev, a_dtype)) return rc;
    if (top_k == 0 || b->n == 0 || b->k == 0 || b->experts == 0) return TWM_OK;  // nothing is added
    if (top_k > (uint32_t)kMaxBankSlots) return api_fail(TWM_SHAPE_ERROR, "twm_bank_down_axpy: at most %d slots per call, got %u", kMaxBankSlots, top_k);
    if (!topk_ids_dev || !topk_weights_dev || !acc_dev) return api_fail(TWM_INVALID_HANDLE, "twm_bank_down_axpy: null pointer");
    if ((b->k * (a_dtype == TWM_F32 ? 4u : 2u)) % 16u != 0)
        return api_fail(TWM_SHAPE_ERROR, "twm_bank_down_axpy: K must keep the activation rows 16-byte aligned");
    HIP_TRY(launch_bank_down_axpy(ctx->stream, bank_view(b), a_all_dev, a_dtype == TWM_F32, topk_ids_dev, topk_weights_dev, top_k, acc_dev,
                                  ctx->force_sub, ctx->force_waves),
            TWM_DEVICE_ERROR, "bank down_axpy launch");
    return TWM_OK;
}

/* ---- the reference's MoE launches on its own slabs (no bank) ------------------------------------ */

static int raw_checks(const char *who, twm_ctx *ctx, const float *a_dev, const uint8_t *packed_buf_dev,
                      const uint16_t *scales_buf_dev, uint32_t n, uint32_t k)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "%s: null context", who);
    if (int rc = check_kn(who, k, n)) return rc;
    if (!a_dev || !packed_buf_dev || !scales_buf_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null input", who);
    // the reference kernels read a record as four 32-bit words: 4-byte alignment is their own limit
    if (((uintptr_t)packed_buf_dev & 3) != 0) return api_fail(TWM_SHAPE_ERROR, "%s: packed must be 4-byte aligned", who);
    if (((uintptr_t)a_dev & 15) != 0 || (k * 4u) % 16u != 0)
        return api_fail(TWM_SHAPE_ERROR, "%s: activation rows must be 16-byte aligned", who);
    return TWM_OK;
}

int twm_batched_marlin_gate_up(twm_ctx *ctx, const float *input_dev, const uint8_t *packed_buf_dev,
                               const uint16_t *scales_buf_dev, const float *topk_ids_dev, float *output_dev,
                               uint32_t packed_bytes_per_expert, uint32_t scales_per_expert, uint32_t n, uint32_t k,
                               uint32_t top_k)
{
    const char *who = "twm_batched_marlin_gate_up";
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "%s: null context", who);
    if (int rc = check_kn(who, k, n)) return rc;
    if (top_k == 0 || n == 0) return TWM_OK;
    if (top_k > 65535u) return api_fail(TWM_SHAPE_ERROR, "%s: at most 65535 slots per call", who);
    if (!output_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null output", who);
    if (k == 0) return twm_memset_zero(ctx, output_dev, (size_t)top_k * n * 4);
    if (int rc = raw_checks(who, ctx, input_dev, packed_buf_dev, scales_buf_dev, n, k)) return rc;
    if (!topk_ids_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null ids", who);
    if (packed_bytes_per_expert % 4u != 0) return api_fail(TWM_SHAPE_ERROR, "%s: the packed stride must be a multiple of 4", who);
    const RawView v = {packed_buf_dev, scales_buf_dev, packed_bytes_per_expert, scales_per_expert, nullptr, nullptr, 0, k, n};
    HIP_TRY(launch_raw_gemv(ctx->stream, v, input_dev, 0, topk_ids_dev, top_k, output_dev, ctx->force_sub, ctx->force_waves),
            TWM_DEVICE_ERROR, "expert gemv launch");
    return TWM_OK;
}

int twm_batched_marlin_down_axpy(twm_ctx *ctx, const float *geglu_all_dev, const uint8_t *packed_buf_dev,
                                 const uint16_t *scales_buf_dev, const float *topk_ids_dev, const float *topk_weights_dev,
                                 float *acc_dev, uint32_t packed_bytes_per_expert, uint32_t scales_per_expert, uint32_t n,
                                 uint32_t k, uint32_t top_k)
{
    const char *who = "twm_batched_marlin_down_axpy";
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "%s: null context", who);
    if (int rc = check_kn(who, k, n)) return rc;
    if (top_k == 0 || n == 0 || k == 0) return TWM_OK;  // nothing is added
    if (int rc = raw_checks(who, ctx, geglu_all_dev, packed_buf_dev, scales_buf_dev, n, k)) return rc;
    if (!topk_ids_dev || !topk_weights_dev || !acc_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null pointer", who);
    if (packed_bytes_per_expert % 4u != 0) return api_fail(TWM_SHAPE_ERROR, "%s: the packed stride must be a multiple of 4", who);
    const RawView v = {packed_buf_dev, scales_buf_dev, packed_bytes_per_expert, scales_per_expert, nullptr, nullptr, 0, k, n};
    HIP_TRY(launch_raw_down_axpy(ctx->stream, v, geglu_all_dev, topk_ids_dev, topk_weights_dev, top_k, acc_dev, ctx->force_sub,
                                 ctx->force_waves),
            TWM_DEVICE_ERROR, "expert down_axpy launch");
    return TWM_OK;
}

int twm_batched_marlin_split_geglu(twm_ctx *ctx, const float *gate_up_dev, float *output_dev, uint32_t moe_dim, uint32_t top_k)
{
    return twm_geglu_rows(ctx, gate_up_dev, top_k, moe_dim, 0, output_dev);
}

int twm_gemm_tw_marlin_m1_indirect(twm_ctx *ctx, const float *a_dev, const uint8_t *packed_buf_dev,
                                   const uint32_t *packed_offsets_dev, const uint16_t *scales_buf_dev,
                                   const uint32_t *scales_offsets_dev, int expert_idx, float *c_dev, uint32_t n, uint32_t k)
{
    const char *who = "twm_gemm_tw_marlin_m1_indirect";
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "%s: null context", who);
    if (int rc = check_kn(who, k, n)) return rc;
    if (n == 0) return TWM_OK;
    if (!c_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null output", who);
    if (k == 0) return twm_memset_zero(ctx, c_dev, (size_t)n * 4);
    if (int rc = raw_checks(who, ctx, a_dev, packed_buf_dev, scales_buf_dev, n, k)) return rc;
    if (!packed_offsets_dev || !scales_offsets_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null offset table", who);
    if (expert_idx < 0) return api_fail(TWM_SHAPE_ERROR, "%s: negative expert index %d", who, expert_idx);
    const RawView v = {packed_buf_dev, scales_buf_dev, 0, 0, packed_offsets_dev, scales_offsets_dev, expert_idx, k, n};
    HIP_TRY(launch_raw_gemv(ctx->stream, v, a_dev, 0, nullptr, 1, c_dev, ctx->force_sub, ctx->force_waves), TWM_DEVICE_ERROR,
            "expert gemv launch");
    return TWM_OK;
}

int twm_geglu_rows(twm_ctx *ctx, const float *gate_up_dev, uint32_t batch, uint32_t dim, int paired, float *out_dev)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_geglu_rows: null context");
    if (paired && dim % kPairWidth != 0)
        return api_fail(TWM_SHAPE_ERROR, "twm_geglu_rows: the paired order needs dim %% %u == 0, got %u", kPairWidth, dim);
    if ((uint64_t)dim * 2 > 0xFFFFFFFFull) return api_fail(TWM_SHAPE_ERROR, "twm_geglu_rows: 2 * dim overflows u32");
    if ((uint64_t)batch * dim == 0) return TWM_OK;
    if (!gate_up_dev || !out_dev) return api_fail(TWM_INVALID_HANDLE, "twm_geglu_rows: null pointer");
    HIP_TRY(launch_geglu_rows(ctx->stream, gate_up_dev, out_dev, dim, batch, paired != 0), TWM_DEVICE_ERROR, "geglu_rows launch");
    return TWM_OK;
}

/* ---- graphs ---------------------------------------------------------------------------------- */

int twm_graph_begin(twm_ctx *ctx)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_graph_begin: null context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_graph_begin: a capture is already open");
    if (ctx->stream == nullptr) return api_fail(TWM_UNSUPPORTED_OP, "twm_graph_begin: cannot capture the null stream");
    HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed), TWM_DEVICE_ERROR, "hipStreamBeginCapture");
    ctx->capturing = true;
    return TWM_OK;
}

twm_graph *twm_graph_end(twm_ctx *ctx)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_graph_end: null context"); return nullptr; }
    if (!ctx->capturing) { api_fail(TWM_UNSUPPORTED_OP, "twm_graph_end: no capture is open"); return nullptr; }
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (e != hipSuccess || !graph) {
        api_fail(TWM_DEVICE_ERROR, "hipStreamEndCapture: %s", hipGetErrorString(e));
        return nullptr;
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        api_fail(TWM_DEVICE_ERROR, "hipGraphInstantiate: %s", hipGetErrorString(e));
        (void)hipGraphDestroy(graph);
        return nullptr;
    }
    twm_graph *g = new (std::nothrow) twm_graph();
    if (!g) {
        api_fail(TWM_MEMORY_ERROR, "twm_graph_end: out of host memory");
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        return nullptr;
    }
    g->graph = graph;
    g->exec = exec;
    return g;
}

int twm_graph_launch(twm_ctx *ctx, twm_graph *g)
{
    if (!ctx || !g) return api_fail(TWM_INVALID_HANDLE, "twm_graph_launch: null handle");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_graph_launch: a capture is open");
    HIP_TRY(hipGraphLaunch(g->exec, ctx->stream), TWM_DEVICE_ERROR, "hipGraphLaunch");
    return TWM_OK;
}

void twm_graph_destroy(twm_graph *g)
{
    if (!g) return;
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->graph);
    delete g;
}

}  // extern "C"

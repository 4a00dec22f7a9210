// C ABI of libtwmarlin_hip.so (declared in include/twmarlin.h), part: contexts and their options, device memory,
// events, the format operations, the GEMV on the reference's own arrays and hipGraph capture/replay.  Host-side
// counterpart of the reference's crates/kernels/src/{quantize.rs:1301-1360, device.rs, tensor.rs, cuda_graph.rs}.
// (Weight handles: twm_api_weights.hip; the dispatcher of twm_gemm: twm_api_gemm.hip; expert banks: twm_api_moe.hip.)
#include "twm_api_impl.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <string>
#include <vector>

using namespace twm;

static thread_local std::string g_err;
static thread_local int g_err_kind = TWM_KIND_NONE;

int twm::api_fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    g_err_kind = code == TWM_MEMORY_ERROR ? TWM_KIND_MEMORY : code == TWM_DEVICE_ERROR ? TWM_KIND_LAUNCH : TWM_KIND_NONE;
    return code;
}

void twm::set_error_kind(int kind) { g_err_kind = kind; }

extern "C" {

const char *twm_version(void) { return "0.1.0"; }

int twm_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

const char *twm_last_error(void) { return g_err.c_str(); }
int twm_last_error_kind(void) { return g_err_kind; }

twm_ctx *twm_ctx_create(int ordinal)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || ordinal < 0 || ordinal >= count) {
        api_fail(TWM_DEVICE_ERROR, "twm_ctx_create: no HIP device %d (%s)", ordinal,
             e != hipSuccess ? hipGetErrorString(e) : "ordinal out of range");
        set_error_kind(TWM_KIND_INIT);
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
    c->trace = TraceBuf{nullptr, 0};
    c->dequant_src = 0;
    c->weight_copies = 0;
    c->tune_on_upload = 0;
    c->m1_exact = 0;
    c->m1_align16 = 0;
    c->m1_splits = 0;
    c->batch_rounded = 0;
    c->prefill_bm = 0;
    c->prefill_min_m = 33;  // M <= 32 is batched decode (exact f32 scales, weights streamed once)
    c->ws = nullptr;
    c->counters = nullptr;
    c->own_stream = nullptr;
    bool ok = hipSetDevice(ordinal) == hipSuccess && hipGetDeviceProperties(&c->prop, ordinal) == hipSuccess;
    if (ok && strncmp(c->prop.gcnArchName, "gfx950", 6) != 0) {
        api_fail(TWM_DEVICE_ERROR, "twm_ctx_create: device %d is %s; this library holds gfx950 code only", ordinal,
             c->prop.gcnArchName);
        set_error_kind(TWM_KIND_CODE_OBJECT);
        delete c;
        return nullptr;
    }
    ok = ok && hipStreamCreateWithFlags(&c->own_stream, hipStreamNonBlocking) == hipSuccess;
    ok = ok && init_prefill() == hipSuccess;
    ok = ok && noalloc_scratch_for_current_device("twm_ctx_create") != nullptr;
    c->stream = c->own_stream;
    c->ws_bytes = kWsBytes;
    c->n_counters = kCounters;
    ok = ok && hipMalloc((void **)&c->ws, c->ws_bytes) == hipSuccess;
    ok = ok && hipMalloc((void **)&c->counters, c->n_counters * sizeof(unsigned)) == hipSuccess;
    ok = ok && hipMemset(c->counters, 0, c->n_counters * sizeof(unsigned)) == hipSuccess;
    ok = ok && hipDeviceSynchronize() == hipSuccess;
    if (!ok) {
        api_fail(TWM_DEVICE_ERROR, "twm_ctx_create: %s", hipGetErrorString(hipGetLastError()));
        set_error_kind(TWM_KIND_INIT);
        if (c->ws) (void)hipFree(c->ws);
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
        api_fail(TWM_DEVICE_ERROR, "twm_ctx_sync: %s", hipGetErrorString(e));
        set_error_kind(TWM_KIND_SYNC);
        return TWM_DEVICE_ERROR;
    }
    return TWM_OK;
}

void *twm_stream_create(twm_ctx *ctx)
{
    if (!ctx) { api_fail(TWM_INVALID_HANDLE, "twm_stream_create: null context"); return nullptr; }
    hipStream_t s = nullptr;
    hipError_t e = hipSetDevice(ctx->ordinal);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    if (e != hipSuccess) {
        api_fail(TWM_DEVICE_ERROR, "twm_stream_create: %s", hipGetErrorString(e));
        set_error_kind(TWM_KIND_INIT);
        return nullptr;
    }
    return (void *)s;
}

int twm_stream_destroy(twm_ctx *ctx, void *hip_stream)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_stream_destroy: null context");
    if (!hip_stream) return TWM_OK;
    if ((hipStream_t)hip_stream == ctx->own_stream) return api_fail(TWM_INVALID_HANDLE, "twm_stream_destroy: that is the context's own stream");
    if ((hipStream_t)hip_stream == ctx->stream) return api_fail(TWM_UNSUPPORTED_OP, "twm_stream_destroy: the context still issues its work on this stream (twm_ctx_set_stream first)");
    HIP_TRY(hipStreamDestroy((hipStream_t)hip_stream), TWM_DEVICE_ERROR, "twm_stream_destroy");
    return TWM_OK;
}

int twm_stream_sync(twm_ctx *ctx, void *hip_stream)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_stream_sync: null context");
    hipError_t e = hipStreamSynchronize((hipStream_t)hip_stream);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        api_fail(TWM_DEVICE_ERROR, "twm_stream_sync: %s", hipGetErrorString(e));
        set_error_kind(TWM_KIND_SYNC);
        return TWM_DEVICE_ERROR;
    }
    return TWM_OK;
}

int twm_debug_trace(twm_ctx *ctx, uint32_t *trace_dev, uint32_t capacity_workgroups)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_debug_trace: null context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_debug_trace: a graph capture is open");
    ctx->trace.ptr = capacity_workgroups ? trace_dev : nullptr;
    ctx->trace.capacity = trace_dev ? capacity_workgroups : 0;
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
    if (strcmp(key, "prefill_min_m") == 0) {
        if (value < 1) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: prefill_min_m must be >= 1");
        ctx->prefill_min_m = value;
        return TWM_OK;
    }
    if (strcmp(key, "tune_on_upload") == 0) {
        if (value < 0 || value > 2) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: tune_on_upload must be 0, 1 or 2");
        ctx->tune_on_upload = value;
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
    if (strcmp(key, "m1_align16") == 0) {
        if (value != 0 && value != 1) return api_fail(TWM_SHAPE_ERROR, "twm_ctx_set_option: m1_align16 must be 0 or 1");
        ctx->m1_align16 = value;
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
    if (e != hipSuccess) {
        (void)hipGetLastError();  // (the runtime keeps the error for the next caller of hipGetLastError otherwise)
        api_fail(TWM_MEMORY_ERROR, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
        return nullptr;
    }
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

int twm_cast_f32_to_f16(twm_ctx *ctx, const float *src_dev, uint16_t *dst_dev, size_t count)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_cast_f32_to_f16: null context");
    if (count == 0) return TWM_OK;
    if (!src_dev || !dst_dev) return api_fail(TWM_INVALID_HANDLE, "twm_cast_f32_to_f16: null buffer");
    HIP_TRY(launch_cast(ctx->stream, src_dev, dst_dev, count, true), TWM_DEVICE_ERROR, "cast kernel launch");
    return TWM_OK;
}

int twm_cast_f16_to_f32(twm_ctx *ctx, const uint16_t *src_dev, float *dst_dev, size_t count)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_cast_f16_to_f32: null context");
    if (count == 0) return TWM_OK;
    if (!src_dev || !dst_dev) return api_fail(TWM_INVALID_HANDLE, "twm_cast_f16_to_f32: null buffer");
    HIP_TRY(launch_cast(ctx->stream, src_dev, dst_dev, count, false), TWM_DEVICE_ERROR, "cast kernel launch");
    return TWM_OK;
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

extern "C++" int check_pair_args(const char *who, uint32_t k, uint32_t ffn_dim)
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

// The launch form of the GEMV on the reference's arrays: chosen here, launched by m1_dispatch, described by
// twm_plan_describe_m1.  Nothing here touches the device.
enum M1Kind { kM1RefOrder = 0, kM1SubTile = 1, kM1WholeTile = 2 };
struct M1Form {
    int kind;
    uint32_t sub, waves, splits;  // sub-tile width (sub-tile form), waves per workgroup, K-splits over workgroups
};
// aligned16: activations and packed records at 16-byte addresses (the MFMA kernels' loads); ws_bytes / n_counters: the
// split-K scratch at hand
static M1Form choose_m1_form(int exact, int force_sub, int force_waves, int force_splits, size_t ws_bytes, uint32_t n_counters,
                             bool aligned16, uint32_t n, uint32_t k)
{
    M1Form f = {kM1RefOrder, 0, 0, 1};
    if (exact || !aligned16) return f;  // f32 activations, f32 FMAs, the reference kernel's order and its own split-K rule
    // the M <= 4 MFMA kernels reading the reference's arrays as they are (f32 activations as two f16 terms)
    const uint32_t n_pad = ((n + 63) / 64) * 64, k_chunks = (k / 32 + kChunkGroups - 1) / kChunkGroups;
    // On the reference's arrays a wave's four group rows of a chunk are N x 16 bytes apart, and many waves in flight
    // with one pass each pay better than on the contiguous copy.  The sub-tile kernel on 16 columns when 64-column tiles
    // number no more than 64 (any K: deeper ones in the pipelined pass loop on sixteen waves: 18944 -> 3584 10.8 us,
    // 14336 -> 4096 9.7) and, eight waves of one pass each, on wide matrices up to K = 4096 (3584 -> 37888 16.3 against
    // 18.1 us on 32 columns, 4096 -> 22016 11.8 against 12.5, 4096 -> 28672 14.6 against 15.8); in between sixteen waves
    // on 32 columns as long as every wave gets a single pass (3584 -> 4608 4.7 against 4.9, 4096 -> 6144 5.1 against
    // 5.5).  Deeper matrices of 256 tiles or more keep the 64-column kernel (its K-split only by option; 8192 -> 57344: 46.6 against
    // 63.7 us).
    // Fitted to sweeps over the Qwen2.5-7B, Llama-2-7B, Llama-3-8B, 13B and 70B projections; option "sub" = 1 keeps the
    // 64-column kernel.
    const uint32_t tiles64 = n_pad / 64, passes16 = (k_chunks + 3) / 4, passes32 = (k_chunks + 1) / 2;
    const bool narrow16 = tiles64 <= 64, wide16 = tiles64 >= 256 && passes16 <= 8;
    // K of 6144 .. 8192 from 128 tiles on: sixteen waves of one pass each on 16 columns (8192 -> 8192 8.9 against 10.0 us on
    // 32 columns, 8192 -> 10240 11.4 / 14.3, 8192 -> 28672 25.0 / 26.2 on whole tiles, 6144 -> 16384 12.4 / 13.2, 6656 -> 13312
    // 12.4 / 12.9, 8192 -> 57344 level; not K = 5120 (5120 -> 15360 11.1 / 10.6) nor fewer tiles (7168 -> 7168 8.2 / 7.9))
    const bool deep16 = tiles64 >= 128 && passes16 >= 12 && passes16 <= 16;
    uint32_t sub = narrow16 || wide16 || deep16 ? 16 : 32, sub_waves = (sub == 16 && passes16 <= 8) ? 8 : 16;
    // 65 .. 255 tiles on a deeper K: still 32 columns, the waves looping over their passes -- sixteen of them up to 128
    // tiles and 160 chunks, eight beyond (13824 -> 5120 12.2 against 14.6 us on whole tiles with a K-split, 8192 -> 8192
    // 9.4 / 12.4, 18944 -> 4608 15.3 / 17.1, 28672 -> 8192 24.2 / 27.5, 8192 -> 10240 14.2 / 15.1, 5120 -> 15360 10.5 / 11.0)
    const bool mid32 = !narrow16 && tiles64 < 256 && passes32 > 16;
    if (mid32 && !(tiles64 <= 128 && k_chunks <= 160)) sub_waves = 8;
    bool use_sub = force_sub != 1 && (sub == 16 || passes32 <= 16 || mid32);
    if (force_sub >= 16) {
        sub = (uint32_t)force_sub;
        sub_waves = 8;
        use_sub = true;
    }
    if (use_sub) {
        uint32_t sp = force_splits ? (uint32_t)force_splits : 1;
        if (!force_splits && sub == 16 && n_pad / 16 <= 64) {
            // A few sub-tiles on a very deep K (16384 -> 256 is sixteen workgroups): cut K over workgroups while that
            // leaves each at least 64 chunks and the workgroups within the CU count -- the hand-over between workgroups
            // (partial sums of a few KB, the last to arrive adds them in split order) costs over a microsecond, and only
            // such ranges are worth it: 16384 -> 256 5.70 us on two ranges against 6.76 on one (four 5.62, eight 7.02),
            // 32768 -> 64 6.09 on four against 12.57; but 8192 -> 200 4.30 on one against 4.76 on two, 4096 -> 1000 3.28 / 4.54.
            while (n_pad / 16 * sp * 2 <= 256 && k_chunks / (sp * 2) >= 64) sp *= 2;
        }
        if (force_waves) sub_waves = (uint32_t)force_waves;
        if (sp > k_chunks) sp = k_chunks;
        while (sp > 1 && (size_t)sp * n_pad * 4 > ws_bytes) sp--;
        if (n_pad / sub > n_counters) sp = 1;
        return M1Form{kM1SubTile, sub, sub_waves, sp};
    }
    // (only matrices of 256 tiles or more on a deep K get here, or option "sub" = 1: no K-split of its own; sixteen
    // waves where there are fewer tiles than CUs)
    f.kind = kM1WholeTile;
    f.waves = tiles64 < 256 ? 16 : 8;
    if (force_waves) f.waves = (uint32_t)force_waves;
    if (force_splits) f.splits = (uint32_t)force_splits;
    if (f.splits > k_chunks) f.splits = k_chunks;
    while (f.splits > 1 && (size_t)f.splits * n_pad * 4 > ws_bytes) f.splits--;
    if (tiles64 > n_counters) f.splits = 1;
    return f;
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
    const bool aligned16 = ((uintptr_t)a_dev & 15) == 0 && ((uintptr_t)packed_dev & 15) == 0;
    const M1Form f = choose_m1_form(env.exact, env.force_sub, env.force_waves, env.splits, env.ws_bytes, env.n_counters, aligned16, n, k);
    const uint32_t n_pad = ((n + 63) / 64) * 64;
    switch (f.kind) {
    case kM1RefOrder: {
        uint32_t nb, sp, gps;
        twm_pick_splits_reference(k, n, &nb, &sp, &gps);
        HIP_TRY(launch_ref_gemv(env.stream, a_dev, packed_dev, scales_dev, c_dev, n, k, sp, gps), TWM_DEVICE_ERROR, "gemv launch");
        return TWM_OK;
    }
    case kM1SubTile:
        if (f.splits > 1 && env.clear_counters)
            HIP_TRY(launch_fill_zero(env.stream, env.counters, (size_t)(n_pad / f.sub) * 4), TWM_DEVICE_ERROR, "fill kernel launch");
        HIP_TRY(launch_gemv4s_ref(env.stream, packed_dev, scales_dev, k, n, a_dev, c_dev, env.ws, env.counters, f.sub, f.waves, f.splits),
                TWM_DEVICE_ERROR, "sub-tile gemv launch");
        return TWM_OK;
    default:
        if (f.splits > 1 && env.clear_counters)
            HIP_TRY(launch_fill_zero(env.stream, env.counters, (size_t)(n_pad / 64) * 4), TWM_DEVICE_ERROR, "fill kernel launch");
        HIP_TRY(launch_gemv4_ref(env.stream, packed_dev, scales_dev, k, n, a_dev, c_dev, env.ws, env.counters, f.waves, f.splits),
                TWM_DEVICE_ERROR, "gemv launch");
        return TWM_OK;
    }
}

int twm_plan_describe_m1(const twm_ctx *ctx, uint32_t k, uint32_t n, char *text, size_t bytes)
{
    if (!text || bytes == 0) return api_fail(TWM_INVALID_HANDLE, "twm_plan_describe_m1: null buffer");
    if (int rc = check_kn("twm_plan_describe_m1", k, n)) return rc;
    if (n == 0 || k == 0) {
        snprintf(text, bytes, n == 0 ? "nothing to launch" : "k_fill_zero");
        return TWM_OK;
    }
    const M1Form f = ctx ? choose_m1_form(ctx->m1_exact, ctx->force_sub, ctx->force_waves, ctx->m1_splits, ctx->ws_bytes, ctx->n_counters, true, n, k)
                         : choose_m1_form(0, 0, 0, 0, kWsBytes, kCounters, true, n, k);
    switch (f.kind) {
    case kM1RefOrder: {
        uint32_t nb, sp, gps;
        twm_pick_splits_reference(k, n, &nb, &sp, &gps);
        snprintf(text, bytes, "k_ref_gemv: one thread per column, %u K-split%s (the reference's rule); reference arrays", sp, sp == 1 ? "" : "s");
        break;
    }
    case kM1SubTile:
        snprintf(text, bytes, "k_gemv4s: %u-column sub-tiles, %u waves, %u K-split%s; reference arrays", f.sub, f.waves, f.splits,
                 f.splits == 1 ? "" : "s");
        break;
    default:
        snprintf(text, bytes, "k_gemv4: 1 x 64-column tiles per workgroup, %u waves, %u K-split%s; reference arrays", f.waves, f.splits,
                 f.splits == 1 ? "" : "s");
        break;
    }
    return TWM_OK;
}

int twm_gemm_tw_marlin_m1(twm_ctx *ctx, const float *a_dev, const uint8_t *packed_dev, const uint16_t *scales_dev,
                          float *c_dev, uint32_t n, uint32_t k)
{
    if (!ctx) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_tw_marlin_m1: null context");
    if (ctx->m1_align16 && !ctx->m1_exact && ((((uintptr_t)a_dev | (uintptr_t)packed_dev) & 15) != 0))
        return api_fail(TWM_SHAPE_ERROR, "twm_gemm_tw_marlin_m1: activations or packed weights are not 16-byte aligned "
                                         "(option m1_align16: the 4-byte path, k_ref_gemv, is about 3.6 times slower)");
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

// C ABI, part: expert banks for mixture-of-experts decode and the reference's MoE launches on its raw slabs
// (crates/kernels/src/moe_batched_marlin.rs, quantize_indirect.rs).
#include "twm_api_impl.h"

using namespace twm;

extern "C" {

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

}  // extern "C"

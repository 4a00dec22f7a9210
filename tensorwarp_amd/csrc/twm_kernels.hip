// gfx950 (CDNA4, wave64) kernels for the TW-Marlin W4A16 quantized-linear path.
//
// Reference semantics (crates/kernels/src/quantize.rs in the reference checkout):
//   GEMV arithmetic ............ :1186-1298   (warp_gemm_tw_marlin_m1[_direct])
//   Q4 unpack to FP16 .......... :534-571     (warp_dequant_q4_to_f16)
//   quantizer .................. :414-474, crates/loader/src/gemma_moe_q4.rs:218-254
//   reorder / fuse ............. :912-956, :1018-1063
//   split_qkv / split_gate_up .. crates/kernels/src/ops.rs:2255-2297
// This file holds the format operations, the GEMV on the reference layout and the repacks into
// the two streaming orders; the MFMA kernels that stream the repacked weights are in twm_gemv4*.hip,
// twm_stream.hip, twm_batch.hip and twm_prefill.hip.
#include "twm_device.h"

namespace twm {

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h)
{
    union { uint16_t u; _Float16 f; } x;
    x.u = h;
    return (float)x.f;  // v_cvt_f32_f16: exact, subnormals kept
}

// scale * q for the Q4 unpack.  The value is pinned in a register between the convert and the
// multiply: left alone, the compiler folds both into v_fma_mix*(s, q, +0), and x*y + (+0) turns
// the product -0.0 (zero scale, negative q) into +0.0, which is not the reference's bit pattern.
__device__ __forceinline__ float scale_times_q(uint16_t scale_bits, int q)
{
    float s = f16_bits_to_f32(scale_bits);
    asm volatile("" : "+v"(s));
    float w = s * (float)q;
    asm volatile("" : "+v"(w));
    return w;
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f)
{
    union { uint16_t u; _Float16 h; } x;
    x.h = (_Float16)f;  // v_cvt_f16_f32: round to nearest even
    return x.u;
}

// ---------------------------------------------------------------------------------
// fill
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_fill_zero(uint32_t *p, size_t words)
{
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t stride = (size_t)gridDim.x * 256;
    for (; i < words; i += stride) p[i] = 0u;
}

hipError_t launch_fill_zero(hipStream_t s, void *ptr, size_t bytes)
{
    size_t words = bytes / 4;
    if (words == 0) return hipSuccess;
    size_t blocks = (words + 255) / 256;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(k_fill_zero, dim3((unsigned)blocks), dim3(256), 0, s, (uint32_t *)ptr, words);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// casts between f32 and f16 rows (crates/kernels/src/fp16.rs:133-166): round to nearest even, as __float2half
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_cast_f32_f16(const float *__restrict__ src, _Float16 *__restrict__ dst, size_t count)
{
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t stride = (size_t)gridDim.x * 256;
    for (; i < count; i += stride) dst[i] = (_Float16)src[i];
}
__global__ __launch_bounds__(256) void k_cast_f16_f32(const _Float16 *__restrict__ src, float *__restrict__ dst, size_t count)
{
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t stride = (size_t)gridDim.x * 256;
    for (; i < count; i += stride) dst[i] = (float)src[i];
}

hipError_t launch_cast(hipStream_t s, const void *src, void *dst, size_t count, bool to_f16)
{
    if (count == 0) return hipSuccess;
    size_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (to_f16) hipLaunchKernelGGL(k_cast_f32_f16, dim3((unsigned)blocks), dim3(256), 0, s, (const float *)src, (_Float16 *)dst, count);
    else hipLaunchKernelGGL(k_cast_f16_f32, dim3((unsigned)blocks), dim3(256), 0, s, (const _Float16 *)src, (float *)dst, count);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// quantizer: one thread per (group, column)
// ---------------------------------------------------------------------------------
struct QGroup {
    float scale;
    uint32_t w[4];
};

__device__ __forceinline__ QGroup quantize_group32(const float *vals)
{
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        float a = fabsf(vals[i]);
        if (a > amax) amax = a;  // NaN never wins, as with Rust's f32::max fold
    }
    QGroup r;
    r.scale = amax / 7.0f;                                 // correctly rounded division
    float inv = (r.scale != 0.0f) ? 7.0f / amax : 0.0f;
#pragma unroll
    for (int wi = 0; wi < 4; wi++) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            float rv = roundf(vals[wi * 8 + j] * inv);     // half away from zero
            int q = (rv != rv) ? 0 : (int)fminf(fmaxf(rv, -64.0f), 64.0f);
            q += 8;
            q = q < 0 ? 0 : (q > 15 ? 15 : q);
            word |= (uint32_t)q << (4 * j);
        }
        r.w[wi] = word;
    }
    return r;
}

// w row-major [K,N] (is_nk == 0) or [N,K] (is_nk != 0)
__device__ __forceinline__ void gather_group(const float *w, int is_nk, uint32_t k, uint32_t n, uint32_t g,
                                             uint32_t col, float *vals)
{
    if (is_nk) {
        const float4 *p = (const float4 *)(w + (size_t)col * k + (size_t)g * 32);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float4 v = p[i];
            vals[4 * i] = v.x; vals[4 * i + 1] = v.y; vals[4 * i + 2] = v.z; vals[4 * i + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 32; i++) vals[i] = w[((size_t)g * 32 + i) * n + col];
    }
}

__global__ __launch_bounds__(256) void k_quantize_q4_0(const float *__restrict__ w, uint32_t k, uint32_t n,
                                                        uint8_t *__restrict__ q4)
{
    uint32_t groups = k / 32;
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // idx = g * n + col (coalesced reads of [K,N])
    if (idx >= (size_t)groups * n) return;
    uint32_t g = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
    float vals[32];
    gather_group(w, 0, k, n, g, col, vals);
    QGroup r = quantize_group32(vals);
    uint32_t *dst = (uint32_t *)(q4 + ((size_t)col * groups + g) * 20);  // 20-byte blocks are 4-byte aligned
    dst[0] = __float_as_uint(r.scale);
    dst[1] = r.w[0]; dst[2] = r.w[1]; dst[3] = r.w[2]; dst[4] = r.w[3];
}

__global__ __launch_bounds__(256) void k_quantize_twm(const float *__restrict__ w, int is_nk, uint32_t k, uint32_t n,
                                                       uint4v *__restrict__ packed, uint16_t *__restrict__ scales)
{
    uint32_t groups = k / 32;
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // g * n + col
    if (idx >= (size_t)groups * n) return;
    uint32_t g = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
    float vals[32];
    gather_group(w, is_nk, k, n, g, col, vals);
    QGroup r = quantize_group32(vals);
    uint4v o = {r.w[0], r.w[1], r.w[2], r.w[3]};
    packed[idx] = o;
    scales[idx] = f32_to_f16_bits(r.scale);
}

hipError_t launch_quantize_q4_0(hipStream_t s, const float *w_kn, uint32_t k, uint32_t n, uint8_t *q4)
{
    size_t total = (size_t)(k / 32) * n;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_q4_0, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, w_kn, k, n, q4);
    return hipGetLastError();
}

hipError_t launch_quantize_twm(hipStream_t s, const float *w, int w_is_nk, uint32_t k, uint32_t n, uint8_t *packed,
                               uint16_t *scales)
{
    size_t total = (size_t)(k / 32) * n;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_twm, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, w, w_is_nk, k, n,
                       (uint4v *)packed, scales);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// reorder Q4_0 column-major -> TW-Marlin; fuse along N
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_reorder(const uint8_t *__restrict__ q4, uint32_t groups, uint32_t n,
                                                  uint4v *__restrict__ packed, uint16_t *__restrict__ scales)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // g * n + col (coalesced writes)
    if (idx >= (size_t)groups * n) return;
    uint32_t g = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
    const uint32_t *src = (const uint32_t *)(q4 + ((size_t)col * groups + g) * 20);
    float scale = __uint_as_float(src[0]);
    uint4v o = {src[1], src[2], src[3], src[4]};
    packed[idx] = o;
    scales[idx] = f32_to_f16_bits(scale);
}

hipError_t launch_reorder(hipStream_t s, const uint8_t *q4, uint32_t k, uint32_t n, uint8_t *packed, uint16_t *scales)
{
    size_t total = (size_t)(k / 32) * n;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_reorder, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, q4, k / 32, n,
                       (uint4v *)packed, scales);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void k_fuse_one(const uint4v *__restrict__ pin, const uint16_t *__restrict__ sin,
                                                   uint32_t groups, uint32_t ni, uint32_t total_n, uint32_t col_off,
                                                   uint4v *__restrict__ pout, uint16_t *__restrict__ sout)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // g * ni + c
    if (idx >= (size_t)groups * ni) return;
    uint32_t g = (uint32_t)(idx / ni), c = (uint32_t)(idx % ni);
    size_t dst = (size_t)g * total_n + col_off + c;
    pout[dst] = pin[idx];
    sout[dst] = sin[idx];
}

hipError_t launch_fuse_one(hipStream_t s, const uint8_t *packed_in, const uint16_t *scales_in, uint32_t groups,
                           uint32_t ni, uint32_t total_n, uint32_t col_off, uint8_t *packed_out, uint16_t *scales_out)
{
    size_t total = (size_t)groups * ni;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_fuse_one, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (const uint4v *)packed_in,
                       scales_in, groups, ni, total_n, col_off, (uint4v *)packed_out, scales_out);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// Q4 unpack from the reference layout: one thread per (k-pair... ) element column-coalesced
// ---------------------------------------------------------------------------------
template <bool F16OUT>
__global__ __launch_bounds__(256) void k_dequant(const uint8_t *__restrict__ packed, const uint16_t *__restrict__ scales,
                                                  uint32_t k, uint32_t n, void *__restrict__ out)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // row * n + col
    if (idx >= (size_t)k * n) return;
    uint32_t row = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
    uint32_t g = row / 32, e = row % 32;
    uint8_t byte = packed[((size_t)g * n + col) * 16 + e / 2];
    int q = (e & 1) ? (byte >> 4) : (byte & 0xF);
    float w = scale_times_q(scales[(size_t)g * n + col], q - 8);  // exact in f32: 11-bit x 4-bit significands
    if (F16OUT) ((uint16_t *)out)[idx] = f32_to_f16_bits(w);
    else ((float *)out)[idx] = w;
}

hipError_t launch_dequant(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                          void *out, bool f16_out)
{
    size_t total = (size_t)k * n;
    if (total == 0) return hipSuccess;
    dim3 grid((unsigned)((total + 255) / 256));
    if (f16_out) hipLaunchKernelGGL(k_dequant<true>, grid, dim3(256), 0, s, packed, scales, k, n, out);
    else hipLaunchKernelGGL(k_dequant<false>, grid, dim3(256), 0, s, packed, scales, k, n, out);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// split_qkv / split_gate_up
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_split_qkv(const float *__restrict__ qkv, float *__restrict__ q,
                                                    float *__restrict__ kk, float *__restrict__ v, uint32_t h,
                                                    uint32_t kv, uint32_t batch)
{
    uint32_t per = h + 2 * kv;
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)batch * per) return;
    uint32_t b = (uint32_t)(idx / per), d = (uint32_t)(idx % per);
    float x = qkv[idx];
    if (d < h) q[(size_t)b * h + d] = x;
    else if (d < h + kv) kk[(size_t)b * kv + (d - h)] = x;
    else v[(size_t)b * kv + (d - h - kv)] = x;
}

__global__ __launch_bounds__(256) void k_split_gate_up(const float *__restrict__ gu, float *__restrict__ g,
                                                        float *__restrict__ u, uint32_t ffn, uint32_t batch)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)batch * 2 * ffn) return;
    uint32_t b = (uint32_t)(idx / (2 * ffn)), d = (uint32_t)(idx % (2 * ffn));
    float x = gu[idx];
    if (d < ffn) g[(size_t)b * ffn + d] = x;
    else u[(size_t)b * ffn + (d - ffn)] = x;
}

// silu(gate) * up, elementwise (warp_fused_silu_mul, crates/kernels/src/ops.rs:966-976).
__global__ __launch_bounds__(256) void k_silu_mul(const float *__restrict__ gate, const float *__restrict__ up,
                                                   float *__restrict__ out, size_t count)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx < count) out[idx] = silu_mul_f32(gate[idx], up[idx]);
}

// out[b][j] = silu(gate_up[b][gate column j]) * gate_up[b][up column j]: the split of
// k_split_gate_up and the SwiGLU gate in one pass.  PAIRED selects where the two columns are:
// [gate | up] halves (the reference's fused order) or the 32-column interleave of paired_col().
template <bool PAIRED>
__global__ __launch_bounds__(256) void k_swiglu_rows(const float *__restrict__ gu, float *__restrict__ out,
                                                      uint32_t ffn, uint32_t batch)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)batch * ffn) return;
    uint32_t b = (uint32_t)(idx / ffn), j = (uint32_t)(idx % ffn);
    const float *row = gu + (size_t)b * 2 * ffn;
    float g, u;
    if (PAIRED) {
        uint32_t c = paired_col(j);
        g = row[c];
        u = row[c + kPairWidth];
    } else {
        g = row[j];
        u = row[ffn + j];
    }
    out[idx] = silu_mul_f32(g, u);
}

// TW-Marlin arrays of gate and up ([G][ffn] records and scales each) -> one [G][2*ffn] pair of
// arrays in the paired column order.  Pure byte moves; one thread per (group, output column).
__global__ __launch_bounds__(256) void k_pair_gate_up(const uint4v *__restrict__ gp, const uint16_t *__restrict__ gs,
                                                       const uint4v *__restrict__ up, const uint16_t *__restrict__ us,
                                                       uint32_t groups, uint32_t ffn, uint4v *__restrict__ pout,
                                                       uint16_t *__restrict__ sout)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // g * 2*ffn + c
    size_t n2 = (size_t)2 * ffn;
    if (idx >= (size_t)groups * n2) return;
    uint32_t g = (uint32_t)(idx / n2), c = (uint32_t)(idx % n2);
    uint32_t j = (c >> 6) * kPairWidth + (c & 31u);
    size_t src = (size_t)g * ffn + j;
    bool is_up = (c & kPairWidth) != 0;
    pout[idx] = is_up ? up[src] : gp[src];
    sout[idx] = is_up ? us[src] : gs[src];
}

// ArgMax along the last dimension with the reference's rule (crates/kernels/src/missing_ops.rs:24-39): the
// first index whose value is greater than every earlier candidate, starting from -1e30 at index 0 (so
// values <= -1e30 and NaNs are never chosen, and an empty or all-small row yields 0).  One workgroup per row:
// each thread scans a strided share in increasing order, then (value, index) pairs are merged preferring
// the larger value and, among equal values, the smaller index.
__global__ __launch_bounds__(1024) void k_argmax(const float *__restrict__ in, uint32_t cols, int *__restrict__ out)
{
    __shared__ float sv[1024];
    __shared__ uint32_t si[1024];
    const float *row = in + (size_t)blockIdx.x * cols;
    float best = -1e30f;
    uint32_t idx = 0xFFFFFFFFu;  // "none yet"
    for (uint32_t c = threadIdx.x; c < cols; c += 1024u) {
        float v = row[c];
        if (v > best) {
            best = v;
            idx = c;
        }
    }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = idx;
    __syncthreads();
    for (uint32_t step = 512; step > 0; step >>= 1) {
        if (threadIdx.x < step) {
            float ov = sv[threadIdx.x + step];
            uint32_t oi = si[threadIdx.x + step];
            if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi < si[threadIdx.x])) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = si[0] == 0xFFFFFFFFu ? 0 : (int)si[0];
}

// Long rows (a vocabulary): phase 1, one workgroup per 8192 columns leaves its (value, index) candidate in
// scratch; phase 2 is k_argmax_merge over the candidates.  Same rule: larger value, then smaller index.
constexpr uint32_t kArgmaxSpan = 8192;

__global__ __launch_bounds__(1024) void k_argmax_partial(const float *__restrict__ in, uint32_t cols, uint32_t spans,
                                                          float *__restrict__ cand_val, uint32_t *__restrict__ cand_idx)
{
    __shared__ float sv[1024];
    __shared__ uint32_t si[1024];
    const float *row = in + (size_t)blockIdx.y * cols;
    const uint32_t c0 = blockIdx.x * kArgmaxSpan;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {  // all eight loads first, then the compares in increasing index order
        uint32_t c = c0 + threadIdx.x + 1024u * j;
        v[j] = c < cols ? row[c] : -1e30f;
    }
    float best = -1e30f;
    uint32_t idx = 0xFFFFFFFFu;
#pragma unroll
    for (int j = 0; j < 8; j++)
        if (v[j] > best) {
            best = v[j];
            idx = c0 + threadIdx.x + 1024u * j;
        }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = idx;
    __syncthreads();
    for (uint32_t step = 512; step > 0; step >>= 1) {
        if (threadIdx.x < step) {
            float ov = sv[threadIdx.x + step];
            uint32_t oi = si[threadIdx.x + step];
            if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi < si[threadIdx.x])) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        cand_val[(size_t)blockIdx.y * spans + blockIdx.x] = sv[0];
        cand_idx[(size_t)blockIdx.y * spans + blockIdx.x] = si[0];
    }
}

__global__ __launch_bounds__(256) void k_argmax_merge(const float *__restrict__ cand_val, const uint32_t *__restrict__ cand_idx,
                                                       uint32_t spans, int *__restrict__ out)
{
    __shared__ float sv[256];
    __shared__ uint32_t si[256];
    float best = -1e30f;
    uint32_t idx = 0xFFFFFFFFu;
    for (uint32_t s = threadIdx.x; s < spans; s += 256u) {  // candidates of later spans have larger indices
        float v = cand_val[(size_t)blockIdx.x * spans + s];
        uint32_t i = cand_idx[(size_t)blockIdx.x * spans + s];
        if (v > best || (v == best && i < idx)) {
            best = v;
            idx = i;
        }
    }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = idx;
    __syncthreads();
    for (uint32_t step = 128; step > 0; step >>= 1) {
        if (threadIdx.x < step) {
            float ov = sv[threadIdx.x + step];
            uint32_t oi = si[threadIdx.x + step];
            if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi < si[threadIdx.x])) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = si[0] == 0xFFFFFFFFu ? 0 : (int)si[0];
}

// `scratch` (scratch_bytes) holds the candidates of the two-phase form; without enough of it, or for short
// rows, one workgroup per row scans the whole row.
hipError_t launch_argmax(hipStream_t s, const float *in, uint32_t rows, uint32_t cols, int *out, void *scratch,
                         size_t scratch_bytes)
{
    if (rows == 0) return hipSuccess;
    uint32_t spans = (cols + kArgmaxSpan - 1) / kArgmaxSpan;
    if (spans >= 4 && rows <= 65535 && scratch && (size_t)rows * spans * 8 <= scratch_bytes) {
        float *cv = (float *)scratch;
        uint32_t *ci = (uint32_t *)(cv + (size_t)rows * spans);
        hipLaunchKernelGGL(k_argmax_partial, dim3(spans, rows), dim3(1024), 0, s, in, cols, spans, cv, ci);
        hipLaunchKernelGGL(k_argmax_merge, dim3(rows), dim3(256), 0, s, cv, ci, spans, out);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(k_argmax, dim3(rows), dim3(1024), 0, s, in, cols, out);
    return hipGetLastError();
}

hipError_t launch_split_qkv(hipStream_t s, const float *qkv, float *q, float *kk, float *v, uint32_t h, uint32_t kv,
                            uint32_t batch)
{
    size_t total = (size_t)batch * (h + 2 * kv);
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_split_qkv, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, qkv, q, kk, v, h, kv, batch);
    return hipGetLastError();
}

hipError_t launch_split_gate_up(hipStream_t s, const float *gu, float *g, float *u, uint32_t ffn, uint32_t batch)
{
    size_t total = (size_t)batch * 2 * ffn;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_split_gate_up, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gu, g, u, ffn, batch);
    return hipGetLastError();
}

hipError_t launch_silu_mul(hipStream_t s, const float *gate, const float *up, float *out, size_t count)
{
    if (count == 0) return hipSuccess;
    hipLaunchKernelGGL(k_silu_mul, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, gate, up, out, count);
    return hipGetLastError();
}

hipError_t launch_swiglu_rows(hipStream_t s, const float *gu, float *out, uint32_t ffn, uint32_t batch, bool paired)
{
    size_t total = (size_t)batch * ffn;
    if (total == 0) return hipSuccess;
    dim3 grid((unsigned)((total + 255) / 256));
    if (paired) hipLaunchKernelGGL(k_swiglu_rows<true>, grid, dim3(256), 0, s, gu, out, ffn, batch);
    else hipLaunchKernelGGL(k_swiglu_rows<false>, grid, dim3(256), 0, s, gu, out, ffn, batch);
    return hipGetLastError();
}

hipError_t launch_pair_gate_up(hipStream_t s, const uint8_t *gate_packed, const uint16_t *gate_scales,
                               const uint8_t *up_packed, const uint16_t *up_scales, uint32_t groups, uint32_t ffn,
                               uint8_t *packed_out, uint16_t *scales_out)
{
    size_t total = (size_t)groups * 2 * ffn;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_pair_gate_up, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       (const uint4v *)gate_packed, gate_scales, (const uint4v *)up_packed, up_scales, groups, ffn,
                       (uint4v *)packed_out, scales_out);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// GEMV on the reference layout, f32 activations (no repack, exact f32 products).
// One lane per output column: a wave reads 64 x 16 B = 1 KiB contiguous per group.
// The activation index is wave-uniform, so A comes in through scalar loads.
// ---------------------------------------------------------------------------------
// ALIGN16: the records are 16-byte aligned (one 128-bit load); otherwise four 32-bit loads, the alignment the
// reference's own kernel needs (quantize.rs:1227-1228).
template <bool ATOMIC, bool ALIGN16>
__global__ __launch_bounds__(256) void k_ref_gemv(float *__restrict__ c, const float *__restrict__ a,
                                                   const uint32_t *__restrict__ packed,
                                                   const uint16_t *__restrict__ scales, uint32_t n, uint32_t groups,
                                                   uint32_t gps)
{
    uint32_t col = blockIdx.x * 256 + threadIdx.x;
    if (col >= n) return;
    uint32_t g0 = blockIdx.y * gps;
    uint32_t g1 = g0 + gps < groups ? g0 + gps : groups;
    float dot = 0.0f;
    for (uint32_t g = g0; g < g1; g++) {
        float s = f16_bits_to_f32(scales[(size_t)g * n + col]);
        const uint32_t *rec = packed + ((size_t)g * n + col) * 4u;
        uint4v v;
        if (ALIGN16) v = *(const uint4v *)rec;
        else v = uint4v{rec[0], rec[1], rec[2], rec[3]};
        const float *ab = a + g * 32;
        float gdot = 0.0f;
#pragma unroll
        for (int wi = 0; wi < 4; wi++) {
            uint32_t w = v[wi];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                int q = (int)((w >> (4 * j)) & 0xFu) - 8;
                gdot = fmaf(ab[wi * 8 + j], (float)q, gdot);
            }
        }
        dot = fmaf(gdot, s, dot);
    }
    if (ATOMIC) atomicAdd(&c[col], dot);
    else c[col] = dot;
}

hipError_t launch_ref_gemv(hipStream_t s, const float *a, const uint8_t *packed, const uint16_t *scales, float *c,
                           uint32_t n, uint32_t k, uint32_t splits, uint32_t groups_per_split)
{
    if (n == 0) return hipSuccess;
    dim3 grid((n + 255) / 256, splits);
    const bool align16 = ((uintptr_t)packed & 15) == 0;
    if (splits > 1) {
        hipError_t e = launch_fill_zero(s, c, (size_t)n * 4);
        if (e != hipSuccess) return e;
    }
#define TWM_REF_GEMV(AT, AL) \
    hipLaunchKernelGGL((k_ref_gemv<AT, AL>), grid, dim3(256), 0, s, c, a, (const uint32_t *)packed, scales, n, k / 32, groups_per_split)
    if (splits > 1) {
        if (align16) TWM_REF_GEMV(true, true);
        else TWM_REF_GEMV(true, false);
    } else {
        if (align16) TWM_REF_GEMV(false, true);
        else TWM_REF_GEMV(false, false);
    }
#undef TWM_REF_GEMV
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// repack: reference layout -> wave tile order (see twm_internal.h)
// ---------------------------------------------------------------------------------
// bit position 4*p of the result holds the nibble of k-offset j, p = j/2 for even j, 4 + j/2 for odd j
__device__ __forceinline__ uint32_t permute_word(uint32_t w)
{
    uint32_t r = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        int p = (j & 1) ? 4 + (j >> 1) : (j >> 1);
        r |= ((w >> (4 * j)) & 0xFu) << (4 * p);
    }
    return r;
}

__global__ __launch_bounds__(256) void k_repack_q(const uint32_t *__restrict__ packed, uint32_t groups, uint32_t n,
                                                   uint32_t n_tiles, uint32_t k_chunks, uint4v *__restrict__ qw)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // (kc * n_tiles + nt) * 64 + lane
    if (idx >= (size_t)n_tiles * k_chunks * 64) return;
    uint32_t lane = (uint32_t)(idx & 63);
    size_t tile = idx >> 6;
    uint32_t nt = (uint32_t)(tile % n_tiles), kc = (uint32_t)(tile / n_tiles);
    uint32_t col = nt * 16 + (lane & 15), kb = lane >> 4;
    uint4v o;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t g = kc * 4 + i;
        uint32_t w = 0x88888888u;
        if (g < groups && col < n) w = packed[((size_t)g * n + col) * 4 + kb];
        o[i] = permute_word(w);
    }
    qw[idx] = o;
}

__global__ __launch_bounds__(256) void k_repack_s(const uint16_t *__restrict__ scales, uint32_t groups, uint32_t n,
                                                   uint32_t n_tiles, uint32_t k_chunks, uint2v *__restrict__ sc)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // (kc * n_tiles + nt) * 16 + c
    if (idx >= (size_t)n_tiles * k_chunks * 16) return;
    uint32_t c = (uint32_t)(idx & 15);
    size_t tile = idx >> 4;
    uint32_t nt = (uint32_t)(tile % n_tiles), kc = (uint32_t)(tile / n_tiles);
    uint32_t col = nt * 16 + c;
    uint32_t h[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t g = kc * 4 + i;
        h[i] = (g < groups && col < n) ? scales[(size_t)g * n + col] : 0u;
    }
    uint2v o = {h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
    sc[idx] = o;
}

hipError_t launch_repack(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n, void *qw,
                         void *sc, uint32_t n_tiles, uint32_t k_chunks)
{
    size_t tq = (size_t)n_tiles * k_chunks * 64, ts = (size_t)n_tiles * k_chunks * 16;
    if (tq == 0) return hipSuccess;
    hipLaunchKernelGGL(k_repack_q, dim3((unsigned)((tq + 255) / 256)), dim3(256), 0, s, (const uint32_t *)packed, k / 32,
                       n, n_tiles, k_chunks, (uint4v *)qw);
    hipLaunchKernelGGL(k_repack_s, dim3((unsigned)((ts + 255) / 256)), dim3(256), 0, s, scales, k / 32, n, n_tiles,
                       k_chunks, (uint2v *)sc);
    return hipGetLastError();
}

// Q4 unpack straight from the wave tile order (used to prove the repack lossless).
__global__ __launch_bounds__(256) void k_weight_dequant_f16(const uint32_t *__restrict__ qw,
                                                             const uint16_t *__restrict__ sc, uint32_t k, uint32_t n,
                                                             uint32_t n_tiles, uint16_t *__restrict__ out)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // row * n + col
    if (idx >= (size_t)k * n) return;
    uint32_t row = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
    uint32_t g = row / 32, e = row % 32;
    uint32_t nt = col / 16, c = col % 16, kc = g / 4, i = g % 4, kb = e / 8, j = e % 8;
    size_t tile = (size_t)kc * n_tiles + nt;
    uint32_t w = qw[(tile * 64 + kb * 16 + c) * 4 + i];
    int p = (j & 1) ? 4 + (j >> 1) : (j >> 1);
    int q = (int)((w >> (4 * p)) & 0xFu) - 8;
    out[idx] = f32_to_f16_bits(scale_times_q(sc[(tile * 16 + c) * 4 + i], q));
}

hipError_t launch_weight_dequant_f16(hipStream_t s, const WeightView &w, uint16_t *out_kn)
{
    size_t total = (size_t)w.k * w.n;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_weight_dequant_f16, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       (const uint32_t *)w.qw, (const uint16_t *)w.sc, w.k, w.n, w.n_tiles, out_kn);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// column-lane copy (layout in twm_gemv4.hip): 4608-byte blocks [tile64][k_chunk], each
// [4 groups][64 columns][16 B nibbles, permuted inside each word] + [64 columns][4 f16 scales]
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_repack_col(const uint4v *__restrict__ packed, const uint16_t *__restrict__ scales,
                                                     uint32_t groups, uint32_t n, uint32_t k_chunks, uint32_t tiles64,
                                                     char *__restrict__ cw, uint32_t pair_ffn)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // ((tile * k_chunks + kc) * 4 + g) * 64 + lane
    if (idx >= (size_t)tiles64 * k_chunks * 256) return;
    uint32_t lane = (uint32_t)(idx & 63), gi = (uint32_t)((idx >> 6) & 3);
    size_t blk = idx >> 8;
    uint32_t kc = (uint32_t)(blk % k_chunks), tile = (uint32_t)(blk / k_chunks);
    uint32_t g = kc * 4 + gi, col = tile * 64 + lane;
    uint4v w = {0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u};
    uint32_t sbits = 0;
    if (g < groups && col < n) {
        // pair_ffn != 0: the source is [gate | up] (n = 2 * pair_ffn) and the copy takes the paired order
        uint32_t src = pair_ffn ? (col >> 6) * kPairWidth + (col & 31u) + ((col & kPairWidth) ? pair_ffn : 0u) : col;
        w = packed[(size_t)g * n + src];
        sbits = scales[(size_t)g * n + src];
    }
    uint4v o = {permute_word(w[0]), permute_word(w[1]), permute_word(w[2]), permute_word(w[3])};
    char *base = cw + blk * kColBlockBytes;
    *(uint4v *)(base + gi * 1024u + lane * 16u) = o;
    *(uint16_t *)(base + 4096u + lane * 8u + gi * 2u) = (uint16_t)sbits;
}

hipError_t launch_repack_col(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                             void *cq, uint32_t n_pad, uint32_t k_chunks, uint32_t pair_ffn)
{
    size_t total = (size_t)(n_pad / 64) * k_chunks * 256;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_repack_col, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (const uint4v *)packed,
                       scales, k / 32, n, k_chunks, n_pad / 64, (char *)cq, pair_ffn);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void k_weight_dequant_f16_col(const char *__restrict__ cw, uint32_t k, uint32_t n,
                                                                 uint32_t k_chunks, uint16_t *__restrict__ out)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // row * n + col
    if (idx >= (size_t)k * n) return;
    uint32_t row = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
    uint32_t g = row / 32, e = row % 32, j = e % 8;
    const char *base = cw + ((size_t)(col / 64) * k_chunks + g / 4) * kColBlockBytes;
    uint32_t lane = col % 64, gi = g % 4;
    uint32_t w = *(const uint32_t *)(base + gi * 1024u + lane * 16u + (e / 8) * 4u);
    int p = (j & 1) ? 4 + (j >> 1) : (j >> 1);
    int q = (int)((w >> (4 * p)) & 0xFu) - 8;
    uint16_t sbits = *(const uint16_t *)(base + 4096u + lane * 8u + gi * 2u);
    out[idx] = f32_to_f16_bits(scale_times_q(sbits, q));
}

hipError_t launch_weight_dequant_f16_col(hipStream_t s, const WeightView &w, uint16_t *out_kn)
{
    size_t total = (size_t)w.k * w.n;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_weight_dequant_f16_col, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       (const char *)w.cq, w.k, w.n, w.k_chunks, out_kn);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// One repacked copy from the other.  Both hold every 32-bit word of the reference's records with the same nibble
// permutation, so the conversion moves words: word kb of column c's record of group g is
//   tile copy:        qw[(kc * n_tiles + c / 16) * 64 + kb * 16 + c % 16][g % 4]
//   column-lane copy: block (c / 64, kc), group row g % 4, lane c % 64, word kb
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_col_to_tile(const char *__restrict__ cw, uint32_t n_tiles, uint32_t k_chunks,
                                                      uint4v *__restrict__ qw, uint2v *__restrict__ sc)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // (kc * n_tiles + nt) * 64 + lane
    if (idx >= (size_t)n_tiles * k_chunks * 64) return;
    const uint32_t lane = (uint32_t)(idx & 63), c = lane & 15, kb = lane >> 4;
    const size_t tile = idx >> 6;
    const uint32_t nt = (uint32_t)(tile % n_tiles), kc = (uint32_t)(tile / n_tiles);
    const char *blk = cw + ((size_t)(nt / 4) * k_chunks + kc) * kColBlockBytes;
    const uint32_t col = (nt % 4) * 16 + c;
    uint4v o;
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = *(const uint32_t *)(blk + i * 1024u + col * 16u + kb * 4u);
    qw[idx] = o;
    if (kb == 0) sc[tile * 16 + c] = *(const uint2v *)(blk + 4096u + col * 8u);
}

__global__ __launch_bounds__(256) void k_tile_to_col(const uint32_t *__restrict__ qw, const uint2v *__restrict__ sc,
                                                      uint32_t n_tiles, uint32_t k_chunks, char *__restrict__ cw)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // ((tile64 * k_chunks + kc) * 4 + g) * 64 + lane
    if (idx >= (size_t)(n_tiles / 4) * k_chunks * 256) return;
    const uint32_t lane = (uint32_t)(idx & 63), gi = (uint32_t)((idx >> 6) & 3);
    const size_t blk = idx >> 8;
    const uint32_t kc = (uint32_t)(blk % k_chunks), tile64 = (uint32_t)(blk / k_chunks);
    const size_t tile = (size_t)kc * n_tiles + tile64 * 4 + lane / 16;
    uint4v o;
#pragma unroll
    for (int kb = 0; kb < 4; kb++) o[kb] = qw[(tile * 64 + kb * 16 + lane % 16) * 4 + gi];
    char *base = cw + blk * kColBlockBytes;
    *(uint4v *)(base + gi * 1024u + lane * 16u) = o;
    if (gi == 0) *(uint2v *)(base + 4096u + lane * 8u) = sc[tile * 16 + lane % 16];
}

hipError_t launch_col_to_tile(hipStream_t s, const void *cq, uint32_t n_tiles, uint32_t k_chunks, void *qw, void *sc)
{
    size_t total = (size_t)n_tiles * k_chunks * 64;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_col_to_tile, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (const char *)cq, n_tiles,
                       k_chunks, (uint4v *)qw, (uint2v *)sc);
    return hipGetLastError();
}

hipError_t launch_tile_to_col(hipStream_t s, const void *qw, const void *sc, uint32_t n_tiles, uint32_t k_chunks, void *cq)
{
    size_t total = (size_t)(n_tiles / 4) * k_chunks * 256;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_tile_to_col, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (const uint32_t *)qw,
                       (const uint2v *)sc, n_tiles, k_chunks, (char *)cq);
    return hipGetLastError();
}

}  // namespace twm

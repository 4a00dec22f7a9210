// gfx950 (CDNA4, wave64) kernels for the TW-Marlin W4A16 quantized-linear path.
//
// Reference semantics (crates/kernels/src/quantize.rs in the reference checkout):
//   GEMV arithmetic ............ :1186-1298   (warp_gemm_tw_marlin_m1[_direct])
//   Q4 unpack to FP16 .......... :534-571     (warp_dequant_q4_to_f16)
//   quantizer .................. :414-474, crates/loader/src/gemma_moe_q4.rs:218-254
//   reorder / fuse ............. :912-956, :1018-1063
//   split_qkv / split_gate_up .. crates/kernels/src/ops.rs:2255-2297
// Nothing here is translated from those kernels: the decode kernels stream weights
// repacked into a wave64 tile order, dequantise in registers with packed-f16 integer
// tricks and contract on the 16x16x32 f16 MFMA with f32 accumulation.
#include "twm_internal.h"

namespace twm {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));

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

// ---------------------------------------------------------------------------------
// GEMV on the reference layout, f32 activations (no repack, exact f32 products).
// One lane per output column: a wave reads 64 x 16 B = 1 KiB contiguous per group.
// The activation index is wave-uniform, so A comes in through scalar loads.
// ---------------------------------------------------------------------------------
template <bool ATOMIC>
__global__ __launch_bounds__(256) void k_ref_gemv(float *__restrict__ c, const float *__restrict__ a,
                                                   const uint4v *__restrict__ packed,
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
        uint4v v = packed[(size_t)g * n + col];
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
    if (splits > 1) {
        hipError_t e = launch_fill_zero(s, c, (size_t)n * 4);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(k_ref_gemv<true>, grid, dim3(256), 0, s, c, a, (const uint4v *)packed, scales, n, k / 32,
                           groups_per_split);
    } else {
        hipLaunchKernelGGL(k_ref_gemv<false>, grid, dim3(256), 0, s, c, a, (const uint4v *)packed, scales, n, k / 32,
                           groups_per_split);
    }
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
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // (nt * k_chunks + kc) * 64 + lane
    if (idx >= (size_t)n_tiles * k_chunks * 64) return;
    uint32_t lane = (uint32_t)(idx & 63);
    size_t tile = idx >> 6;
    uint32_t kc = (uint32_t)(tile % k_chunks), nt = (uint32_t)(tile / k_chunks);
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
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // (nt * k_chunks + kc) * 16 + c
    if (idx >= (size_t)n_tiles * k_chunks * 16) return;
    uint32_t c = (uint32_t)(idx & 15);
    size_t tile = idx >> 4;
    uint32_t kc = (uint32_t)(tile % k_chunks), nt = (uint32_t)(tile / k_chunks);
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
                                                             uint32_t k_chunks, uint16_t *__restrict__ out)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // row * n + col
    if (idx >= (size_t)k * n) return;
    uint32_t row = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
    uint32_t g = row / 32, e = row % 32;
    uint32_t nt = col / 16, c = col % 16, kc = g / 4, i = g % 4, kb = e / 8, j = e % 8;
    size_t tile = (size_t)nt * k_chunks + kc;
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
                       (const uint32_t *)w.qw, (const uint16_t *)w.sc, w.k, w.n, w.k_chunks, out_kn);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// decode kernel, M = 1..32
// ---------------------------------------------------------------------------------
// One u32 of the tile order -> eight f16 values (q - 8), exact.
//   (w & 0x000F000F) | 0x6400 6400 : two halves 1024 + q       (nibbles at bits 0..3)
//   (w & 0x00F000F0) | 0x5400 5400 : two halves   64 + q       (nibbles at bits 4..7)
// then a packed subtract of 1032 / 72.  Thanks to the nibble permutation done at repack the
// four resulting registers hold k-offsets (0,1) (2,3) (4,5) (6,7): the MFMA B-operand order.
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t magic)
{
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(magic));
    return r;
}

__device__ __forceinline__ half8 dequant_word(uint32_t w, uint32_t magic_lo, uint32_t magic_hi)
{
    union { uint32_t u[4]; half2v h2[4]; half8 h; } r;
    uint32_t w8 = w >> 8;
    r.u[0] = and_or(w, 0x000F000Fu, magic_lo);
    r.u[1] = and_or(w, 0x00F000F0u, magic_hi);
    r.u[2] = and_or(w8, 0x000F000Fu, magic_lo);
    r.u[3] = and_or(w8, 0x00F000F0u, magic_hi);
    const half2v b_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
    const half2v b_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    r.h2[0] += b_lo;
    r.h2[1] += b_hi;
    r.h2[2] += b_lo;
    r.h2[3] += b_hi;
    return r.h;
}

__device__ __forceinline__ void store_out(const OutSpec &out, uint32_t m, uint32_t col, float v)
{
#pragma unroll
    for (uint32_t s = 0; s < kMaxSegs; s++) {
        if (s < out.count) {
            uint32_t rel = col - out.seg[s].start;
            if (rel < out.seg[s].width) out.seg[s].ptr[(size_t)m * out.seg[s].width + rel] = v;
        }
    }
}

// Workgroup = 4 waves. It owns NT n-tiles (16*NT columns) and the k-chunks
// [split*cps, (split+1)*cps) of them; wave w takes chunks w, w+4, ... of that range, the four
// partial tiles are summed through LDS, and, when the launch is split along K, the workgroup
// parks its tile in `ws` and the last workgroup to arrive for the tile adds the `splits`
// partials in ascending order (deterministic) and stores the result.
//   MT : 16-row blocks of A (1 for M <= 16, 2 for M <= 32)
//   RL : accumulator registers that can hold live rows (M for M < 4, else 4)
// Block ids are dealt round-robin to the 8 XCDs; the id is unfolded so that every split of a
// tile lands on the same XCD and the partials stay in that XCD's L2.
template <int NT, int MT, int RL, bool AF32>
__global__ __launch_bounds__(256) void k_decode(const uint4v *__restrict__ qw, const uint2v *__restrict__ sc,
                                                 const void *__restrict__ a_any, OutSpec out, float *__restrict__ ws,
                                                 unsigned *__restrict__ counters, uint32_t m_rows, uint32_t k,
                                                 uint32_t n, uint32_t k_chunks, uint32_t tile_groups, uint32_t splits,
                                                 uint32_t cps)
{
    constexpr int IDX = NT * MT * 4;
    __shared__ float red[4][IDX][64];
    __shared__ int s_last;

    const uint32_t b = blockIdx.x;
    const uint32_t xcd = b & 7u, jj = b >> 3;
    const uint32_t sp = jj % splits;
    const uint32_t tg = (jj / splits) * 8u + xcd;
    if (tg >= tile_groups) return;  // whole workgroup leaves together

    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const uint32_t c = lane & 15u, kb = lane >> 4;
    const uint32_t nt0 = tg * NT;
    const uint32_t kc0 = sp * cps;
    const uint32_t kc1 = (kc0 + cps < k_chunks) ? kc0 + cps : k_chunks;

    uint32_t magic_lo = 0x64006400u, magic_hi = 0x54005400u;
    asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));  // keep the two constants in VGPRs

    float4v acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[t][mt] = float4v{0.f, 0.f, 0.f, 0.f};

    for (uint32_t kc = kc0 + wave; kc < kc1; kc += 4) {
        uint4v wq[NT];
        uint2v ws4[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            size_t tile = (size_t)(nt0 + t) * k_chunks + kc;
            wq[t] = qw[tile * 64 + lane];
            ws4[t] = sc[tile * 16 + c];
        }
        half8 af[4][MT];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t k0 = kc * 128u + i * 32u + kb * 8u;
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                uint32_t row = mt * 16 + c;
                half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
                if (row < m_rows && k0 < k) {
                    if (AF32) {
                        const float4 *p = (const float4 *)((const float *)a_any + (size_t)row * k + k0);
                        float4 x = p[0], y = p[1];
                        v = half8{(_Float16)x.x, (_Float16)x.y, (_Float16)x.z, (_Float16)x.w,
                                  (_Float16)y.x, (_Float16)y.y, (_Float16)y.z, (_Float16)y.w};
                    } else {
                        v = *(const half8 *)((const _Float16 *)a_any + (size_t)row * k + k0);
                    }
                }
                af[i][mt] = v;
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            union { uint2v u; _Float16 h[4]; } sv;
            sv.u = ws4[t];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                half8 bfrag = dequant_word(wq[t][i], magic_lo, magic_hi);
                float s = (float)sv.h[i];
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    float4v d = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i][mt], bfrag, float4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < RL; r++) acc[t][mt][r] = fmaf(d[r], s, acc[t][mt][r]);
                }
            }
        }
    }

    // ---- sum the four waves through LDS ----
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int r = 0; r < RL; r++) red[wave][(t * MT + mt) * 4 + r][lane] = acc[t][mt][r];
    __syncthreads();

    const uint32_t n_ld = ((n + kNPadTo - 1) / kNPadTo) * kNPadTo;  // row stride of the split-K scratch

    float val[NT * MT];
    bool live[NT * MT];
    uint32_t om[NT * MT], on[NT * MT];
#pragma unroll
    for (int x = 0; x < NT * MT; x++) {
        uint32_t idx = wave + 4 * x;        // this thread's entries: idx = (t*MT+mt)*4 + r, lane = lane
        uint32_t r = idx & 3u, tm = idx >> 2;
        uint32_t mt = tm % MT, t = tm / MT;
        om[x] = mt * 16 + kb * 4 + r;
        on[x] = (nt0 + t) * 16 + c;
        live[x] = (r < (uint32_t)RL) && om[x] < m_rows && on[x] < n;
        float v = 0.f;
        if (live[x]) v = (red[0][idx][lane] + red[1][idx][lane]) + (red[2][idx][lane] + red[3][idx][lane]);
        val[x] = v;
    }

    if (splits == 1) {
#pragma unroll
        for (int x = 0; x < NT * MT; x++)
            if (live[x]) store_out(out, om[x], on[x], val[x]);
        return;
    }

    // ---- cross-workgroup split-K: park the partial, last arrival reduces ----
#pragma unroll
    for (int x = 0; x < NT * MT; x++)
        if (live[x]) ws[((size_t)sp * m_rows + om[x]) * n_ld + on[x]] = val[x];
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned prev = atomicAdd(&counters[tg], 1u);
        s_last = (prev == splits - 1);
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
#pragma unroll
    for (int x = 0; x < NT * MT; x++) {
        if (live[x]) {
            float v = 0.f;
            for (uint32_t s = 0; s < splits; s++)
                v += __builtin_nontemporal_load(&ws[((size_t)s * m_rows + om[x]) * n_ld + on[x]]);
            store_out(out, om[x], on[x], v);
        }
    }
    if (threadIdx.x == 0) counters[tg] = 0u;  // ready for the next launch
}

template <int NT, int MT, int RL>
static hipError_t launch_decode_t(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m,
                                  const OutSpec &out, float *ws, unsigned *counters, uint32_t splits)
{
    uint32_t tile_groups = w.n_tiles / NT;
    uint32_t cps = (w.k_chunks + splits - 1) / splits;
    uint32_t blocks = ((tile_groups + 7) / 8) * 8 * splits;
    if (a_f32)
        hipLaunchKernelGGL((k_decode<NT, MT, RL, true>), dim3(blocks), dim3(256), 0, s, (const uint4v *)w.qw,
                           (const uint2v *)w.sc, a, out, ws, counters, m, w.k, w.n, w.k_chunks, tile_groups, splits, cps);
    else
        hipLaunchKernelGGL((k_decode<NT, MT, RL, false>), dim3(blocks), dim3(256), 0, s, (const uint4v *)w.qw,
                           (const uint2v *)w.sc, a, out, ws, counters, m, w.k, w.n, w.k_chunks, tile_groups, splits, cps);
    return hipGetLastError();
}

template <int NT>
static hipError_t launch_decode_nt(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m,
                                   const OutSpec &out, float *ws, unsigned *counters, uint32_t splits)
{
    if (m == 1) return launch_decode_t<NT, 1, 1>(s, w, a, a_f32, m, out, ws, counters, splits);
    if (m == 2) return launch_decode_t<NT, 1, 2>(s, w, a, a_f32, m, out, ws, counters, splits);
    if (m <= 16) return launch_decode_t<NT, 1, 4>(s, w, a, a_f32, m, out, ws, counters, splits);
    return launch_decode_t<NT, 2, 4>(s, w, a, a_f32, m, out, ws, counters, splits);
}

hipError_t launch_decode(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                         float *ws, unsigned *counters, DecodePlan plan)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    switch (plan.nt) {
    case 1: return launch_decode_nt<1>(s, w, a, a_f32, m, out, ws, counters, plan.splits);
    case 2: return launch_decode_nt<2>(s, w, a, a_f32, m, out, ws, counters, plan.splits);
    case 4: return launch_decode_nt<4>(s, w, a, a_f32, m, out, ws, counters, plan.splits);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace twm

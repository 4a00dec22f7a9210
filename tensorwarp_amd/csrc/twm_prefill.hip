// Prefill kernel (M > 16): C[M,N] = A[M,K] * dequant(W), FP16 MFMA with FP32 accumulation.
//
// Semantics: gemm_q4_0 (crates/kernels/src/quantize.rs:1825-1858 / kernel :186-246 in the reference),
// i.e. C[m][n] = sum_k A[m][k] * w[k][n].  Here w is the reference's Q4 unpack to FP16,
// f16_rne(f32(scale) * (q - 8)) (quantize.rs:534-571), produced in registers: (q - 8) is exact in f16 and
// one packed f16 multiply by the scale rounds exactly like the reference's __float2half(scale * q).
//
// Block = 128 rows x 256 columns, 4 waves; wave w owns 64 columns (four 16-column tiles of the tile-order
// copy) for all 128 rows, so no weight is unpacked twice inside a block.  Per 128-deep k-chunk:
//   A tile (128 x 128 f16) : global -> registers -> LDS, double buffered, row stride 272 B so that the
//                            sixteen rows of a 16-byte-per-lane operand read hit distinct banks;
//   B : 16 bytes of nibbles + four scales per lane per tile, straight from HBM into registers (prefetched
//       one chunk ahead), unpacked to MFMA B operands;
//   128 v_mfma_f32_16x16x32_f16 per wave (8 row blocks x 4 column tiles x 4 groups), 128 accumulator
//   registers per lane.
#include "twm_device.h"

namespace twm {

constexpr int kPfBM = 128;
constexpr int kPfRowStride = 136;  // halves per LDS row: 128 + 8 (272 bytes)
constexpr int kPfTileHalves = kPfBM * kPfRowStride;

struct PfConsts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};

__device__ __forceinline__ PfConsts make_pf_consts()
{
    PfConsts c = {0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(c.mask_lo), "+s"(c.mask_hi), "+v"(c.magic_lo), "+v"(c.magic_hi));
    return c;
}

// eight nibbles -> eight FP16 weights f16(scale * (q - 8)); `s2` holds the scale in both halves
__device__ __forceinline__ half8 pf_dequant_word(uint32_t w, half2v s2, const PfConsts &c)
{
    union { uint32_t u[4]; half2v h2[4]; half8 h; } r;
    uint32_t w8 = w >> 8;
    r.u[0] = (w & c.mask_lo) | c.magic_lo;
    r.u[1] = (w & c.mask_hi) | c.magic_hi;
    r.u[2] = (w8 & c.mask_lo) | c.magic_lo;
    r.u[3] = (w8 & c.mask_hi) | c.magic_hi;
    const half2v b_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
    const half2v b_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    r.h2[0] = (r.h2[0] + b_lo) * s2;
    r.h2[1] = (r.h2[1] + b_hi) * s2;
    r.h2[2] = (r.h2[2] + b_lo) * s2;
    r.h2[3] = (r.h2[3] + b_hi) * s2;
    return r.h;
}

__device__ __forceinline__ void pf_store_out(const OutSpec &out, uint32_t m, uint32_t col, float v)
{
#pragma unroll
    for (uint32_t s = 0; s < kMaxSegs; s++) {
        if (s < out.count) {
            uint32_t rel = col - out.seg[s].start;
            if (rel < out.seg[s].width) out.seg[s].ptr[(size_t)m * out.seg[s].width + rel] = v;
        }
    }
}

template <bool AF32>
__global__ __launch_bounds__(256) void k_prefill(const uint4v *__restrict__ qw, const uint2v *__restrict__ sc,
                                                  const void *__restrict__ a_any, OutSpec out, uint32_t m_rows,
                                                  uint32_t k, uint32_t n, uint32_t n_tiles, uint32_t k_chunks)
{
    extern __shared__ _Float16 a_lds[];  // two tiles of kPfTileHalves

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t c = lane & 15u, kb = lane >> 4;
    const uint32_t m0 = blockIdx.y * kPfBM;
    const uint32_t nt0 = (blockIdx.x * 4u + wave) * 4u;  // first of this wave's four 16-column tiles

    const PfConsts dq = make_pf_consts();

    // this wave's tiles; tiles past the end replay the last tile and are never stored
    uint32_t nt[4];
#pragma unroll
    for (int t = 0; t < 4; t++) nt[t] = nt0 + t < n_tiles ? nt0 + t : n_tiles - 1;

    float4v acc[8][4];
#pragma unroll
    for (int mt = 0; mt < 8; mt++)
#pragma unroll
        for (int t = 0; t < 4; t++) acc[mt][t] = float4v{0.f, 0.f, 0.f, 0.f};

    // ---- A staging: thread handles eight 16-byte vectors: idx = tid + 256*j, row = idx/16, vec = idx%16 ----
    uint4v a_stage[8];
    auto load_a = [&](uint32_t kc) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t idx = threadIdx.x + 256u * j;
            uint32_t row = m0 + (idx >> 4), kk = kc * 128u + (idx & 15u) * 8u;
            uint4v v = {0u, 0u, 0u, 0u};
            if (row < m_rows && kk < k) {
                if (AF32) {
                    const float4 *p = (const float4 *)((const float *)a_any + (size_t)row * k + kk);
                    float4 x = p[0], y = p[1];
                    union { half8 h; uint4v u; } cv;
                    cv.h = half8{(_Float16)x.x, (_Float16)x.y, (_Float16)x.z, (_Float16)x.w,
                                 (_Float16)y.x, (_Float16)y.y, (_Float16)y.z, (_Float16)y.w};
                    v = cv.u;
                } else {
                    v = *(const uint4v *)((const _Float16 *)a_any + (size_t)row * k + kk);
                }
            }
            a_stage[j] = v;
        }
    };
    auto store_a = [&](uint32_t buf) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t idx = threadIdx.x + 256u * j;
            *(uint4v *)(a_lds + buf * kPfTileHalves + (idx >> 4) * kPfRowStride + (idx & 15u) * 8u) = a_stage[j];
        }
    };

    uint4v bq[2][4];
    uint2v bs[2][4];
    auto load_b = [&](int slot, uint32_t kc) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            size_t tile = (size_t)kc * n_tiles + nt[t];
            bq[slot][t] = qw[tile * 64 + lane];
            bs[slot][t] = sc[tile * 16 + c];
        }
    };

    auto compute = [&](int slot, uint32_t buf) {
        const _Float16 *ap = a_lds + buf * kPfTileHalves + c * kPfRowStride + kb * 8u;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            half8 bf[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                uint32_t pair = bs[slot][t][g >> 1];
                uint32_t s16 = (g & 1) ? (pair >> 16) : (pair & 0xFFFFu);
                union { uint32_t u; half2v h; } s2;
                s2.u = s16 | (s16 << 16);
                bf[t] = pf_dequant_word(bq[slot][t][g], s2.h, dq);
            }
#pragma unroll
            for (int mt = 0; mt < 8; mt++) {
                half8 af = *(const half8 *)(ap + mt * 16 * kPfRowStride + g * 32);
#pragma unroll
                for (int t = 0; t < 4; t++)
                    acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, bf[t], acc[mt][t], 0, 0, 0);
            }
        }
    };

    // ---- pipeline over k-chunks ----
    load_a(0);
    load_b(0, 0);
    store_a(0);
    __syncthreads();
    for (uint32_t kc = 0; kc < k_chunks; kc += 2) {
        // even chunk: slot 0 / buffer 0
        if (kc + 1 < k_chunks) { load_a(kc + 1); load_b(1, kc + 1); }
        compute(0, 0);
        if (kc + 1 >= k_chunks) break;
        store_a(1);
        __syncthreads();
        // odd chunk: slot 1 / buffer 1
        if (kc + 2 < k_chunks) { load_a(kc + 2); load_b(0, kc + 2); }
        compute(1, 1);
        if (kc + 2 >= k_chunks) break;
        store_a(0);
        __syncthreads();
    }

    // ---- store: lane (c, kb) holds rows 4*kb + r of row block mt, column 16*tile + c ----
#pragma unroll
    for (int t = 0; t < 4; t++) {
        if (nt0 + t >= n_tiles) continue;
        uint32_t on = (nt0 + t) * 16u + c;
        if (on >= n) continue;
#pragma unroll
        for (int mt = 0; mt < 8; mt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                uint32_t om = m0 + mt * 16u + kb * 4u + r;
                if (om < m_rows) pf_store_out(out, om, on, acc[mt][t][r]);
            }
    }
}

hipError_t launch_prefill(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    static bool attr_set = false;
    size_t lds = (size_t)2 * kPfTileHalves * sizeof(_Float16);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void *)k_prefill<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void *)k_prefill<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    dim3 grid((w.n_tiles + 15) / 16, (m + kPfBM - 1) / kPfBM);
    if (a_f32)
        hipLaunchKernelGGL(k_prefill<true>, grid, dim3(256), lds, s, (const uint4v *)w.qw, (const uint2v *)w.sc, a, out, m,
                           w.k, w.n, w.n_tiles, w.k_chunks);
    else
        hipLaunchKernelGGL(k_prefill<false>, grid, dim3(256), lds, s, (const uint4v *)w.qw, (const uint2v *)w.sc, a, out, m,
                           w.k, w.n, w.n_tiles, w.k_chunks);
    return hipGetLastError();
}

}  // namespace twm

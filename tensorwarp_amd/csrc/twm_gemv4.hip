// Decode kernel for M <= 4 rows of activations: one lane per output column.
//
// C[m][n] = sum_g f32(scale[g][n]) * sum_{k in g} A[m][k] * (q[k][n] - 8), f32 accumulation (the
// arithmetic of warp_gemm_tw_marlin_m1, crates/kernels/src/quantize.rs:1186-1298 in the reference),
// on the "column-lane" copy of the weights: one 4608-byte block per (64-column tile, 128-deep chunk),
//   block(tile, kc) at ((tile * k_chunks + kc) * 4608) bytes:
//     [g = 0..3][lane = 0..63][16 B]   the 16-byte record of (group 4*kc+g, column 64*tile+lane),
//                                       nibbles permuted inside each 32-bit word as in twm_internal.h
//     [lane = 0..63][8 B]              the four f16 scales of that column for the chunk's groups
// so a chunk is one contiguous read and a tile's chunks follow each other: a workgroup streams one
// contiguous region (scales included) instead of touching every group row of the matrix.
// A wave owns 64 consecutive columns (lane = column) per tile.  The 32-term sum of a group is done by
// eight chained v_mfma_f32_4x4x4_16B_f16: the instruction holds 16 independent 4x4 blocks, block b =
// lanes 4b..4b+3 = four columns, and with CBSZ=4 every block takes its A matrix (4 rows x 4 k) from
// the block named by ABID.  So ONE 16-byte-per-lane load of activations per 128-deep chunk (lane l
// holds row l%4, k-piece l/4) feeds all 32 MFMAs of the chunk, the piece being chosen by the ABID
// immediate: no LDS, no per-MFMA operand traffic, and the output row m of column n is register m of
// lane n.  Per 1 KiB of nibbles the wave spends 36 VALU on the unpack, 8 MFMA and 1 scale-FMA.
#include "twm_gemv4_core.h"

#include <cstring>

namespace twm {

__device__ __forceinline__ void gemv4_store_out(const OutSpec &out, uint32_t m, uint32_t col, float v)
{
#pragma unroll
    for (uint32_t s = 0; s < kMaxSegs; s++) {
        if (s < out.count) {
            uint32_t rel = col - out.seg[s].start;
            if (rel < out.seg[s].width) out.seg[s].ptr[(size_t)m * out.seg[s].width + rel] = out.seg[s].bias ? v + out.seg[s].bias[rel] : v;
        }
    }
}

// Workgroup = `waves` waves (blockDim.x / 64) that share NT tiles of 64 columns and split the
// k-chunks [split*cps, (split+1)*cps) among themselves (wave w: chunks w, w + waves, ...).
// REFL: cw is the reference's packed array and ref_scales its scales (no repack; M = 1, f32 activations).
template <int NT, int RL, bool AF32, bool REFL = false>
__global__ __launch_bounds__(1024) void k_gemv4(const char *__restrict__ cw, const void *__restrict__ a_any,
                                                 uint32_t m_rows, uint32_t k, uint32_t n, uint32_t n_pad, uint32_t k_chunks,
                                                 uint32_t tile_groups, uint32_t splits, uint32_t cps,
                                                 const uint16_t *__restrict__ ref_scales, float *__restrict__ ws,
                                                 unsigned *__restrict__ counters, float *__restrict__ swiglu_out, OutSpec out)
{
    extern __shared__ float red[];  // [waves][NT][RL][64]
    __shared__ int s_last;

    const uint32_t b = blockIdx.x;
    const uint32_t xcd = b & 7u, jj = b >> 3;
    const uint32_t sp = jj % splits;
    const uint32_t tg = (jj / splits) * 8u + xcd;
    if (tg >= tile_groups) return;

    const uint32_t waves = blockDim.x >> 6;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t kc0 = sp * cps;
    const uint32_t kc1 = (kc0 + cps < k_chunks) ? kc0 + cps : k_chunks;
    // byte address of this lane's first record in block (tile tg*NT + t, chunk 0)
    const char *wbase[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) wbase[t] = cw + (size_t)(tg * NT + t) * k_chunks * kColBlockBytes;
    const uint32_t lane16 = lane * 16u, lane8 = 4096u + lane * 8u;

    const Gemv4Consts dq = make_gemv4_consts();

    // activations: lane l reads row min(l % 4, M-1), halves [kc*128 + 8*(l/4), +8); with row-packed f32 terms
    // row min((l % 4) / 2, M-1), odd lanes holding the residual term
    constexpr int TERMS = REFL ? kTermsRowPacked : gemv4_terms<AF32, RL>();
    uint32_t arow = TERMS == kTermsRowPacked ? (lane & 3u) >> 1 : lane & 3u;
    if (arow > m_rows - 1) arow = m_rows - 1;
    const bool lane_is_lo = TERMS == kTermsRowPacked && (lane & 1u) != 0;
    const uint32_t apiece = (lane >> 2) * 8u;

    float acc[NT][RL];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int r = 0; r < RL; r++) acc[t][r] = 0.f;

    constexpr int RG = (RL + 3) / 4;  // rows beyond four repeat the MFMA chain (f16 activations)
    auto load_chunk = [&](Chunk4<NT, RG> &r, uint32_t kc) {
        if constexpr (REFL)
            gemv4_load_chunk_ref<NT>(r, cw, ref_scales, tg * NT, kc, lane, n, k / 32u, (const float *)a_any, apiece, k,
                                     lane_is_lo);
        else
            gemv4_load_chunk<NT, AF32, TERMS, RG>(r, wbase, kc, lane16, lane8, a_any, arow, apiece, k, lane_is_lo, m_rows);
    };
    auto compute_chunk = [&](const Chunk4<NT, RG> &r) { gemv4_compute_chunk<NT, RL, TERMS>(r, dq, acc); };

    {
        // two register sets used alternately: the loads of one are in flight while the other is consumed
        Chunk4<NT, RG> r0, r1;
        uint32_t kc = kc0 + wave;
        if (kc < kc1) {
            load_chunk(r0, kc);
            while (true) {
                uint32_t kn = kc + waves;
                if (kn < kc1) load_chunk(r1, kn);
                compute_chunk(r0);
                if (kn >= kc1) break;
                kc = kn + waves;
                if (kc < kc1) load_chunk(r0, kc);
                compute_chunk(r1);
                if (kc >= kc1) break;
            }
        }
    }

    // ---- sum the waves' partial vectors through LDS: thread (wave 0.., lane) adds column `lane` ----
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int r = 0; r < RL; r++) red[((wave * NT + t) * RL + r) * 64 + lane] = acc[t][r];
    __syncthreads();

    const uint32_t threads = blockDim.x;
    const uint32_t entries = NT * RL * 64;  // entry e = (t*RL + r)*64 + lane
    // Paired gate_up weight: every 64-column tile holds 32 gate columns followed by the up columns of the
    // same 32 features, so the thread that sums lane ln < 32 also sums lane ln + 32 and writes silu(gate) * up.
    const bool swiglu = swiglu_out != nullptr;
    const uint32_t ffn = n >> 1;
    const uint32_t pair_entries = NT * RL * 32;  // entry e = (t*RL + r)*32 + ln
    if (splits == 1) {
        if (swiglu) {
            for (uint32_t e = threadIdx.x; e < pair_entries; e += threads) {
                uint32_t ln = e & 31u, tr = e >> 5, r = tr % RL, t = tr / RL;
                uint32_t feat = (tg * NT + t) * 32u + ln;
                if (r < m_rows && feat < ffn) {
                    float g = 0.f, u = 0.f;
                    for (uint32_t w = 0; w < waves; w++) {
                        g += red[(w * NT * RL + tr) * 64 + ln];
                        u += red[(w * NT * RL + tr) * 64 + 32 + ln];
                    }
                    swiglu_out[(size_t)r * ffn + feat] = gated_mul(out.gate_act, g, u);
                }
            }
            return;
        }
        for (uint32_t e = threadIdx.x; e < entries; e += threads) {
            uint32_t ln = e & 63u, tr = e >> 6, r = tr % RL, t = tr / RL;
            uint32_t on = (tg * NT + t) * 64u + ln;
            if (r < m_rows && on < n) {
                float v = 0.f;
                for (uint32_t w = 0; w < waves; w++) v += red[(w * NT * RL + tr) * 64 + ln];
                gemv4_store_out(out, r, on, v);
            }
        }
        return;
    }

    // cross-workgroup split-K: park the partial (agent-scope relaxed atomics: coherent across the XCDs'
    // L2s without a cache write-back), bump the arrival counter once the stores have completed; the
    // last workgroup to arrive adds the partials in ascending split order.
    for (uint32_t e = threadIdx.x; e < entries; e += threads) {
        uint32_t ln = e & 63u, tr = e >> 6, r = tr % RL, t = tr / RL;
        uint32_t on = (tg * NT + t) * 64u + ln;
        if (r < m_rows && on < n) {
            float v = 0.f;
            for (uint32_t w = 0; w < waves; w++) v += red[(w * NT * RL + tr) * 64 + ln];
            __hip_atomic_store(&ws[((size_t)sp * m_rows + r) * n_pad + on], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): this wave's scratch stores have completed
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned prev = __hip_atomic_fetch_add(&counters[tg], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (prev == splits - 1);
    }
    __syncthreads();
    if (!s_last) return;
    if (swiglu) {
        for (uint32_t e = threadIdx.x; e < pair_entries; e += threads) {
            uint32_t ln = e & 31u, tr = e >> 5, r = tr % RL, t = tr / RL;
            uint32_t feat = (tg * NT + t) * 32u + ln, on = (tg * NT + t) * 64u + ln;
            if (r < m_rows && feat < ffn) {
                float g = 0.f, u = 0.f;
                for (uint32_t s = 0; s < splits; s++) {
                    const float *row = &ws[((size_t)s * m_rows + r) * n_pad + on];
                    g += __hip_atomic_load(row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    u += __hip_atomic_load(row + 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                swiglu_out[(size_t)r * ffn + feat] = gated_mul(out.gate_act, g, u);
            }
        }
        if (threadIdx.x == 0) __hip_atomic_store(&counters[tg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    for (uint32_t e = threadIdx.x; e < entries; e += threads) {
        uint32_t ln = e & 63u, tr = e >> 6, r = tr % RL, t = tr / RL;
        uint32_t on = (tg * NT + t) * 64u + ln;
        if (r < m_rows && on < n) {
            float v = 0.f;
            for (uint32_t s = 0; s < splits; s++)
                v += __hip_atomic_load(&ws[((size_t)s * m_rows + r) * n_pad + on], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            gemv4_store_out(out, r, on, v);
        }
    }
    if (threadIdx.x == 0) __hip_atomic_store(&counters[tg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int NT, int RL>
static hipError_t launch_gemv4_t(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m,
                                 const OutSpec &out, float *ws, unsigned *counters, uint32_t waves, uint32_t splits,
                                 float *swiglu_out)
{
    uint32_t n_pad = w.n_tiles * kTileN;                 // multiple of 64
    uint32_t tiles64 = n_pad / 64;
    uint32_t tile_groups = (tiles64 + NT - 1) / NT;
    uint32_t cps = (w.k_chunks + splits - 1) / splits;
    splits = (w.k_chunks + cps - 1) / cps;               // no empty split
    uint32_t blocks = ((tile_groups + 7) / 8) * 8 * splits;
    size_t lds = (size_t)waves * NT * RL * 64 * sizeof(float);
    if (a_f32) {
        if constexpr (RL <= 4)
            hipLaunchKernelGGL((k_gemv4<NT, RL, true>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)w.cq, a, m, w.k, w.n,
                               n_pad, w.k_chunks, tile_groups, splits, cps, (const uint16_t *)nullptr, ws, counters, swiglu_out, out);
        else
            return hipErrorInvalidValue;  // more than four rows: f16 activations only
    } else
        hipLaunchKernelGGL((k_gemv4<NT, RL, false>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)w.cq, a, m, w.k, w.n,
                           n_pad, w.k_chunks, tile_groups, splits, cps, (const uint16_t *)nullptr, ws, counters, swiglu_out, out);
    return hipGetLastError();
}

// M = 1 on the reference's arrays (no repack), f32 activations; one 64-column tile per workgroup.
hipError_t launch_gemv4_ref(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                            const float *a, float *c, float *ws, unsigned *counters, uint32_t waves, uint32_t splits)
{
    if (n == 0) return hipSuccess;
    if (k == 0 || k % 32 != 0 || splits == 0) return hipErrorInvalidValue;
    if (waves != 1 && waves != 2 && waves != 4 && waves != 8 && waves != 16) return hipErrorInvalidValue;
    uint32_t tiles64 = (n + 63) / 64, n_pad = tiles64 * 64;
    uint32_t k_chunks = (k / 32 + 3) / 4;
    uint32_t cps = (k_chunks + splits - 1) / splits;
    splits = (k_chunks + cps - 1) / cps;
    uint32_t blocks = ((tiles64 + 7) / 8) * 8 * splits;
    size_t lds = (size_t)waves * 64 * sizeof(float);
    OutSpec out;
    memset(&out, 0, sizeof out);
    out.count = 1;
    out.seg[0].ptr = c;
    out.seg[0].start = 0;
    out.seg[0].width = n;
    hipLaunchKernelGGL((k_gemv4<1, 1, true, true>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)packed,
                       (const void *)a, 1u, k, n, n_pad, k_chunks, tiles64, splits, cps, scales, ws, counters, (float *)nullptr, out);
    return hipGetLastError();
}

hipError_t launch_gemv4(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                        float *ws, unsigned *counters, uint32_t nt, uint32_t waves, uint32_t splits, float *swiglu_out)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    if (swiglu_out && w.n % 64 != 0) return hipErrorInvalidValue;
    if (m > 8 || (m > 4 && (a_f32 || nt != 1)) || splits == 0 || !w.cq) return hipErrorInvalidValue;
    if (waves != 1 && waves != 2 && waves != 4 && waves != 8 && waves != 16) return hipErrorInvalidValue;
    // a tile group past the end of the padded columns must not exist: NT has to divide the 64-column tile count
    uint32_t tiles64 = w.n_tiles * kTileN / 64;
    if (nt == 0 || tiles64 % nt != 0) return hipErrorInvalidValue;
    uint32_t rl = m;  // rows 0..m-1 live in registers 0..m-1
    if (nt == 1) {
        if (rl == 1) return launch_gemv4_t<1, 1>(s, w, a, a_f32, m, out, ws, counters, waves, splits, swiglu_out);
        if (rl == 2) return launch_gemv4_t<1, 2>(s, w, a, a_f32, m, out, ws, counters, waves, splits, swiglu_out);
        if (rl <= 4) return launch_gemv4_t<1, 4>(s, w, a, a_f32, m, out, ws, counters, waves, splits, swiglu_out);
        // five to eight rows (f16): a second group of four rows repeats the MFMA chain on the unpacked weights
        return launch_gemv4_t<1, 8>(s, w, a, a_f32, m, out, ws, counters, waves, splits, swiglu_out);
    }
    if (nt == 2) {
        if (rl == 1) return launch_gemv4_t<2, 1>(s, w, a, a_f32, m, out, ws, counters, waves, splits, swiglu_out);
        if (rl == 2) return launch_gemv4_t<2, 2>(s, w, a, a_f32, m, out, ws, counters, waves, splits, swiglu_out);
        return launch_gemv4_t<2, 4>(s, w, a, a_f32, m, out, ws, counters, waves, splits, swiglu_out);
    }
    return hipErrorInvalidValue;
}

}  // namespace twm

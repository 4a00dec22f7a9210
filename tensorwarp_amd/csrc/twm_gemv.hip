// Small-M (M <= 16) decode kernel with the activations staged in LDS.
//
// Same arithmetic as twm_decode.hip (one 16x16x32 f16 MFMA per 32-wide group, f32 scale and
// accumulate; reference: crates/kernels/src/quantize.rs:1186-1298) but organised for the
// fewest instructions per weight byte, because at 6+ TB/s the vector ALU is the second
// bottleneck of this kernel:
//   * every wave owns its n-tiles for the whole k-range of the workgroup: no cross-wave
//     reduction, no barrier after the prologue;
//   * the workgroup's slice of A is converted/copied into LDS once and MFMA A-operands are
//     read from there just in time (for M = 1 the sixteen rows of the operand all read row 0,
//     a broadcast);
//   * weight and scale addresses are wave-uniform bases advanced by scalar adds, with the lane
//     offset in one VGPR and the prefetch distance in the instruction's immediate;
//   * P chunks are in flight per wave; loads are unconditional (the tail re-reads the last
//     chunk) so the waits the compiler places are exact.
#include "twm_device.h"

namespace twm {

struct GemvConsts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};

__device__ __forceinline__ GemvConsts make_gemv_consts()
{
    // opaque to the optimiser so that (w & mask) | magic becomes one v_and_or_b32
    GemvConsts c = {0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(c.mask_lo), "+s"(c.mask_hi), "+v"(c.magic_lo), "+v"(c.magic_hi));
    return c;
}

// eight nibbles of the tile order -> eight exact f16 values q - 8 (see twm_decode.hip)
__device__ __forceinline__ half8 gemv_dequant_word(uint32_t w, const GemvConsts &c)
{
    union { uint32_t u[4]; half2v h2[4]; half8 h; } r;
    uint32_t w8 = w >> 8;
    r.u[0] = (w & c.mask_lo) | c.magic_lo;
    r.u[1] = (w & c.mask_hi) | c.magic_hi;
    r.u[2] = (w8 & c.mask_lo) | c.magic_lo;
    r.u[3] = (w8 & c.mask_hi) | c.magic_hi;
    const half2v b_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
    const half2v b_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    r.h2[0] += b_lo;
    r.h2[1] += b_hi;
    r.h2[2] += b_lo;
    r.h2[3] += b_hi;
    return r.h;
}

__device__ __forceinline__ void gemv_store_out(const OutSpec &out, uint32_t m, uint32_t col, float v)
{
#pragma unroll
    for (uint32_t s = 0; s < kMaxSegs; s++) {
        if (s < out.count) {
            uint32_t rel = col - out.seg[s].start;
            if (rel < out.seg[s].width) out.seg[s].ptr[(size_t)m * out.seg[s].width + rel] = v;
        }
    }
}

// Workgroup = 4 waves; wave w owns n-tiles (tg*4 + w)*NT .. +NT and the k-chunks
// [split*cps, (split+1)*cps).  RL = number of accumulator registers that hold live rows
// (min(M, 4)); rows 4..15 of a 16-row tile live in lanes 16..63 of the same registers.
template <int NT, int RL, int P, bool AF32>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 8))) void k_gemv_lds(const uint4v *__restrict__ qw, const uint2v *__restrict__ sc,
                                                   const void *__restrict__ a_any, OutSpec out, float *__restrict__ ws,
                                                   unsigned *__restrict__ counters, uint32_t m_rows, uint32_t k,
                                                   uint32_t n, uint32_t n_tiles, uint32_t k_chunks, uint32_t tile_groups,
                                                   uint32_t splits, uint32_t cps)
{
    extern __shared__ _Float16 a_lds[];  // [m_rows][kr + 8]
    __shared__ int s_last;

    const uint32_t b = blockIdx.x;
    const uint32_t xcd = b & 7u, jj = b >> 3;
    const uint32_t sp = jj % splits;
    const uint32_t tg = (jj / splits) * 8u + xcd;
    if (tg >= tile_groups) return;

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t c = lane & 15u, kb = lane >> 4;
    const uint32_t kc0 = sp * cps;
    const uint32_t kc1 = (kc0 + cps < k_chunks) ? kc0 + cps : k_chunks;
    const uint32_t nchunks = kc1 > kc0 ? kc1 - kc0 : 0;
    const uint32_t kr = nchunks * 128u;
    const uint32_t stride = kr + 8u;  // halves; +16 B per row keeps the 16 rows of a b128 read on distinct banks

    // ---- this wave's tiles; a wave past the end works on the last tiles and stores nothing ----
    uint32_t nt_w = (tg * 4u + wave) * NT;
    const bool wave_live = nt_w < n_tiles;
    if (!wave_live) nt_w = n_tiles - NT;

    // ---- issue the first P chunks of weights before touching A, so both latencies overlap ----
    // Addresses are (wave-uniform byte pointer) + (per-lane 32-bit offset): scalar base, one VGPR.
    const char *qb[NT];
    const char *sb[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        qb[t] = (const char *)(qw + ((size_t)kc0 * n_tiles + nt_w + t) * 64);
        sb[t] = (const char *)(sc + ((size_t)kc0 * n_tiles + nt_w + t) * 16);
    }
    const uint32_t lane16 = lane * 16u, c8 = c * 8u;
    const size_t qstep = (size_t)n_tiles * 1024u, sstep = (size_t)n_tiles * 128u;  // bytes between k-chunks
    const uint32_t last = nchunks ? nchunks - 1 : 0;
    // Two rings of P slots.  Nibbles of chunk j live in slot j % P and are refilled, in place, with
    // chunk j + P as soon as they have been unpacked.  A scale is still needed after the MFMA, so the
    // scale slot of step j is refilled one step later (with chunk j + P): no value is ever live
    // across its own refill, hence no register copies and no wait for a load just issued.
    uint4v wq_ring[P][NT];
    uint2v sc_ring[P][NT];
#pragma unroll
    for (int p = 0; p < P; p++) {
        uint32_t j = (uint32_t)p < last ? (uint32_t)p : last;
        if (nchunks == 0) break;  // never launched (the host normalises the split count); no load without a chunk
#pragma unroll
        for (int t = 0; t < NT; t++) {
            wq_ring[p][t] = *(const uint4v *)(qb[t] + (size_t)j * qstep + lane16);
            if (p < P - 1) sc_ring[p][t] = *(const uint2v *)(sb[t] + (size_t)j * sstep + c8);
        }
    }

    // ---- stage A[0..m_rows)[kc0*128 .. kc1*128) into LDS as f16 ----
    {
        const uint32_t vec_per_row = kr / 8u;
        const uint32_t total = m_rows * vec_per_row;
        for (uint32_t idx = threadIdx.x; idx < total; idx += 256u) {
            uint32_t row = idx / vec_per_row, v8 = idx - row * vec_per_row;
            uint32_t kk = kc0 * 128u + v8 * 8u;
            half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (kk < k) {  // k-chunks past K exist only as zero padding of the last chunk
                if (AF32) {
                    const float4 *p = (const float4 *)((const float *)a_any + (size_t)row * k + kk);
                    float4 x = p[0], y = p[1];
                    v = half8{(_Float16)x.x, (_Float16)x.y, (_Float16)x.z, (_Float16)x.w,
                              (_Float16)y.x, (_Float16)y.y, (_Float16)y.z, (_Float16)y.w};
                } else {
                    v = *(const half8 *)((const _Float16 *)a_any + (size_t)row * k + kk);
                }
            }
            *(half8 *)(a_lds + row * stride + v8 * 8u) = v;
        }
    }
    __syncthreads();

    const GemvConsts dq = make_gemv_consts();
    uint32_t arow = c < m_rows ? c : m_rows - 1;  // rows >= M replay row M-1; their outputs are never stored
    const _Float16 *ap = a_lds + arow * stride + kb * 8u;

    float acc[NT][RL];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int r = 0; r < RL; r++) acc[t][r] = 0.f;

    // One chunk (slot p = j % P): unpack, refill, then one MFMA per 32-wide group, scale and
    // accumulate in f32.  The scheduling barriers keep the three phases in this order: left free, the
    // instruction scheduler hoists the refill above the unpack (forcing copies) or sinks all loads of
    // the unrolled body to its end (putting a full memory latency on every trip).
    auto process = [&](const int p, uint32_t j, bool refill) {
        half8 bf[NT][4];
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) bf[t][i] = gemv_dequant_word(wq_ring[p][t][i], dq);
        if (refill) {
            // an empty asm (no instruction) that consumes the unpacked registers and clobbers memory:
            // the unpack cannot sink below it, the refill loads cannot rise above it
#pragma unroll
            for (int t = 0; t < NT; t++)
                asm volatile("" : "+v"(bf[t][0]), "+v"(bf[t][1]), "+v"(bf[t][2]), "+v"(bf[t][3]) : : "memory");
            const uint32_t jq = j + P < last ? j + P : last;          // the tail re-reads the last chunk
            const uint32_t js = j + P - 1 < last ? j + P - 1 : last;
            const int ps = (p + P - 1) % P;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                wq_ring[p][t] = *(const uint4v *)(qb[t] + (size_t)jq * qstep + lane16);
                sc_ring[ps][t] = *(const uint2v *)(sb[t] + (size_t)js * sstep + c8);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        half8 af[4];
#pragma unroll
        for (int i = 0; i < 4; i++) af[i] = *(const half8 *)(ap + (j * 128u + i * 32u));
#pragma unroll
        for (int t = 0; t < NT; t++) {
            union { uint2v u; _Float16 h[4]; } sv;
            sv.u = sc_ring[p][t];
            float4v d[4];
#pragma unroll
            for (int i = 0; i < 4; i++)
                d[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], bf[t][i], float4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float s = (float)sv.h[i];
#pragma unroll
                for (int r = 0; r < RL; r++) acc[t][r] = fmaf(d[i][r], s, acc[t][r]);
            }
        }
    };

    // ---- steady state: whole groups of P chunks, no guards, so every wait count is exact ----
    const uint32_t full = nchunks - nchunks % P;
    for (uint32_t j0 = 0; j0 < full; j0 += P) {
#pragma unroll
        for (int p = 0; p < P; p++) process(p, j0 + p, true);
    }
    // ---- tail: the last nchunks % P chunks are already in the rings ----
#pragma unroll
    for (int p = 0; p < P - 1; p++)
        if (full + p < nchunks) process(p, full + p, false);

    // ---- epilogue: lane (c, kb) holds rows kb*4 + r of column (nt_w + t)*16 + c ----
    const uint32_t n_ld = ((n + kNPadTo - 1) / kNPadTo) * kNPadTo;
    if (splits == 1) {
        if (wave_live) {
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int r = 0; r < RL; r++) {
                    uint32_t om = kb * 4u + r, on = (nt_w + t) * 16u + c;
                    if (om < m_rows && on < n) gemv_store_out(out, om, on, acc[t][r]);
                }
        }
        return;
    }

    // cross-workgroup split-K: park the partial tile (agent-scope relaxed atomics: coherent across
    // the XCDs' L2s without a cache write-back), bump the arrival counter once the stores have
    // completed; the last workgroup to arrive adds the partials in ascending split order.
    if (wave_live) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int r = 0; r < RL; r++) {
                uint32_t om = kb * 4u + r, on = (nt_w + t) * 16u + c;
                if (om < m_rows && on < n)
                    __hip_atomic_store(&ws[((size_t)sp * m_rows + om) * n_ld + on], acc[t][r], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
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
    if (wave_live) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int r = 0; r < RL; r++) {
                uint32_t om = kb * 4u + r, on = (nt_w + t) * 16u + c;
                if (om < m_rows && on < n) {
                    float v = 0.f;
                    for (uint32_t s = 0; s < splits; s++)
                        v += __hip_atomic_load(&ws[((size_t)s * m_rows + om) * n_ld + on], __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                    gemv_store_out(out, om, on, v);
                }
            }
    }
    if (threadIdx.x == 0) __hip_atomic_store(&counters[tg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int NT, int RL, int P>
static hipError_t launch_gemv_t(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m,
                                const OutSpec &out, float *ws, unsigned *counters, uint32_t splits)
{
    uint32_t tile_groups = (w.n_tiles + 4 * NT - 1) / (4 * NT);
    uint32_t cps = (w.k_chunks + splits - 1) / splits;
    splits = (w.k_chunks + cps - 1) / cps;  // no empty split: every workgroup has at least one k-chunk
    uint32_t blocks = ((tile_groups + 7) / 8) * 8 * splits;
    size_t lds = (size_t)m * (cps * 128 + 8) * sizeof(_Float16);
    if (a_f32)
        hipLaunchKernelGGL((k_gemv_lds<NT, RL, P, true>), dim3(blocks), dim3(256), lds, s, (const uint4v *)w.qw,
                           (const uint2v *)w.sc, a, out, ws, counters, m, w.k, w.n, w.n_tiles, w.k_chunks, tile_groups,
                           splits, cps);
    else
        hipLaunchKernelGGL((k_gemv_lds<NT, RL, P, false>), dim3(blocks), dim3(256), lds, s, (const uint4v *)w.qw,
                           (const uint2v *)w.sc, a, out, ws, counters, m, w.k, w.n, w.n_tiles, w.k_chunks, tile_groups,
                           splits, cps);
    return hipGetLastError();
}

template <int NT, int P>
static hipError_t launch_gemv_nt(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m,
                                 const OutSpec &out, float *ws, unsigned *counters, uint32_t splits)
{
    if (m == 1) return launch_gemv_t<NT, 1, P>(s, w, a, a_f32, m, out, ws, counters, splits);
    if (m == 2) return launch_gemv_t<NT, 2, P>(s, w, a, a_f32, m, out, ws, counters, splits);
    return launch_gemv_t<NT, 4, P>(s, w, a, a_f32, m, out, ws, counters, splits);
}

// LDS needed by a launch: the workgroup's slice of A as f16 plus one pad vector per row.
size_t gemv_lds_bytes(uint32_t m, uint32_t k_chunks, uint32_t splits)
{
    uint32_t cps = (k_chunks + splits - 1) / splits;
    return (size_t)m * (cps * 128 + 8) * 2;
}

hipError_t launch_gemv_lds(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                           float *ws, unsigned *counters, uint32_t nt, uint32_t depth, uint32_t splits)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    if (m > 16 || splits == 0 || w.n_tiles < nt) return hipErrorInvalidValue;
    if (gemv_lds_bytes(m, w.k_chunks, splits) > kGemvMaxLds) return hipErrorInvalidValue;
    if (depth == 2) {
        if (nt == 1) return launch_gemv_nt<1, 2>(s, w, a, a_f32, m, out, ws, counters, splits);
        if (nt == 2) return launch_gemv_nt<2, 2>(s, w, a, a_f32, m, out, ws, counters, splits);
        if (nt == 4) return launch_gemv_nt<4, 2>(s, w, a, a_f32, m, out, ws, counters, splits);
    } else if (depth == 4) {
        if (nt == 1) return launch_gemv_nt<1, 4>(s, w, a, a_f32, m, out, ws, counters, splits);
        if (nt == 2) return launch_gemv_nt<2, 4>(s, w, a, a_f32, m, out, ws, counters, splits);
        if (nt == 4) return launch_gemv_nt<4, 4>(s, w, a, a_f32, m, out, ws, counters, splits);
    }
    return hipErrorInvalidValue;
}

}  // namespace twm

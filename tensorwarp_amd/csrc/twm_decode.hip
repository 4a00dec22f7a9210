// Decode kernel on the 16-column tile order, M = 1..16 rows of activations (used for M = 5..16;
// M <= 4 runs the one-lane-per-column kernel of twm_gemv4.hip).
//
// C[m][n] = sum_g f32(scale[g][n]) * sum_{k in g} A[m][k] * (q[k][n] - 8), f32 accumulation: the
// arithmetic of warp_gemm_tw_marlin_m1 (crates/kernels/src/quantize.rs:1186-1245 in the
// reference) with the inner 32-term sum done by one 16x16x32 f16 MFMA per group.  The kernel is
// HBM-bound: every weight byte is read once, 16 B per lane, 1 KiB per wave per load.
#include "twm_device.h"

namespace twm {

// One u32 of the tile order -> eight f16 values (q - 8), exact.
//   (w & 0x000F000F) | 0x64006400 : two halves 1024 + q       (nibbles at bits 0..3)
//   (w & 0x00F000F0) | 0x54005400 : two halves   64 + q       (nibbles at bits 4..7)
// then a packed subtract of 1032 / 72.  Thanks to the nibble permutation done at repack the
// four resulting registers hold k-offsets (0,1) (2,3) (4,5) (6,7): the MFMA B-operand order.
struct DequantConsts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};

// The four constants are made opaque to the optimiser (an empty asm that emits nothing), so that
// they live in registers and (w & mask) | magic is selected as one v_and_or_b32 instead of a
// v_and + v_or pair with literals.  No instruction is written in inline asm: the compiler must
// see every VALU write to place the wait states MFMA results need.
__device__ __forceinline__ DequantConsts make_dequant_consts()
{
    DequantConsts c = {0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(c.mask_lo), "+s"(c.mask_hi), "+v"(c.magic_lo), "+v"(c.magic_hi));
    return c;
}

__device__ __forceinline__ half8 dequant_word(uint32_t w, const DequantConsts &c)
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

__device__ __forceinline__ void store_out(const OutSpec &out, uint32_t m, uint32_t col, float v)
{
#pragma unroll
    for (uint32_t s = 0; s < kMaxSegs; s++) {
        if (s < out.count) {
            uint32_t rel = col - out.seg[s].start;
            if (rel < out.seg[s].width) out.seg[s].ptr[(size_t)m * out.seg[s].width + rel] = out.seg[s].bias ? v + out.seg[s].bias[rel] : v;
        }
    }
}

template <int NT>
struct ChunkRegs {
    uint4v wq[NT];     // 16 B of nibbles per lane per n-tile
    uint2v sc[NT];     // four f16 scales (the chunk's four groups) of this lane's column
    half8 a[4];        // MFMA A operands: 8 consecutive k of row (lane % 16) per group
};

// Workgroup = `waves` waves (blockDim.x / 64).  It owns NT n-tiles (16*NT columns) and the
// k-chunks [split*cps, (split+1)*cps) of them; wave w takes chunks w, w+waves, ... of that range
// with the next chunk's loads in flight while the current one is computed.  The per-wave partial
// tiles are summed through LDS, and, when the launch is also split along K across workgroups, the
// workgroup parks its tile in `ws` and the last workgroup to arrive for the tile adds the `splits`
// partials in ascending order (deterministic) and stores the result.
//   RL : accumulator registers that can hold live rows (M for M < 4, else 4)
// Rows of A beyond M are read from row M-1 instead of being zeroed (no branches in the loop);
// the output rows they produce are never stored.
// Block ids are dealt round-robin to the 8 XCDs; the id is unfolded so that every split of a
// tile lands on the same XCD and the partials stay in that XCD's L2.
template <int NT, int RL, bool AF32>
__global__ __launch_bounds__(1024) void k_decode(const uint4v *__restrict__ qw, const uint2v *__restrict__ sc,
                                                  const void *__restrict__ a_any, OutSpec out, float *__restrict__ ws,
                                                  unsigned *__restrict__ counters, uint32_t m_rows, uint32_t k,
                                                  uint32_t n, uint32_t k_chunks, uint32_t tile_groups, uint32_t splits,
                                                  uint32_t cps)
{
    constexpr int MT = 1;  // one 16-row block of A
    constexpr int IDX = NT * MT * 4;
    extern __shared__ float red[];  // [waves][IDX][64]
    __shared__ int s_last;

    const uint32_t b = blockIdx.x;
    const uint32_t xcd = b & 7u, jj = b >> 3;
    const uint32_t sp = jj % splits;
    const uint32_t tg = (jj / splits) * 8u + xcd;
    if (tg >= tile_groups) return;  // whole workgroup leaves together

    const uint32_t waves = blockDim.x >> 6;
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const uint32_t c = lane & 15u, kb = lane >> 4;
    const uint32_t nt0 = tg * NT;
    const uint32_t kc0 = sp * cps;
    const uint32_t kc1 = (kc0 + cps < k_chunks) ? kc0 + cps : k_chunks;

    const DequantConsts dq = make_dequant_consts();

    // per-lane bases; the loop only adds chunk offsets
    const uint32_t n_tiles = tile_groups * NT;
    const uint4v *qbase = qw + (size_t)nt0 * 64 + lane;
    const uint2v *sbase = sc + (size_t)nt0 * 16 + c;
    size_t a_row_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        uint32_t row = mt * 16 + c;
        if (row > m_rows - 1) row = m_rows - 1;
        a_row_off[mt] = (size_t)row * k;
    }

    float4v acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[t][mt] = float4v{0.f, 0.f, 0.f, 0.f};

    auto load_chunk = [&](ChunkRegs<NT> &r, uint32_t kc) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            r.wq[t] = qbase[((size_t)kc * n_tiles + t) * 64];
            r.sc[t] = sbase[((size_t)kc * n_tiles + t) * 16];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t k0 = kc * 128u + i * 32u + kb * 8u;
            if (k0 > k - 8u) k0 = k - 8u;  // padded groups carry scale 0; any finite A will do
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                if (AF32) {
                    const float4 *p = (const float4 *)((const float *)a_any + a_row_off[mt] + k0);
                    float4 x = p[0], y = p[1];
                    r.a[i] = half8{(_Float16)x.x, (_Float16)x.y, (_Float16)x.z, (_Float16)x.w,
                                       (_Float16)y.x, (_Float16)y.y, (_Float16)y.z, (_Float16)y.w};
                } else {
                    r.a[i] = *(const half8 *)((const _Float16 *)a_any + a_row_off[mt] + k0);
                }
            }
        }
    };

    auto compute_chunk = [&](const ChunkRegs<NT> &r) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            union { uint2v u; _Float16 h[4]; } sv;
            sv.u = r.sc[t];
            half8 bf[4];
#pragma unroll
            for (int i = 0; i < 4; i++) bf[i] = dequant_word(r.wq[t][i], dq);
            float4v d[4][MT];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
                    d[i][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.a[i], bf[i], float4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float s = (float)sv.h[i];
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int r2 = 0; r2 < RL; r2++) acc[t][mt][r2] = fmaf(d[i][mt][r2], s, acc[t][mt][r2]);
            }
        }
    };

    {
        // two register sets used alternately: the loads of one are in flight while the other is
        // consumed, and no set is ever copied (a copy would have to wait for its loads)
        ChunkRegs<NT> r0, r1;
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

    // ---- sum the waves' partial tiles through LDS ----
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int r = 0; r < RL; r++) red[(wave * IDX + (t * MT + mt) * 4 + r) * 64 + lane] = acc[t][mt][r];
    __syncthreads();

    const uint32_t n_ld = ((n + kNPadTo - 1) / kNPadTo) * kNPadTo;  // row stride of the split-K scratch
    const uint32_t threads = blockDim.x;

    // entry e = idx * 64 + ln, idx = (t*MT + mt)*4 + r : output row mt*16 + (ln/16)*4 + r, column (nt0+t)*16 + ln%16
    if (splits == 1) {
        for (uint32_t e = threadIdx.x; e < (uint32_t)IDX * 64u; e += threads) {
            uint32_t idx = e >> 6, ln = e & 63u;
            uint32_t r = idx & 3u, tm = idx >> 2;
            uint32_t om = (tm % MT) * 16 + (ln >> 4) * 4 + r, on = (nt0 + tm / MT) * 16 + (ln & 15u);
            if (r < (uint32_t)RL && om < m_rows && on < n) {
                float v = 0.f;
                for (uint32_t w = 0; w < waves; w++) v += red[(w * IDX + idx) * 64 + ln];
                store_out(out, om, on, v);
            }
        }
        return;
    }

    // ---- cross-workgroup split-K: park the partial, last arrival reduces ----
    // The scratch is written and read with agent-scope relaxed atomics (accesses that are coherent
    // across the XCDs' L2s by themselves), so no cache write-back / invalidate fence is needed:
    // waiting for the stores to complete before the arrival counter is bumped orders them.
    for (uint32_t e = threadIdx.x; e < (uint32_t)IDX * 64u; e += threads) {
        uint32_t idx = e >> 6, ln = e & 63u;
        uint32_t r = idx & 3u, tm = idx >> 2;
        uint32_t om = (tm % MT) * 16 + (ln >> 4) * 4 + r, on = (nt0 + tm / MT) * 16 + (ln & 15u);
        if (r < (uint32_t)RL && om < m_rows && on < n) {
            float v = 0.f;
            for (uint32_t w = 0; w < waves; w++) v += red[(w * IDX + idx) * 64 + ln];
            __hip_atomic_store(&ws[((size_t)sp * m_rows + om) * n_ld + on], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
    for (uint32_t e = threadIdx.x; e < (uint32_t)IDX * 64u; e += threads) {
        uint32_t idx = e >> 6, ln = e & 63u;
        uint32_t r = idx & 3u, tm = idx >> 2;
        uint32_t om = (tm % MT) * 16 + (ln >> 4) * 4 + r, on = (nt0 + tm / MT) * 16 + (ln & 15u);
        if (r < (uint32_t)RL && om < m_rows && on < n) {
            float v = 0.f;
            for (uint32_t s = 0; s < splits; s++)
                v += __hip_atomic_load(&ws[((size_t)s * m_rows + om) * n_ld + on], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            store_out(out, om, on, v);
        }
    }
    if (threadIdx.x == 0) __hip_atomic_store(&counters[tg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
}

template <int NT, int RL>
static hipError_t launch_decode_t(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m,
                                  const OutSpec &out, float *ws, unsigned *counters, const DecodePlan &plan)
{
    uint32_t tile_groups = w.n_tiles / NT;
    uint32_t cps = (w.k_chunks + plan.splits - 1) / plan.splits;
    uint32_t nsplits = (w.k_chunks + cps - 1) / cps;  // no empty split
    uint32_t blocks = ((tile_groups + 7) / 8) * 8 * nsplits;
    uint32_t threads = plan.waves * 64;
    size_t lds = (size_t)plan.waves * NT * 4 * 64 * sizeof(float);
    if (a_f32)
        hipLaunchKernelGGL((k_decode<NT, RL, true>), dim3(blocks), dim3(threads), lds, s, (const uint4v *)w.qw,
                           (const uint2v *)w.sc, a, out, ws, counters, m, w.k, w.n, w.k_chunks, tile_groups, nsplits, cps);
    else
        hipLaunchKernelGGL((k_decode<NT, RL, false>), dim3(blocks), dim3(threads), lds, s, (const uint4v *)w.qw,
                           (const uint2v *)w.sc, a, out, ws, counters, m, w.k, w.n, w.k_chunks, tile_groups, nsplits, cps);
    return hipGetLastError();
}

template <int NT>
static hipError_t launch_decode_nt(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m,
                                   const OutSpec &out, float *ws, unsigned *counters, const DecodePlan &plan)
{
    if (m == 1) return launch_decode_t<NT, 1>(s, w, a, a_f32, m, out, ws, counters, plan);
    if (m == 2) return launch_decode_t<NT, 2>(s, w, a, a_f32, m, out, ws, counters, plan);
    return launch_decode_t<NT, 4>(s, w, a, a_f32, m, out, ws, counters, plan);
}

hipError_t launch_decode(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                         float *ws, unsigned *counters, DecodePlan plan)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    if (m > (uint32_t)kMaxDecodeM || plan.splits == 0) return hipErrorInvalidValue;
    if (plan.waves != 4 && plan.waves != 8 && plan.waves != 16) return hipErrorInvalidValue;
    if (plan.waves * plan.nt > 64) return hipErrorInvalidValue;  // LDS reduction buffer <= 64 KiB
    switch (plan.nt) {
    case 1: return launch_decode_nt<1>(s, w, a, a_f32, m, out, ws, counters, plan);
    case 2: return launch_decode_nt<2>(s, w, a, a_f32, m, out, ws, counters, plan);
    case 4: return launch_decode_nt<4>(s, w, a, a_f32, m, out, ws, counters, plan);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace twm

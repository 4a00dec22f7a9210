// Sub-tile variant of the lane-per-column decode kernel (M <= 4; up to M = 16 with f16 rows): finer workgroups
// without a cross-workgroup reduction.
//
// k_gemv4 gives a workgroup a whole 64-column tile; with 592 tiles on 256 CUs that is 2.3 long-lived
// workgroups per CU, and a plain read of the same bytes in that decomposition is 1.3 - 1.6 us slower than in
// many short-lived workgroups.  Here a workgroup owns SUB = 32 or 16 columns of a tile and a wave covers
// 64 / SUB consecutive k-chunks of them in one pass: lane l = (chunk l / SUB of the pass, column l % SUB).
// The column-lane copy is read as it is (a sub-tile's 16-byte records of one group are SUB * 16 contiguous
// bytes).  The 4x4x4 MFMA broadcasts its A block inside groups of 2^CBSZ blocks, so with CBSZ = log2(SUB / 4)
// every group of SUB lanes takes the activations of its own chunk: one A register holds 2 * SUB of the
// chunk's 128 k-values (SUB / 4 pieces of eight), 64 / SUB registers the whole chunk.  The MFMA count per
// byte of weights is unchanged (every lane of every MFMA is a live column).  With 28 chunks and SUB = 16 a
// workgroup of eight waves makes exactly one pass: every load of the launch is issued at once, the kernel has
// no loop and needs about 50 registers, and 3584 -> 37888 becomes 2368 short-lived workgroups.
// Rows five to sixteen (f16) repeat the MFMA chain on the unpacked weights per group of four rows.
// One row of activations, f16 in the pipelined loop or f32 anywhere, is loaded a piece per lane and handed round the
// quads of lanes by DPP (the term modes kTermsOneRow / kTermsOneRowF32 of twm_gemv4_core.h); f32 values are taken as
// two f16 terms, first term and residual, which ride in rows 0 and 1 of the MFMA's A block.
//
// Arithmetic and output as k_gemv4 (crates/kernels/src/quantize.rs:1186-1298).
#include "twm_gemv4_core.h"
#include "twm_internal.h"
#include <cstring>

namespace twm {

namespace {

// the launch's small numbers in one argument word: K-splits (bits 0-11; the launchers cap the factor at 4095), gated
// store (12), waves per workgroup (13-17), rows (18-22), a contiguous run of sub-tiles per XCD (23)
__host__ __device__ __forceinline__ uint32_t gemv4s_cfg(uint32_t splits, bool gated, uint32_t waves, uint32_t rows, bool runs = false)
{
    return splits | (gated ? 0x1000u : 0u) | (waves << 13) | (rows << 18) | (runs ? 0x800000u : 0u);
}
__device__ __forceinline__ bool cfg_runs(uint32_t cfg) { return (cfg & 0x800000u) != 0; }
__device__ __forceinline__ uint32_t cfg_splits(uint32_t cfg) { return cfg & 0xFFFu; }
__device__ __forceinline__ bool cfg_gated(uint32_t cfg) { return (cfg & 0x1000u) != 0; }
__device__ __forceinline__ uint32_t cfg_waves(uint32_t cfg) { return (cfg >> 13) & 0x1Fu; }
__device__ __forceinline__ uint32_t cfg_rows(uint32_t cfg) { return (cfg >> 18) & 0x1Fu; }

__device__ __forceinline__ void gemv4s_store_out(const OutSpec &out, uint32_t m, uint32_t col, float v)
{
#pragma unroll
    for (uint32_t s = 0; s < kMaxSegs; s++) {
        if (s < out.count) {
            uint32_t rel = col - out.seg[s].start;
            if (rel < out.seg[s].width) out.seg[s].ptr[(size_t)m * out.seg[s].width + rel] = out.seg[s].bias ? v + out.seg[s].bias[rel] : v;
        }
    }
}

}  // namespace

// grid: sub-tiles (rounded up to the 8 XCDs) x splits, unfolded like k_gemv4; workgroup = `waves` waves that
// take the passes (64 / SUB chunks each) of the k-range in turn.
// REFL: cw is the reference's packed array u8 [G][N][16] and ref_scales its f16 [G][N] (no repack; one row of f32
// activations): a sub-tile's records of one group are still SUB * 16 contiguous bytes.
// NP >= 2 (16 columns, one row): every wave makes up to NP passes and issues all their loads before its first unpack
// (gemv4s_run_upfront): a workgroup that is alone on its CU has its whole share of the matrix in flight at once, like
// the one-pass form, where the pass loop keeps two passes per wave in flight and walks K one memory round trip at a time.
template <int SUB, int RL, bool AF32, bool ONE, bool REFL, int NP = 0>
__device__ __forceinline__ void gemv4s_body(const char *__restrict__ cw, const void *__restrict__ a_any, const OutSpec &out,
                                            float *__restrict__ ws, unsigned *__restrict__ counters, uint32_t cfg,
                                            uint32_t k, uint32_t n, uint32_t n_pad, uint32_t k_chunks,
                                            uint32_t sub_tiles, uint32_t cps,
                                            const uint16_t *__restrict__ ref_scales, uint32_t *trace_loaded)
{
    const uint32_t splits = cfg_splits(cfg), waves = cfg_waves(cfg), m_rows = cfg_rows(cfg);
    const bool gated_store = cfg_gated(cfg);
    static_assert(!REFL || (AF32 && RL == 1), "the reference-layout variant is the M = 1, f32-activation entry point");
    constexpr int CPP = 64 / SUB;     // chunks per pass
    // f16 activations on 16 columns, several passes per wave (deep K), up to four rows: the pipelined pass loop, and for
    // one row the shared-piece form of the activations (18944 -> 3584: 8.9 against 10.0 us at M = 1, 9.95 against 10.35
    // at M = 2, level at M = 4).  A wave that makes a single pass gains nothing from either, and the other variants
    // run out of registers with both sets live.
    // One row of f32 activations: the shared-piece form as well (a lane splits one piece instead of two or four),
    // which on 16 columns also leaves room for the pipelined loop.
    constexpr bool F32_PIECE = AF32 && RL == 1;
    constexpr bool UPFRONT = NP >= 2;
    static_assert(!UPFRONT || (!ONE && RL == 1 && SUB == 16), "several passes up front: one row on 16 columns");
    constexpr bool PIPE = !ONE && !UPFRONT && (!AF32 || F32_PIECE) && RL <= 4 && SUB == 16;
    constexpr int TERMS = F32_PIECE ? kTermsOneRowF32 : ((PIPE || UPFRONT) && RL == 1) ? kTermsOneRow : gemv4_terms<AF32, RL>();
    extern __shared__ float red[];    // [waves][RL][SUB]
    __shared__ int s_last;

    const uint32_t b = blockIdx.x;
    const uint32_t xcd = b & 7u, jj = b >> 3;
    // (unsplit, as the planner's sub-tile forms are: no division in front of the first loads)
    const uint32_t sp = splits == 1 ? 0u : jj % splits, jt = splits == 1 ? jj : jj / splits;
    // Workgroups reach the eight XCDs in turn by linear id.  Repacked copy: sub-tile = id (every block of the copy belongs
    // to one workgroup).  The reference's arrays: neighbouring sub-tiles share the 128-byte lines of the scale rows (32 or
    // 64 bytes per sub-tile and group), so each XCD takes a contiguous run of sub-tiles and the shared lines meet in its L2.
    const uint32_t st = (REFL || cfg_runs(cfg)) ? xcd * ((sub_tiles + 7u) >> 3) + jt : jt * 8u + xcd;
    if (st >= sub_tiles) return;

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t cl = lane % SUB, cg = lane / SUB;          // column in the sub-tile, chunk of the pass
    const uint32_t tile = st / CPP, part = st % CPP;           // CPP sub-tiles per 64-column tile
    const uint32_t kc0 = sp * cps;
    const uint32_t kc1 = (kc0 + cps < k_chunks) ? kc0 + cps : k_chunks;
    const uint32_t passes = (kc1 - kc0 + CPP - 1) / CPP;

    // Gated store (paired gate_up weight: each 64-column tile is 32 gate columns, then the up columns of the same
    // features): the workgroup takes SUB / 2 gate columns and their up columns, so that it can write the products.
    const bool gated = !REFL && gated_store;  // (= out.swiglu != nullptr, as an argument of its own: see k_gemv4s)
    auto col_in_tile = [&](uint32_t c) {
        return gated ? (c / (SUB / 2)) * 32u + part * (SUB / 2) + c % (SUB / 2) : part * SUB + c;
    };
    const char *tbase = cw + (size_t)tile * k_chunks * kColBlockBytes;
    const uint32_t ref_col = st * SUB + cl < n ? st * SUB + cl : n - 1u;  // REFL: columns past n replay the last one
    const uint32_t ref_groups = k / 32u;
    const Gemv4Consts dq = make_gemv4_consts();

    uint32_t arow = (TERMS == kTermsOneRow || TERMS == kTermsOneRowF32) ? 0u : TERMS == kTermsRowPacked ? (cl & 3u) >> 1 : cl & 3u;
    if (arow > m_rows - 1) arow = m_rows - 1;
    const bool lane_is_lo = TERMS == kTermsRowPacked && (cl & 1u) != 0;

    float acc[RL];
#pragma unroll
    for (int r = 0; r < RL; r++) acc[r] = 0.f;

    constexpr int RG = (RL + 3) / 4;  // rows beyond four repeat the MFMA chain (f16 activations)
    auto load_pass = [&](ChunkS<SUB, RG> &r, uint32_t pass) {
        uint32_t kc = kc0 + pass * CPP + cg;
        const bool live = kc < kc1;
        kc = live ? kc : kc1 - 1u;  // a chunk past the k-range replays the last one with scale 0
        if (REFL) {
            gemv4s_load_pass_ref<SUB, TERMS, RG>(r, cw, ref_scales, a_any, arow, kc, live, ref_col, st * SUB + cl < n, n, ref_groups,
                                                 cl, k, lane_is_lo);
        } else {
            if (PIPE || UPFRONT) {
                // activations first: loads complete in the order of their issue, and these come from the cache
                gemv4s_load_a<SUB, AF32, TERMS, REFL, RG>(r, a_any, arow, kc, cl, k, lane_is_lo, m_rows);
                gemv4s_load_w<SUB, RG, true>(r, tbase + (size_t)kc * kColBlockBytes, col_in_tile(cl), live);
            } else if (F32_PIECE) {
                // (the same order: the split of the f32 piece can then run while the weights are on their way)
                gemv4s_load_a<SUB, AF32, TERMS, REFL, RG>(r, a_any, arow, kc, cl, k, lane_is_lo, m_rows);
                gemv4s_load_w<SUB, RG, false>(r, tbase + (size_t)kc * kColBlockBytes, col_in_tile(cl), live);
            } else {
                gemv4s_load_w<SUB, RG, false>(r, tbase + (size_t)kc * kColBlockBytes, col_in_tile(cl), live);
                gemv4s_load_a<SUB, AF32, TERMS, REFL, RG>(r, a_any, arow, kc, cl, k, lane_is_lo, m_rows);
            }
        }
    };
    auto compute_pass = [&](const ChunkS<SUB, RG> &r) { gemv4s_compute<SUB, RL, TERMS, REFL>(r, dq, acc); };
    // (ONE: the launcher saw that no wave has a second pass: one register set, no loop)
    if constexpr (UPFRONT) gemv4s_run_upfront<SUB, NP, RG>(wave, waves, passes, load_pass, compute_pass);
    else gemv4s_run_passes<SUB, ONE, RG, PIPE>(wave, waves, passes, load_pass, compute_pass);
    if (trace_loaded && threadIdx.x == 0) *trace_loaded = (uint32_t)__builtin_amdgcn_s_memrealtime();  // data arrived and unpacked

    // ---- sum over the chunks of a pass (lane groups) inside the wave, over the waves through LDS ----
    // In the wave: lanes l, l + SUB, ... hold the same column; two lane swaps (v_permlane32_swap, v_permlane16_swap)
    // and two adds leave the wave's total of a column in every lane that holds it - no LDS, no wait.  Across the waves:
    // one LDS hop of waves * RL * SUB floats.  Where the RL * SUB entries of the workgroup fit one wave (one or two
    // rows, four on 16 columns), wave 0 alone finishes: 64 / E lanes per entry each add every (64 / E)-th wave's value,
    // four independent reads at a time, and the same lane swaps add those - against one thread walking waves * 64 / SUB
    // values one dependent read after the other, which took longer than the unpack of a pass.
    constexpr int E = RL * SUB;       // entries of the workgroup: e = r * SUB + column
    // (More entries than a wave has lanes, i.e. five rows and more: two lane swaps per row and wave are sixteen to
    // thirty-two swaps per wave, which with four waves on a SIMD cost more than they save -- 3584 -> 4608 at 16 rows 8.2
    // against 7.7 us; there every lane writes its sums and the thread that finishes an entry adds the lane groups too.)
    constexpr bool WIDE = E > 64;
    if constexpr (WIDE) {
#pragma unroll
        for (int r = 0; r < RL; r++) red[(wave * RL + r) * 64 + lane] = acc[r];
    } else {
#pragma unroll
        for (int r = 0; r < RL; r++) acc[r] = sum_lane_groups<SUB>(acc[r]);
        if (cg == 0) {
#pragma unroll
            for (int r = 0; r < RL; r++) red[wave * E + r * SUB + cl] = acc[r];
        }
    }
    __syncthreads();

    const uint32_t ffn = n >> 1;
    auto col_of = [&](uint32_t c) { return REFL ? st * SUB + c : tile * 64u + col_in_tile(c); };
    // Four values at a time of entry e, waves first, first + step, ...: the reads are independent, the sum is in
    // wave order.  (A wave past the last one re-reads wave 0's value and counts as zero: no branch round a read.)
    auto sum_waves = [&](uint32_t e, uint32_t first, uint32_t step) {
        float t = 0.f;
        for (uint32_t w0 = first; w0 < waves; w0 += 4u * step) {
            float x[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t w = w0 + j * step;
                x[j] = red[(w < waves ? w : 0u) * E + e];
            }
#pragma unroll
            for (int j = 0; j < 4; j++) t += (w0 + j * step < waves) ? x[j] : 0.f;
        }
        return t;
    };
    // `total` of entry (r, c), held by the calling lane: to its destination
    auto finish = [&](uint32_t r, uint32_t c, float total, float partner, bool owner) {
        if (gated) {
            // partner = the total of column c + SUB / 2, the up column of gate column c
            const uint32_t feat = tile * 32u + part * (SUB / 2) + c;
            if (owner && c < SUB / 2 && r < m_rows && feat < ffn) out.swiglu[(size_t)r * ffn + feat] = gated_mul(out.gate_act, total, partner);
        } else {
            const uint32_t on = col_of(c);
            if (owner && r < m_rows && on < n) gemv4s_store_out(out, r, on, total);
        }
    };
    if constexpr (E <= 64) {
        // wave 0 finishes; the other waves are done
        if (wave != 0) return;
        constexpr int PARTS = 64 / E;
        const uint32_t e = lane % E, r = e / SUB, c = e % SUB;
        float total = sum_lane_groups<E>(sum_waves(e, lane / E, PARTS));   // (every lane of an entry holds it)
        const bool owner = lane < E;
        if (splits == 1) {
            finish(r, c, total, gated ? __shfl_down(total, SUB / 2, 64) : 0.f, owner);
            return;
        }
        // cross-workgroup split-K as in k_gemv4: park the partial, count arrivals, the last one adds in split order
        const uint32_t on = col_of(c);
        const bool valid = owner && r < m_rows && on < n;
        if (valid) __hip_atomic_store(&ws[((size_t)sp * m_rows + r) * n_pad + on], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): this wave's scratch stores have completed
        unsigned prev = 0;
        if (lane == 0) prev = __hip_atomic_fetch_add(&counters[st], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((unsigned)__builtin_amdgcn_readfirstlane((int)prev) != splits - 1) return;
        total = 0.f;
        if (valid)
            for (uint32_t s2 = 0; s2 < splits; s2++)
                total += __hip_atomic_load(&ws[((size_t)s2 * m_rows + r) * n_pad + on], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        finish(r, c, total, gated ? __shfl_down(total, SUB / 2, 64) : 0.f, owner);
        if (lane == 0) __hip_atomic_store(&counters[st], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    } else {
        // more entries than a wave has lanes (four rows on 32 columns, five to sixteen rows): a thread per entry, which
        // adds the waves' lane groups (64 / SUB reads in flight at a time)
        const uint32_t threads = waves * 64u;
        auto sum_wide = [&](uint32_t r, uint32_t c) {
            float v = 0.f;
            for (uint32_t w = 0; w < waves; w++)
#pragma unroll
                for (int q = 0; q < CPP; q++) v += red[(w * RL + r) * 64 + q * SUB + c];
            return v;
        };
        if (splits == 1) {
            for (uint32_t e = threadIdx.x; e < (uint32_t)E; e += threads) {
                const uint32_t r = e / SUB, c = e % SUB;
                if (gated) {
                    if (c < SUB / 2) finish(r, c, sum_wide(r, c), sum_wide(r, c + SUB / 2), true);
                } else {
                    finish(r, c, sum_wide(r, c), 0.f, true);
                }
            }
            return;
        }
        for (uint32_t e = threadIdx.x; e < (uint32_t)E; e += threads) {
            const uint32_t r = e / SUB, c = e % SUB, on = col_of(c);
            if (r < m_rows && on < n)
                __hip_atomic_store(&ws[((size_t)sp * m_rows + r) * n_pad + on], sum_wide(r, c), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): this wave's scratch stores have completed
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned prev = __hip_atomic_fetch_add(&counters[st], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = (prev == splits - 1);
        }
        __syncthreads();
        if (!s_last) return;
        auto parked = [&](uint32_t r, uint32_t on) {
            float v = 0.f;
            if (r < m_rows && on < n)
                for (uint32_t s2 = 0; s2 < splits; s2++)
                    v += __hip_atomic_load(&ws[((size_t)s2 * m_rows + r) * n_pad + on], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return v;
        };
        for (uint32_t e = threadIdx.x; e < (uint32_t)E; e += threads) {
            const uint32_t r = e / SUB, c = e % SUB;
            if (gated) {
                if (c < SUB / 2) finish(r, c, parked(r, col_of(c)), parked(r, col_of(c + SUB / 2)), true);
            } else {
                finish(r, c, parked(r, col_of(c)), 0.f, true);
            }
        }
        if (threadIdx.x == 0) __hip_atomic_store(&counters[st], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Argument order: what the address arithmetic of the first loads needs comes first, thirteen 32-bit words in all, which
// the build has the hardware preload into scalar registers at wave start (-amdgpu-kernarg-preload-count; thirteen is what
// the user scalar registers hold beside the argument pointer); the scratch pointers and the output description, a few
// hundred bytes that only the store needs, come last.  A wave that has to fetch an argument first starts its weight loads
// one round trip to the scalar cache later, and with one workgroup per CU nothing hides that -- hence also the packed
// word `cfg` (gemv4s_cfg: split factor, gated store, waves per workgroup, rows), which keeps the workgroup size out of
// the dispatch packet's hidden arguments, where a read of blockDim would fetch it from.
template <int SUB, int RL, bool AF32, bool ONE, bool REFL = false>
__global__ __launch_bounds__(1024) void k_gemv4s(const char *__restrict__ cw, const void *__restrict__ a_any,
                                                  const uint16_t *__restrict__ ref_scales, uint32_t cfg, uint32_t k,
                                                  uint32_t k_chunks, uint32_t sub_tiles, uint32_t cps, uint32_t n,
                                                  uint32_t n_pad, float *__restrict__ ws, unsigned *__restrict__ counters,
                                                  OutSpec out)
{
    gemv4s_body<SUB, RL, AF32, ONE, REFL>(cw, a_any, out, ws, counters, cfg, k, n, n_pad, k_chunks, sub_tiles, cps, ref_scales,
                                          nullptr);
}

// 16 columns, one row, up to NP passes per wave with all their loads issued up front.
template <bool AF32, bool REFL, int NP>
__global__ __launch_bounds__(1024) void k_gemv4s_upfront(const char *__restrict__ cw, const void *__restrict__ a_any,
                                                          const uint16_t *__restrict__ ref_scales, uint32_t cfg, uint32_t k,
                                                          uint32_t k_chunks, uint32_t sub_tiles, uint32_t cps, uint32_t n,
                                                          uint32_t n_pad, float *__restrict__ ws, unsigned *__restrict__ counters,
                                                          OutSpec out)
{
    gemv4s_body<16, 1, AF32, false, REFL, NP>(cw, a_any, out, ws, counters, cfg, k, n, n_pad, k_chunks, sub_tiles, cps, ref_scales,
                                              nullptr);
}

// The same kernel with a trace (twm_debug_trace; one row of f16 activations only): workgroup b writes four words at
// trace[4 b]: the 100 MHz clock at its start, after wave 0 has unpacked its passes, and at its end, and the hardware
// id of the CU it ran on.  A kernel of its own: reading the trace pointer first would put a second, dependent kernel
// argument fetch in front of every wave of the product kernel.
template <int SUB, bool ONE>
__global__ __launch_bounds__(1024) void k_gemv4s_traced(const char *__restrict__ cw, const void *__restrict__ a_any, OutSpec out,
                                                         float *__restrict__ ws, unsigned *__restrict__ counters,
                                                         uint32_t m_rows, uint32_t k, uint32_t n, uint32_t n_pad,
                                                         uint32_t k_chunks, uint32_t sub_tiles, uint32_t splits, uint32_t cps,
                                                         uint32_t *__restrict__ trace)
{
    uint32_t *tr = trace + 4u * blockIdx.x;
    if (threadIdx.x == 0) {
        tr[0] = (uint32_t)__builtin_amdgcn_s_memrealtime();
        tr[1] = 0u;
        // HW_ID (register 4): wave, SIMD, CU, SH, SE ids; XCC_ID (register 20): the XCD
        tr[3] = (__builtin_amdgcn_s_getreg((31 << 11) | 4) & 0xFFFFu) | (__builtin_amdgcn_s_getreg((3 << 11) | 20) << 16);
    }
    gemv4s_body<SUB, 1, false, ONE, false>(cw, a_any, out, ws, counters, gemv4s_cfg(splits, out.swiglu != nullptr, blockDim.x >> 6, m_rows),
                                           k, n, n_pad, k_chunks, sub_tiles, cps, nullptr, tr + 1);
    if (threadIdx.x == 0) tr[2] = (uint32_t)__builtin_amdgcn_s_memrealtime();
}

template <int SUB, int RL>
static hipError_t launch_gemv4s_t(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m,
                                  const OutSpec &out, float *ws, unsigned *counters, uint32_t waves, uint32_t splits, TraceBuf trace)
{
    uint32_t n_pad = w.n_tiles * kTileN;  // whole 64-column tiles
    uint32_t sub_tiles = n_pad / SUB;
    if (splits > 4095) splits = 4095;
    uint32_t cps = (w.k_chunks + splits - 1) / splits;
    splits = (w.k_chunks + cps - 1) / cps;
    uint32_t blocks = ((sub_tiles + 7) / 8) * 8 * splits;
    size_t lds = (size_t)waves * RL * (RL * SUB > 64 ? 64 : SUB) * sizeof(float);   // (five rows and more: every lane writes, see gemv4s_body)
    const bool one = (cps + 64 / SUB - 1) / (64 / SUB) <= waves;
    const bool runs = blocks <= 512;  // few workgroups per CU: a contiguous run of sub-tiles per XCD
#define TWM_S_LAUNCH(AF, ONEV)                                                                                          \
    hipLaunchKernelGGL((k_gemv4s<SUB, RL, AF, ONEV>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)w.cq, a,         \
                       (const uint16_t *)nullptr, gemv4s_cfg(splits, out.swiglu != nullptr, waves, m, runs), w.k, w.k_chunks, \
                       sub_tiles, cps, w.n, n_pad, ws, counters, out)
    if constexpr (RL == 1) {
        if (!a_f32 && trace.ptr && blocks <= trace.capacity) {
            if (one)
                hipLaunchKernelGGL((k_gemv4s_traced<SUB, true>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)w.cq, a, out,
                                   ws, counters, m, w.k, w.n, n_pad, w.k_chunks, sub_tiles, splits, cps, trace.ptr);
            else
                hipLaunchKernelGGL((k_gemv4s_traced<SUB, false>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)w.cq, a, out,
                                   ws, counters, m, w.k, w.n, n_pad, w.k_chunks, sub_tiles, splits, cps, trace.ptr);
            return hipGetLastError();
        }
    }
    if constexpr (SUB == 16 && RL == 1) {
        const uint32_t np = ((cps + 3) / 4 + waves - 1) / waves;  // passes per wave
        if ((np == 2 || np == 3) && !out.swiglu) {
#define TWM_S_UP(AF, NPV)                                                                                               \
    hipLaunchKernelGGL((k_gemv4s_upfront<AF, false, NPV>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)w.cq, a,    \
                       (const uint16_t *)nullptr, gemv4s_cfg(splits, false, waves, m, runs), w.k, w.k_chunks, sub_tiles, cps, \
                       w.n, n_pad, ws, counters, out)
            if (a_f32) { if (np == 2) TWM_S_UP(true, 2); else TWM_S_UP(true, 3); }
            else { if (np == 2) TWM_S_UP(false, 2); else TWM_S_UP(false, 3); }
#undef TWM_S_UP
            return hipGetLastError();
        }
    }
    if (a_f32) {
        if constexpr (RL <= 4) {
            if (one) TWM_S_LAUNCH(true, true);
            else TWM_S_LAUNCH(true, false);
        } else {
            return hipErrorInvalidValue;  // more than four rows: f16 activations only
        }
    } else {
        if (one) TWM_S_LAUNCH(false, true);
        else TWM_S_LAUNCH(false, false);
    }
#undef TWM_S_LAUNCH
    return hipGetLastError();
}

// sub = 32 or 16 columns per workgroup; waves 1 .. 16; out.swiglu set: the gated store of a paired weight.
// m <= 4 with f16 or f32 activations, m = 5 .. 16 with f16 activations.
hipError_t launch_gemv4s(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                         float *ws, unsigned *counters, uint32_t sub, uint32_t waves, uint32_t splits, TraceBuf trace)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    if (m > 16 || (m > 4 && a_f32) || splits == 0 || !w.cq) return hipErrorInvalidValue;
    if (out.swiglu && w.n % 64 != 0) return hipErrorInvalidValue;
    if (waves < 1 || waves > 16) return hipErrorInvalidValue;
    if (sub != 32 && sub != 16) return hipErrorInvalidValue;
#define TWM_S_CASE(SUBV)                                                                                       \
    if (sub == SUBV) {                                                                                         \
        if (m == 1) return launch_gemv4s_t<SUBV, 1>(s, w, a, a_f32, m, out, ws, counters, waves, splits, trace); \
        if (m == 2) return launch_gemv4s_t<SUBV, 2>(s, w, a, a_f32, m, out, ws, counters, waves, splits, trace); \
        if (m <= 4) return launch_gemv4s_t<SUBV, 4>(s, w, a, a_f32, m, out, ws, counters, waves, splits, trace); \
        if (m <= 8) return launch_gemv4s_t<SUBV, 8>(s, w, a, a_f32, m, out, ws, counters, waves, splits, trace); \
        return launch_gemv4s_t<SUBV, 16>(s, w, a, a_f32, m, out, ws, counters, waves, splits, trace);          \
    }
    TWM_S_CASE(32)
    TWM_S_CASE(16)
#undef TWM_S_CASE
    return hipErrorInvalidValue;
}

// M = 1 on the reference's arrays (no repack), f32 activations.
hipError_t launch_gemv4s_ref(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                             const float *a, float *c, float *ws, unsigned *counters, uint32_t sub, uint32_t waves,
                             uint32_t splits)
{
    if (n == 0) return hipSuccess;
    if (k == 0 || k % 32 != 0 || splits == 0) return hipErrorInvalidValue;
    if (waves < 1 || waves > 16 || (sub != 32 && sub != 16)) return hipErrorInvalidValue;
    const uint32_t n_pad = ((n + 63) / 64) * 64, sub_tiles = n_pad / sub;
    const uint32_t k_chunks = (k / 32 + 3) / 4;
    if (splits > 4095) splits = 4095;
    const uint32_t cps = (k_chunks + splits - 1) / splits;
    splits = (k_chunks + cps - 1) / cps;
    const uint32_t blocks = ((sub_tiles + 7) / 8) * 8 * splits;
    const size_t lds = (size_t)waves * sub * sizeof(float);
    const bool one = (cps + 64 / sub - 1) / (64 / sub) <= waves;
    OutSpec out;
    memset(&out, 0, sizeof out);
    out.count = 1;
    out.seg[0].ptr = c;
    out.seg[0].start = 0;
    out.seg[0].width = n;
#define TWM_S_REF(SUBV, ONEV)                                                                                          \
    hipLaunchKernelGGL((k_gemv4s<SUBV, 1, true, ONEV, true>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)packed, \
                       (const void *)a, scales, gemv4s_cfg(splits, false, waves, 1u), k, k_chunks, sub_tiles, cps, n, n_pad, ws,  \
                       counters, out)
    const uint32_t np = ((cps + 3) / 4 + waves - 1) / waves;  // passes per wave on 16 columns
    if (sub == 16 && (np == 2 || np == 3)) {
        if (np == 2)
            hipLaunchKernelGGL((k_gemv4s_upfront<true, true, 2>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)packed, (const void *)a,
                               scales, gemv4s_cfg(splits, false, waves, 1u), k, k_chunks, sub_tiles, cps, n, n_pad, ws, counters, out);
        else
            hipLaunchKernelGGL((k_gemv4s_upfront<true, true, 3>), dim3(blocks), dim3(waves * 64), lds, s, (const char *)packed, (const void *)a,
                               scales, gemv4s_cfg(splits, false, waves, 1u), k, k_chunks, sub_tiles, cps, n, n_pad, ws, counters, out);
        return hipGetLastError();
    }
    if (sub == 32) {
        if (one) TWM_S_REF(32, true);
        else TWM_S_REF(32, false);
    } else {
        if (one) TWM_S_REF(16, true);
        else TWM_S_REF(16, false);
    }
#undef TWM_S_REF
    return hipGetLastError();
}

}  // namespace twm

// Batched-decode kernel with the activations shared through LDS (M = 17 .. 32; M = 9 .. 16 on wide matrices and with
// f32 rows; M = 5 .. 8 with f32 rows on shallow K).
//
// Semantics, up to 16 rows: as the streaming kernel (reference order, crates/kernels/src/quantize.rs:1219-1238; M > 1
// has the meaning of gemm_q4_0, quantize.rs:1825-1858): per 32-deep group the products a * (q - 8) are summed in f32
// by one v_mfma_f32_16x16x32_f16 with a zero accumulator ((q - 8) and the f16 activations are exact operands), the
// group sum is scaled once by f32(scale) and added to the running f32 sum, groups in ascending order.
// 17 .. 32 rows: the same arithmetic on two 16-row blocks (eight f32 multiply-adds per tile and group after the
// MFMAs), so that a row's result does not depend on how many rows are batched with it.
// Option (RND): the reference's dequant-then-FP16-GEMM arithmetic (quantize.rs:534-571, :1825-1858), as the prefill
// kernel: the B operand is f16_rne(f32(scale) * (q - 8)), made by one packed f16 multiply, and the MFMAs accumulate
// over K directly (f32 activations still as two f16 terms).
//
// Why a second kernel: the streaming kernel keeps a whole chunk of activations (32 rows x 128 k) per wave in
// registers, twice, so only two waves fit a SIMD and each has one chunk of weights in flight; at 32 rows it is
// bound by the memory latency, not by HBM.  Here the waves of a slice (4, 8 or 12: one, two or three 64-column
// quads) advance through K together and share the activations through LDS:
//   A : the first 4 MT waves load four rows each of the chunk's 16 MT x 128 f16 tile (with four waves: MT times four
//       rows), three chunks ahead in four register slots, and write them to LDS one chunk ahead of their use (two
//       LDS buffers, 256-byte rows with XOR-swizzled 16-byte slots: conflict-free writes and operand reads); f32
//       activations are split beforehand into two f16 arrays (hi, lo) and both tiles are staged;
//   B : a wave owns TPW 16-column tiles; per chunk and tile 16 bytes of nibbles + 8 bytes of scales per lane,
//       three chunks ahead in four register slots (6 TPW registers each);
//   one barrier per chunk.
// A wave then needs 70 to 100 registers with three chunks of loads in flight (the streaming kernel: 170 with
// one).  A wave holds complete sums of its tiles (or a K-split's partial sums; k-slices of one workgroup add theirs
// through LDS at the end).
// Bound: HBM for the weights, read once; the activation tile comes from L2 once per workgroup and chunk and its
// requests share the CU's memory requests in flight with the weight stream, which is why more columns per
// workgroup pay where they do not unbalance the CUs (the host's cost model chooses).
#include "twm_device.h"

namespace twm {

namespace {

#define TWM_GLOBAL __attribute__((address_space(1)))

__device__ __forceinline__ const TWM_GLOBAL char *bt_scalar_base(const void *p, size_t byte_offset)
{
    uint64_t v = (uint64_t)p + byte_offset;
    asm("" : "+s"(v));  // a uniform base kept in scalar registers: loads take saddr + 32-bit lane offset
    return (const TWM_GLOBAL char *)v;
}

struct BtConsts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};

// eight nibbles of word w -> eight f16 values (q - 8), exact
__device__ __forceinline__ half8 bt_unpack(uint32_t w, const BtConsts &c)
{
    union { uint32_t u[4]; half2v h2[4]; half8 h; } r;
    const half2v b_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
    const half2v b_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    uint32_t w8 = w >> 8;
    r.u[0] = (w & c.mask_lo) | c.magic_lo;
    r.u[1] = (w & c.mask_hi) | c.magic_hi;
    r.u[2] = (w8 & c.mask_lo) | c.magic_lo;
    r.u[3] = (w8 & c.mask_hi) | c.magic_hi;
    r.h2[0] += b_lo;
    r.h2[1] += b_hi;
    r.h2[2] += b_lo;
    r.h2[3] += b_hi;
    return r.h;
}

constexpr int kBtRow = 128;  // halves per LDS row (256 bytes)
// register slots of a wave's loads (even: the LDS buffer of a chunk is slot & 1).  Three chunks in flight are enough:
// with six or eight slots 3584 -> 37888 at M = 32 read 23.5 / 24.9 us against 23.5 - 24.1, narrower matrices 4 - 8 % more
constexpr int kBtSlots = 4;

}  // namespace

// MT: 16-row blocks (1 or 2); TERMS: 1 = f16 activations, 2 = f32 activations as two f16 terms;
// TPW: tiles per wave.  TPW = 1: the workgroup owns one quad of tiles (64 columns), wave w tile w.
// TPW = 2: two quads (128 columns), wave w tiles (w & 1) and (w & 1) + 2 of quad w >> 1 -- in a paired gate/up
// weight a gate tile and the up tile of the same features, which the gated store needs in one lane.
// KS: k-slices per workgroup (1, 2, 4): the workgroup has 4 KS waves, slice s = wave / 4 takes the chunks s, s + KS, ...
// of the workgroup's k-range with its own LDS buffers, and the slices' sums are added through LDS at the end -- more
// waves per CU where the column quads alone are too few workgroups, without the partial-sum traffic of a K-split
// over workgroups.
// WPS: waves per slice (4, 8 or 12; TPW = 1 above 4): WPS / 4 quads per workgroup share one activation tile, so the
// tile is fetched from L2 once per 64 WPS / 4 columns -- its requests compete with the weight stream for the CU's
// memory requests in flight.  The first 4 MT waves of a slice stage the tile (four rows each, or MT times four with
// WPS = 4); the others issue the same load on one 16-byte address and write a spare LDS row, which keeps every
// wave's count of loads in flight the same.
template <int MT, bool RND, int TERMS, int TPW, int KS, int WPS>
__global__ __launch_bounds__(64 * WPS * KS) void k_batch(const uint4v *__restrict__ qw, const uint2v *__restrict__ sc,
                                                const void *__restrict__ a_any, uint32_t m_rows, uint32_t k, uint32_t n,
                                                uint32_t n_tiles, uint32_t k_chunks, uint32_t chunks_per_split,
                                                uint32_t lo_offset, float *__restrict__ partials, OutSpec out)
{
    constexpr bool kRounded = RND;           // weights rounded to f16 as in the reference's dequant-then-FP16-GEMM route (option)
    constexpr int S = kBtSlots;              // register slots: chunk kc lives in slot kc % S, S - 1 chunks are in flight
    constexpr int kTile = 16 * MT * kBtRow;  // halves of one term's tile
    constexpr int kBuf = TERMS * kTile;      // halves of one LDS buffer
    static_assert(TPW == 1 || WPS == 4, "two tiles per wave: four waves per slice");
    static_assert(64 * WPS * KS <= 1024, "workgroup size");
    constexpr int NVW = (4 * MT + WPS - 1) / WPS;  // A loads per wave and chunk (four rows of the tile each)
    constexpr int kSpare = NVW * WPS > 4 * MT ? 512 : 0;  // halves: where the waves without a part of the tile write
    __shared__ __attribute__((aligned(16))) _Float16 lds_all[KS * (2 * kBuf + kSpare)];

    const uint32_t wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wave = wave_all % WPS, slice = wave_all / WPS;  // wave: index inside the slice
    _Float16 *a_lds = lds_all + slice * (2 * kBuf + kSpare);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t c = lane & 15u, kb = lane >> 4;
    const uint32_t kc0 = blockIdx.y * chunks_per_split;
    const uint32_t nchunks = k_chunks - kc0 < chunks_per_split ? k_chunks - kc0 : chunks_per_split;
    const uint32_t last = nchunks - 1;
    // this slice's chunks (relative to kc0): slice, slice + KS, ...; my_count of them (0 when the range is shorter
    // than the slice index); every slice walks `steps` steps, the barriers being common
    const uint32_t my_count = nchunks > slice ? (nchunks - slice + KS - 1) / KS : 0u;
    const uint32_t my_last = my_count ? slice + (my_count - 1u) * KS : last;
    const uint32_t steps = (nchunks + KS - 1) / KS;

    // this wave's tiles; tiles past the end replay the last tile and are never stored
    uint32_t tile_of[TPW], nt[TPW];
#pragma unroll
    for (int i = 0; i < TPW; i++) {
        tile_of[i] = TPW == 1 ? blockIdx.x * (uint32_t)WPS + wave : (blockIdx.x * 2u + (wave >> 1)) * 4u + (wave & 1u) + 2u * i;
        nt[i] = tile_of[i] < n_tiles ? tile_of[i] : n_tiles - 1;
    }

    BtConsts dq = {0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(dq.mask_lo), "+s"(dq.mask_hi), "+v"(dq.magic_lo), "+v"(dq.magic_hi));

    float4v acc[MT][TPW];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int i = 0; i < TPW; i++) acc[mt][i] = float4v{0.f, 0.f, 0.f, 0.f};

    // ---- A tile: the tile's 4 MT row quads (four rows each) go to the slice's waves in turn, load j of wave w takes
    // quad w + j WPS; lane L takes row L / 16 of the quad and the row's vector (L % 16) ^ (row % 16) (8 halves) and
    // writes it to slot L % 16 of that row, so that slot s of row r holds vector s ^ (r % 16).  Rows past m_rows replay
    // the last row (never stored); vectors past K replay the chunk's first vector of the row (the padded weights
    // there are zero).  A load past the last quad reads one 16-byte address with all lanes and lands in the spare row.
    uint32_t a_vec[NVW], a_off[NVW], a_dst[NVW];
#pragma unroll
    for (int j = 0; j < NVW; j++) {
        const uint32_t quad = wave + (uint32_t)j * WPS;
        const bool real = quad < 4u * MT;
        uint32_t row = real ? 4u * quad + (lane >> 4) : 0u;
        a_vec[j] = real ? (lane & 15u) ^ (row & 15u) : 0u;
        row = row < m_rows ? row : m_rows - 1;
        a_off[j] = (row * k + a_vec[j] * 8u) * 2u;
        a_dst[j] = real ? 4u * quad * kBtRow + lane * 8u : 2u * kBuf + (lane & 63u) * 8u;  // halves, inside a buffer / the spare row
    }
    uint4v ar[S][TERMS][NVW];
    uint4v wq[S][TPW];
    uint2v ws[S][TPW];
    const uint32_t q_off = lane * 16u, s_off = c * 8u;
    auto load_chunk = [&](int slot, uint32_t kc) {  // kc relative to kc0; the same loads in every call
        const uint32_t kg = kc0 + kc;
#pragma unroll
        for (int t = 0; t < TERMS; t++) {
            const TWM_GLOBAL char *src = bt_scalar_base(a_any, (size_t)t * lo_offset + (size_t)kg * 256u);
#pragma unroll
            for (int j = 0; j < NVW; j++) {
                const uint32_t back = kg * 128u + a_vec[j] * 8u < k ? 0u : a_vec[j] * 16u;
                ar[slot][t][j] = *(const TWM_GLOBAL uint4v *)(src + (a_off[j] - back));
            }
        }
#pragma unroll
        for (int i = 0; i < TPW; i++) {
            const size_t tile = (size_t)kg * n_tiles + nt[i];
            // (weights are read once per launch: non-temporal)
            wq[slot][i] = __builtin_nontemporal_load((const TWM_GLOBAL uint4v *)(bt_scalar_base(qw, tile * 1024u) + q_off));
            ws[slot][i] = __builtin_nontemporal_load((const TWM_GLOBAL uint2v *)(bt_scalar_base(sc, tile * 128u) + s_off));
        }
    };
    auto stage_a = [&](int slot, int buf) {  // this wave's part of a tile: registers -> LDS
#pragma unroll
        for (int t = 0; t < TERMS; t++)
#pragma unroll
            for (int j = 0; j < NVW; j++) {
                // (the spare row lies behind both buffers: its offset takes neither the buffer nor the term)
                const uint32_t at = a_dst[j] < 2u * kBuf ? buf * kBuf + t * kTile + a_dst[j] : a_dst[j];
                *(uint4v *)(a_lds + at) = ar[slot][t][j];
            }
    };

    uint32_t rd_off[4];  // row c of a row block, vector 4 g + kb of the chunk -> slot (4 g + kb) ^ c
#pragma unroll
    for (int g = 0; g < 4; g++) rd_off[g] = c * kBtRow + (((4u * g + kb) ^ c) * 8u);

    auto compute = [&](int slot, int bufi) {
        const _Float16 *buf = a_lds + bufi * kBuf;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            half8 af[TERMS][MT];
#pragma unroll
            for (int t = 0; t < TERMS; t++)
#pragma unroll
                for (int mt = 0; mt < MT; mt++) af[t][mt] = *(const half8 *)(buf + t * kTile + mt * 16 * kBtRow + rd_off[g]);
#pragma unroll
            for (int i = 0; i < TPW; i++) {
                const half8 bf = bt_unpack(wq[slot][i][g], dq);
                union { uint32_t u; half2v h; } pair;
                pair.u = ws[slot][i][g >> 1];
                const _Float16 scale16 = pair.h[g & 1];
                if constexpr (kRounded) {
                    // B = f16(scale * (q - 8)): one packed multiply per two weights, and the MFMAs add up K directly
                    union { half8 h; half2v h2[4]; } bw;
                    bw.h = bf;
                    const half2v s2 = {scale16, scale16};
#pragma unroll
                    for (int j = 0; j < 4; j++) bw.h2[j] *= s2;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        acc[mt][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[0][mt], bw.h, acc[mt][i], 0, 0, 0);
                        if constexpr (TERMS == 2)
                            acc[mt][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[1][mt], bw.h, acc[mt][i], 0, 0, 0);
                    }
                    continue;
                }
                const float scale = (float)scale16;
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    float4v d = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[0][mt], bf, float4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    if constexpr (TERMS == 2) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[1][mt], bf, d, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[mt][i][r] += d[r] * scale;
                }
            }
        }
    };

    // One chunk (slot = kc % S, LDS buffer kc % 2): loads of chunk kc + S - 1 go out first; the chunk is computed from its
    // LDS buffer and its weight slot; then this wave's part of A tile kc + 1 goes from its registers to the other
    // buffer (every wave finished reading that buffer before the previous barrier); the barrier makes the tile
    // complete.  Past the end the last chunk is loaded again and never used, so that every step issues the same loads
    // (the compiler's count of loads in flight stays exact).
    auto chunk_of = [&](uint32_t i) {  // the slice's i-th chunk, clamped to its last one
        const uint32_t rel = slice + i * KS;
        return rel < my_last ? rel : my_last;
    };
    auto step = [&](int slot, uint32_t i) {
        load_chunk((slot + S - 1) % S, chunk_of(i + (uint32_t)(S - 1)));
        if (KS == 1 || i < my_count) compute(slot, slot & 1);  // (uniform over the wave)
        stage_a((slot + 1) % S, (slot + 1) & 1);
        __syncthreads();
    };

#pragma unroll
    for (int s = 0; s < S - 1; s++) load_chunk(s, chunk_of((uint32_t)s));
    stage_a(0, 0);
    __syncthreads();
    uint32_t i0 = 0;
    for (; i0 + S <= steps; i0 += S) {
#pragma unroll
        for (int s = 0; s < S; s++) step(s, i0 + s);
    }
#pragma unroll
    for (int s = 0; s < S - 1; s++)
        if (i0 + s < steps) step(s, i0 + s);  // (uniform over the workgroup)

    if constexpr (KS > 1) {
        // the slices' sums, added in slice order through LDS (the staging buffers are idle: the last step ended with
        // a barrier); slice 0 stores
        constexpr int kRegs = MT * TPW * 4;
        float *red = (float *)lds_all;  // [KS - 1][WPS waves][kRegs][64 lanes]
        if (slice > 0) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int t = 0; t < TPW; t++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        red[(((slice - 1u) * WPS + wave) * kRegs + (mt * TPW + t) * 4 + r) * 64u + lane] = acc[mt][t][r];
        }
        __syncthreads();
        if (slice > 0) return;
#pragma unroll
        for (int sl = 1; sl < KS; sl++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int t = 0; t < TPW; t++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        acc[mt][t][r] += red[(((sl - 1) * WPS + wave) * kRegs + (mt * TPW + t) * 4 + r) * 64u + lane];
    }

    // ---- store: lane (c, kb) holds rows 16 mt + 4 kb + r of column 16 tile + c
    const uint32_t n_ld = n_tiles * 16u;
    if (out.row_scale && !partials) {
        // f32 rows that were scaled into the f16 range: their sums back, before bias and gate (the K-split's sum kernel
        // does it for partial sums).  A step of its own ahead of the stores: inside the store loops it moved the main
        // loop's prefetches of one variant down to their use.
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t row = 16u * mt + 4u * kb + r;
                const float rs = out.row_scale[row < m_rows ? row : m_rows - 1u];
#pragma unroll
                for (int i = 0; i < TPW; i++) acc[mt][i][r] *= rs;
            }
    }
    if (partials) {
        float *dst = partials + (size_t)blockIdx.y * m_rows * n_ld;
#pragma unroll
        for (int i = 0; i < TPW; i++) {
            if (tile_of[i] >= n_tiles) continue;
            const uint32_t on = tile_of[i] * 16u + c;
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const uint32_t row = 16u * mt + 4u * kb + r;
                    if (row < m_rows) dst[(size_t)row * n_ld + on] = acc[mt][i][r];
                }
        }
        return;
    }
    if constexpr (TPW == 2) {
        if (out.swiglu) {
            // paired gate/up weight: tile 0 of this wave holds gate columns, tile 1 the up columns of the same features
            if (tile_of[1] >= n_tiles) return;
            const uint32_t ffn = n >> 1, feat = paired_feature(tile_of[0] * 16u + c);
            if (feat >= ffn) return;
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const uint32_t row = 16u * mt + 4u * kb + r;
                    if (row < m_rows) out.swiglu[(size_t)row * ffn + feat] = gated_mul(out.gate_act, acc[mt][0][r], acc[mt][1][r]);
                }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < TPW; i++) {
        if (tile_of[i] >= n_tiles) continue;
        const uint32_t on = tile_of[i] * 16u + c;
        if (on >= n) continue;
#pragma unroll
        for (uint32_t sg = 0; sg < kMaxSegs; sg++) {
            if (sg >= out.count) continue;
            const uint32_t rel = on - out.seg[sg].start;
            if (rel >= out.seg[sg].width) continue;
            const float b = out.seg[sg].bias ? out.seg[sg].bias[rel] : 0.f;
            const bool has_b = out.seg[sg].bias != nullptr;
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const uint32_t row = 16u * mt + 4u * kb + r;
                    if (row < m_rows) out.seg[sg].ptr[(size_t)row * out.seg[sg].width + rel] = has_b ? acc[mt][i][r] + b : acc[mt][i][r];
                }
        }
    }
}

template <int MT, bool RND, int TERMS, int TPW, int KS, int WPS = 4>
static hipError_t launch_batch_t(hipStream_t s, const WeightView &w, const void *a, uint32_t m, const OutSpec &out,
                                 uint32_t splits, float *partials, uint32_t lo_offset)
{
    uint32_t cps = (w.k_chunks + splits - 1) / splits;
    splits = (w.k_chunks + cps - 1) / cps;  // no empty split
    const uint32_t quads = w.n_tiles / 4;   // n_tiles is a multiple of 4
    constexpr uint32_t kQuadsPerGroup = WPS * TPW / 4;
    dim3 grid((quads + kQuadsPerGroup - 1) / kQuadsPerGroup, splits);
    hipLaunchKernelGGL((k_batch<MT, RND, TERMS, TPW, KS, WPS>), grid, dim3(64 * WPS * KS), 0, s, (const uint4v *)w.qw, (const uint2v *)w.sc, a,
                       m, w.k, w.n, w.n_tiles, w.k_chunks, cps, lo_offset, splits > 1 ? partials : nullptr, out);
    if (splits > 1) {
        hipError_t e = launch_splitk_reduce(s, partials, out, m, w.n, w.n_tiles * 16, splits);
        if (e != hipSuccess) return e;
    }
    return hipGetLastError();
}

// Four k-slices (sixteen waves) only with one tile per wave (register file) and not for the 32-row two-term variant
// (its staging buffers would need 128 KB of LDS); otherwise two.
template <int MT, bool RND, int TERMS, int TPW>
static hipError_t launch_batch_slices(hipStream_t s, const WeightView &w, const void *a, uint32_t m, const OutSpec &out,
                                      uint32_t splits, uint32_t k_slices, uint32_t quads_per_group, float *partials,
                                      uint32_t lo_offset)
{
    if constexpr (TPW == 1) {
        // two or three quads per workgroup (eight or twelve waves per slice; two slices only with eight)
        if (quads_per_group == 3) return launch_batch_t<MT, RND, TERMS, 1, 1, 12>(s, w, a, m, out, splits, partials, lo_offset);
        if (quads_per_group == 2) {
            if constexpr (!(MT == 2 && TERMS == 2)) {
                if (k_slices >= 2) return launch_batch_t<MT, RND, TERMS, 1, 2, 8>(s, w, a, m, out, splits, partials, lo_offset);
            }
            return launch_batch_t<MT, RND, TERMS, 1, 1, 8>(s, w, a, m, out, splits, partials, lo_offset);
        }
    }
    if constexpr (TPW == 1 && !(MT == 2 && TERMS == 2)) {
        if (k_slices == 4) return launch_batch_t<MT, RND, TERMS, TPW, 4>(s, w, a, m, out, splits, partials, lo_offset);
    }
    if (k_slices >= 2) return launch_batch_t<MT, RND, TERMS, TPW, 2>(s, w, a, m, out, splits, partials, lo_offset);
    return launch_batch_t<MT, RND, TERMS, TPW, 1>(s, w, a, m, out, splits, partials, lo_offset);
}

// M <= 32.  quads_per_group: 1, 2 or 3 column quads per workgroup sharing one activation tile (one tile per wave; with
// two tiles per wave the workgroup owns two quads anyway).  rounded: weights rounded to f16 and accumulated over K by
// the MFMAs (always on the 32-row variant, so that one call runs one arithmetic whatever its last block's height);
// otherwise the exact per-group f32 scaling.  tiles_per_wave: 1 or 2 (a gated store without split-K needs 2).  `scratch` holds, for f32 activations,
// their two f16 terms (2 x M x K halves) and after them the split-K partials (splits x M x (n_tiles * 16) floats);
// the split factor is cut to what fits.
hipError_t launch_batch(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out_in,
                        uint32_t splits, uint32_t tiles_per_wave, uint32_t k_slices, uint32_t quads_per_group,
                        bool rounded, float *scratch, size_t scratch_bytes)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    if (m > 32 || w.k_chunks == 0 || w.n_tiles % 4 != 0) return hipErrorInvalidValue;
    if (tiles_per_wave != 1 && tiles_per_wave != 2) return hipErrorInvalidValue;
    if (quads_per_group < 1 || quads_per_group > 3) return hipErrorInvalidValue;
    if (k_slices != 1 && k_slices != 2 && k_slices != 4) return hipErrorInvalidValue;
    float *partials = scratch;
    size_t partial_bytes = scratch ? scratch_bytes : 0;
    uint32_t lo_offset = 0;
    OutSpec out = out_in;
    if (a_f32) {
        // the rows' power-of-two factors (256 bytes), their two f16 terms, then the partial sums
        size_t term_bytes = (((size_t)m * w.k * 2) + 255) & ~(size_t)255;
        if (!scratch || scratch_bytes < 256 + 2 * term_bytes || term_bytes > 0x7FFFFFFFu) return hipErrorInvalidValue;
        float *row_scale = scratch;
        _Float16 *hi = (_Float16 *)((char *)scratch + 256), *lo = (_Float16 *)((char *)scratch + 256 + term_bytes);
        hipError_t e = launch_f32_rows_to_f16(s, (const float *)a, hi, lo, row_scale, m, w.k);
        if (e != hipSuccess) return e;
        a = hi;
        out.row_scale = row_scale;
        lo_offset = (uint32_t)term_bytes;
        partials = (float *)((char *)scratch + 256 + 2 * term_bytes);
        partial_bytes = scratch_bytes - 256 - 2 * term_bytes;
    }
    if (splits < 1) splits = 1;
    size_t per_split = (size_t)m * w.n_tiles * 16 * 4;
    if (!partials || per_split == 0) splits = 1;
    else if (splits > partial_bytes / per_split) splits = (uint32_t)(partial_bytes / per_split);
    if (splits < 1) splits = 1;
    if (w.k_chunks < splits) splits = w.k_chunks;
    if (out.swiglu && splits == 1) tiles_per_wave = 2;
#define TWM_BATCH_CASE(MT, R, T, P) return launch_batch_slices<MT, R, T, P>(s, w, a, m, out, splits, k_slices, quads_per_group, partials, lo_offset)
    if (rounded) {
        if (tiles_per_wave == 2) { if (a_f32) TWM_BATCH_CASE(2, true, 2, 2); TWM_BATCH_CASE(2, true, 1, 2); }
        if (a_f32) TWM_BATCH_CASE(2, true, 2, 1);
        TWM_BATCH_CASE(2, true, 1, 1);
    }
    if (m <= 16) {
        if (tiles_per_wave == 2) { if (a_f32) TWM_BATCH_CASE(1, false, 2, 2); TWM_BATCH_CASE(1, false, 1, 2); }
        if (a_f32) TWM_BATCH_CASE(1, false, 2, 1);
        TWM_BATCH_CASE(1, false, 1, 1);
    }
    if (tiles_per_wave == 2) { if (a_f32) TWM_BATCH_CASE(2, false, 2, 2); TWM_BATCH_CASE(2, false, 1, 2); }
    if (a_f32) TWM_BATCH_CASE(2, false, 2, 1);
    TWM_BATCH_CASE(2, false, 1, 1);
#undef TWM_BATCH_CASE
}

}  // namespace twm

// Building blocks of the one-lane-per-column GEMV (M <= 4): nibble unpack, the chunk's register set, its
// loads and its 32 chained 4x4x4 MFMAs, in the 64-column form (twm_gemv4.hip) and the sub-tile form
// (twm_gemv4s.hip, twm_moe.hip); everything is force-inlined.
#pragma once
#include "twm_device.h"

namespace twm {

typedef _Float16 half4v __attribute__((ext_vector_type(4)));

struct Gemv4Consts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};

// Weights are read once per launch: a non-temporal load keeps them from displacing the activations (and the
// next launch's working set) in the caches.  3584 -> 37888 at M = 1: 14.8 against 15.8 us; LM head 48.5 against 51.
template <class T>
__device__ __forceinline__ T ld_once(const T *p)
{
    return __builtin_nontemporal_load(p);
}

__device__ __forceinline__ Gemv4Consts make_gemv4_consts()
{
    // opaque to the optimiser so that (w & mask) | magic becomes one v_and_or_b32
    Gemv4Consts c = {0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(c.mask_lo), "+s"(c.mask_hi), "+v"(c.magic_lo), "+v"(c.magic_hi));
    return c;
}

// eight nibbles -> eight exact f16 values q - 8 in k order, as two half4 (k 0..3 and k 4..7)
__device__ __forceinline__ void gemv4_dequant_word(uint32_t w, const Gemv4Consts &c, half4v &lo4, half4v &hi4)
{
    union { uint32_t u[2]; half2v h2[2]; half4v h; } a, b;
    uint32_t w8 = w >> 8;
    a.u[0] = (w & c.mask_lo) | c.magic_lo;    // 1024 + q of k0, k1
    a.u[1] = (w & c.mask_hi) | c.magic_hi;    //   64 + q of k2, k3
    b.u[0] = (w8 & c.mask_lo) | c.magic_lo;   // k4, k5
    b.u[1] = (w8 & c.mask_hi) | c.magic_hi;   // k6, k7
    const half2v b_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
    const half2v b_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    a.h2[0] += b_lo;
    a.h2[1] += b_hi;
    b.h2[0] += b_lo;
    b.h2[1] += b_hi;
    lo4 = a.h;
    hi4 = b.h;
}

// RG = row groups of four: rows 4 .. 4*RG-1 repeat the MFMA chain on the same unpacked weights (f16 rows only).
template <int NT, int RG = 1>
struct Chunk4 {
    uint4v wq[NT][4];  // [tile][group in chunk]: this lane's column, 32 nibbles
    uint2v sc[NT];     // four f16 scales
    uint4v a[RG];      // activations: row 4*rg + lane%4, k-piece lane/4 (8 halves)
    uint4v a_lo;       // f32 activations only: the f16 residuals a - f16(a) of the same eight values
    float a_inv[4];    // f32 activations only: what the sums of the four A rows are multiplied by (f32_terms_range)
};

// f32 activations enter the f16 MFMA as two terms, a = f16(a) + f16(a - f16(a)) (about 22 significant bits;
// the subtraction is exact), so that a caller's f32 values are not silently cut to 11 bits.  Values beyond the
// f16 range are scaled into it first, a chunk of a wave at a time (f32_terms_range).
__device__ __forceinline__ void split_f32x8(const float (&v)[8], uint4v &hi, uint4v &lo)
{
    union { half8 h; uint4v u; } ch, cl;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        _Float16 h = (_Float16)v[i];
        ch.h[i] = h;
        cl.h[i] = (_Float16)(v[i] - (float)h);
    }
    hi = ch.u;
    lo = cl.u;
}

// f32 activations beyond the f16 range.  The wave's values of one chunk (or pass) are about to be taken as f16 terms.
// Lanes with the same lane % 4 hold the same activation row (one row of the MFMA's A operand); when any value of
// the wave exceeds the largest f16, every such row scales its values by a power of two of its own that brings its
// largest below 2^15 (exact), and inv[i] is what the sums of A row i are multiplied by afterwards (exact as well): the
// results come out as with unbounded terms.  A row whose values in the wave are all below 2^-6 is scaled up the same
// way, so that its residual terms do not fall into the f16 subnormals.  In range every factor is 1 and nothing is
// touched, at the price of a maximum over the lane's values and one vote per call.  (Infinities and NaNs stay what they are.)
// ONE_ROW: every lane of the wave holds values of the same activation row: one factor for the wave.
template <int NV, bool ONE_ROW = false>
__device__ __forceinline__ void f32_terms_range(float (&v)[NV], float (&inv)[4])
{
    float m = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) m = fmaxf(m, fabsf(v[i]));
#pragma unroll
    for (int i = 0; i < 4; i++) inv[i] = 1.f;
    // (a lane whose values are all small, below 2^-6, votes too: when that holds for the row's whole stretch, the residual
    // terms, 2^-11 of their values, would fall into the f16 subnormals (below 2^-14), and the stretch is scaled up instead)
    if (__builtin_amdgcn_ballot_w64(!(m <= 65000.f) || (m < 0.015625f && m > 0.f)) == 0) return;
    if (!(m == m)) m = __builtin_inff();  // (fmaxf drops a NaN; the vote saw it through the negated comparison)
#pragma unroll
    for (int off = 32; off >= (ONE_ROW ? 1 : 4); off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));   // over the lanes of this row
    float mine = 1.f;
    if (m > 16384.f || (m < 0.015625f && m >= 1e-30f)) {
        const uint32_t e = (__float_as_uint(m) >> 23) & 0xFFu;       // biased exponent of the row's largest value
        const float down = __uint_as_float((254u + 14u - e) << 23);   // 2^(14 - (e - 127))
#pragma unroll
        for (int i = 0; i < NV; i++) v[i] *= down;
        mine = __uint_as_float((e - 14u) << 23);                     // 2^((e - 127) - 14)
    }
    if (ONE_ROW) {
#pragma unroll
        for (int i = 0; i < 4; i++) inv[i] = mine;
        return;
    }
    const int quad = (int)(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)) & ~3u);
#pragma unroll
    for (int i = 0; i < 4; i++) inv[i] = __shfl(mine, quad + i, 64);
}

template <int P>
__device__ __forceinline__ float4v mfma_piece(half4v a, half4v b, float4v c)
{
    return __builtin_amdgcn_mfma_f32_4x4x4f16(a, b, c, 4, P, 0);  // CBSZ = 4: all 16 blocks use block P's A
}

// Loads chunk kc of NT tiles (wbase[t] = this tile's block 0) and the lane's 16 bytes of activations:
// lane l reads row arow, halves [kc*128 + apiece, +8).
// Term modes of the activations: one f16 term; two terms as two MFMA passes (a_lo holds the second); or, for
// at most two rows, two terms packed into the four MFMA rows (lane l: row (l % 4) / 2, term l % 2), which
// costs no extra MFMA: the 4x4x4 instruction computes four rows anyway.
enum { kTermsOne = 0, kTermsTwoPasses = 1, kTermsRowPacked = 2, kTermsOneRow = 3, kTermsOneRowF32 = 4 };
// kTermsOneRow (sub-tile kernels, one row of f16 activations): a lane loads ONE 8-wide piece of its chunk instead of the
// 64 / SUB pieces its MFMA block supplies, and the unpack hands the pieces round inside each quad of lanes
// (gemv4s_load_a, gemv4s_compute).
// kTermsOneRowF32: the same for one row of f32 activations: a lane loads and splits ONE piece (a and a_lo hold its two
// f16 terms), and the unpack hands both terms round the quad: lanes 0 and 2 of a quad take the first term, lanes 1 and 3
// the residual, so that rows 0 and 1 of the MFMA's A block are the two terms (rows 2 and 3 repeat them, unused).
template <bool AF32, int RL>
constexpr int gemv4_terms() { return AF32 ? (RL <= 2 ? kTermsRowPacked : kTermsTwoPasses) : kTermsOne; }

// arow: the activation row this lane reads (see the term modes); lane_is_lo: row-packed mode, this lane holds
// the residual term
template <int NT, bool AF32, int TERMS = AF32 ? kTermsTwoPasses : kTermsOne, int RG = 1>
__device__ __forceinline__ void gemv4_load_chunk(Chunk4<NT, RG> &r, const char *(&wbase)[NT], uint32_t kc,
                                                 uint32_t lane16, uint32_t lane8, const void *a_any, uint32_t arow,
                                                 uint32_t apiece, uint32_t k, bool lane_is_lo = false, uint32_t m_rows = 0)
{
    static_assert(RG == 1 || !AF32, "more than four rows: f16 activations only");
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const char *blk = wbase[t] + (size_t)kc * kColBlockBytes;
#pragma unroll
        for (int g = 0; g < 4; g++) r.wq[t][g] = ld_once((const uint4v *)(blk + g * 1024u + lane16));
        r.sc[t] = ld_once((const uint2v *)(blk + lane8));
    }
    uint32_t k0 = kc * 128u + apiece;
    if (k0 > k - 8u) k0 = k - 8u;  // only the zero-padded groups of a last partial chunk get here
    if (AF32) {
        const float4 *p = (const float4 *)((const float *)a_any + (size_t)arow * k + k0);
        float4 x = p[0], y = p[1];
        float v[8] = {x.x, x.y, x.z, x.w, y.x, y.y, y.z, y.w};
        f32_terms_range(v, r.a_inv);
        split_f32x8(v, r.a[0], r.a_lo);
        if (TERMS == kTermsRowPacked) {
#pragma unroll
            for (int i = 0; i < 4; i++) r.a[0][i] = lane_is_lo ? r.a_lo[i] : r.a[0][i];
        }
    } else {
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            uint32_t row = arow + 4u * rg;
            if (RG > 1 && row > m_rows - 1u) row = m_rows - 1u;
            r.a[rg] = *(const uint4v *)((const _Float16 *)a_any + (size_t)row * k + k0);
        }
    }
}

// The same chunk taken from the reference's own arrays, without a repack (packed u8 [G][N][16], scales f16
// [G][N], crates/kernels/src/quantize.rs:892-907): lane = column, so a wave still reads 1 KiB contiguous per
// group.  Columns past n and groups past the end replay the last valid one with scale 0 (weight exactly 0).
// The nibbles are in their natural order here, which the mask-and-magic unpack turns into the k order
// (0,4,1,5 | 2,6,3,7) per eight; the f32 activations (one row) are converted into that same order.
template <int NT>
__device__ __forceinline__ void gemv4_load_chunk_ref(Chunk4<NT, 1> &r, const char *packed, const uint16_t *scales,
                                                     uint32_t tile0, uint32_t kc, uint32_t lane, uint32_t n,
                                                     uint32_t groups, const float *a, uint32_t apiece, uint32_t k,
                                                     bool lane_is_lo)
{
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const uint32_t col = (tile0 + t) * 64u + lane;
        const uint32_t colc = col < n ? col : n - 1u;
        uint32_t sb[4], keep[4];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t gg = kc * 4u + g;
            const uint32_t ggc = gg < groups ? gg : groups - 1u;
            const size_t idx = (size_t)ggc * n + colc;
            r.wq[t][g] = ld_once((const uint4v *)(packed + idx * 16u));
            sb[g] = ld_once(scales + idx);
            keep[g] = (gg < groups && col < n) ? 0xFFFFu : 0u;
        }
        // (dead groups masked after the packing: a select on a freshly loaded value becomes a branch around the load)
        r.sc[t] = uint2v{(sb[0] | (sb[1] << 16)) & (keep[0] | (keep[1] << 16)), (sb[2] | (sb[3] << 16)) & (keep[2] | (keep[3] << 16))};
    }
    uint32_t k0 = kc * 128u + apiece;
    if (k0 > k - 8u) k0 = k - 8u;
    const float4 *p = (const float4 *)(a + k0);
    float4 x = p[0], y = p[1];
    float v[8] = {x.x, y.x, x.y, y.y, x.z, y.z, x.w, y.w};
    f32_terms_range(v, r.a_inv);
    split_f32x8(v, r.a[0], r.a_lo);
#pragma unroll
    for (int i = 0; i < 4; i++) r.a[0][i] = lane_is_lo ? r.a_lo[i] : r.a[0][i];  // one row: row-packed terms
}

// acc[t][row] += f32(scale) * (sum over the group of A * (q - 8)) for the four groups of the chunk
template <int NT, int RL, int TERMS = kTermsOne>
__device__ __forceinline__ void gemv4_compute_chunk(const Chunk4<NT, (RL + 3) / 4> &r, const Gemv4Consts &dq, float (&acc)[NT][RL])
{
    constexpr bool A2 = TERMS == kTermsTwoPasses;
    constexpr int RG = (RL + 3) / 4;
    static_assert(TERMS != kTermsRowPacked || RL <= 2, "row-packed terms hold at most two rows");
    static_assert(RG == 1 || TERMS == kTermsOne, "more than four rows: one f16 term");
    union { uint4v u; half4v h[2]; } av[RG], al;
#pragma unroll
    for (int rg = 0; rg < RG; rg++) av[rg].u = r.a[rg];  // h[0] = k 0..3 of the lane's piece, h[1] = k 4..7
    if (A2) al.u = r.a_lo;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        union { uint2v u; _Float16 h[4]; } sv;
        sv.u = r.sc[t];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            float4v d[RG];
#pragma unroll
            for (int rg = 0; rg < RG; rg++) d[rg] = float4v{0.f, 0.f, 0.f, 0.f};
            half4v lo4, hi4;
#define TWM_PIECE(W, PIECE)                                       \
    gemv4_dequant_word(r.wq[t][g][W], dq, lo4, hi4);              \
    _Pragma("unroll") for (int rg = 0; rg < RG; rg++) {           \
        d[rg] = mfma_piece<PIECE>(av[rg].h[0], lo4, d[rg]);       \
        d[rg] = mfma_piece<PIECE>(av[rg].h[1], hi4, d[rg]);       \
    }                                                             \
    if (A2) {                                                     \
        d[0] = mfma_piece<PIECE>(al.h[0], lo4, d[0]);             \
        d[0] = mfma_piece<PIECE>(al.h[1], hi4, d[0]);             \
    }
            if (g == 0) { TWM_PIECE(0, 0) TWM_PIECE(1, 1) TWM_PIECE(2, 2) TWM_PIECE(3, 3) }
            if (g == 1) { TWM_PIECE(0, 4) TWM_PIECE(1, 5) TWM_PIECE(2, 6) TWM_PIECE(3, 7) }
            if (g == 2) { TWM_PIECE(0, 8) TWM_PIECE(1, 9) TWM_PIECE(2, 10) TWM_PIECE(3, 11) }
            if (g == 3) { TWM_PIECE(0, 12) TWM_PIECE(1, 13) TWM_PIECE(2, 14) TWM_PIECE(3, 15) }
#undef TWM_PIECE
            const float s = (float)sv.h[g];
#pragma unroll
            for (int rr = 0; rr < RL; rr++) {
                // (a_inv: 1 unless the f32 activations of that row were scaled into the f16 range)
                if (TERMS == kTermsRowPacked) acc[t][rr] = fmaf(d[0][2 * rr] + d[0][2 * rr + 1], s * r.a_inv[2 * rr], acc[t][rr]);
                else if (TERMS == kTermsTwoPasses) acc[t][rr] = fmaf(d[0][rr], s * r.a_inv[rr], acc[t][rr]);
                else acc[t][rr] = fmaf(d[rr / 4][rr % 4], s, acc[t][rr]);
            }
        }
    }
}

// ---- sub-tile form: a wave covers 64 / SUB consecutive chunks of SUB columns in one pass ------------------
// Lane l = (chunk l / SUB of the pass, column l % SUB).  With CBSZ = log2(SUB / 4) the MFMA broadcasts an A block
// inside groups of SUB lanes only, so every lane group takes the activations of its own chunk: one A register
// holds 2 * SUB of the chunk's 128 k-values (SUB / 4 pieces of eight), 64 / SUB registers the whole chunk.
// RG = row groups of four: rows 4 .. 4*RG-1 repeat the MFMA chain on the same unpacked weights (f16 rows only).
template <int SUB, int RG = 1>
struct ChunkS {
    uint4v wq[4];                 // this lane's column, its chunk: four groups of 32 nibbles
    uint2v sc;                    // four f16 scales
    uint4v a[RG][64 / SUB];       // activations: row 4*rg + (lane % SUB) % 4, piece (lane % SUB) / 4 of every 2*SUB-wide slice
    uint4v a_lo[64 / SUB];        // f32 activations as two passes: the residual terms
    float a_inv[4];               // f32 activations: what the sums of the four A rows are multiplied by (f32_terms_range)
    bool live;                    // false: a chunk past the k-range, replayed from a valid one; its scales count as 0
};

template <int SUB, int P>
__device__ __forceinline__ float4v mfma_sub(half4v a, half4v b, float4v c)
{
    static_assert(SUB == 32 || SUB == 16, "sub-tiles are 32 or 16 columns wide");
    constexpr int CBSZ = SUB == 32 ? 3 : 2;
    return __builtin_amdgcn_mfma_f32_4x4x4f16(a, b, c, CBSZ, P, 0);
}

// f32 activations in two steps, so that a caller can issue its weight loads between them: the loads of the lane's
// 64 / SUB pieces of eight (ref_order: in the k order (0,4,1,5 | 2,6,3,7) the unpack of the reference's nibble order
// yields), then the range check and the split into f16 terms, which wait for the values.
template <int SUB, bool REF_ORDER>
__device__ __forceinline__ void gemv4s_load_a_f32(float (&v)[64 / SUB * 8], const void *a_any, uint32_t arow, uint32_t kc,
                                                  uint32_t cl, uint32_t k)
{
#pragma unroll
    for (int j = 0; j < 64 / SUB; j++) {
        uint32_t k0 = kc * 128u + j * (2u * SUB) + (cl >> 2) * 8u;
        if (k0 > k - 8u) k0 = k - 8u;  // only the zero-padded groups of a last partial chunk get here
        const float4 *p = (const float4 *)((const float *)a_any + (size_t)arow * k + k0);
        float4 x = p[0], y = p[1];
        const float w[8] = {x.x, REF_ORDER ? y.x : x.y, REF_ORDER ? x.y : x.z, REF_ORDER ? y.y : x.w,
                            REF_ORDER ? x.z : y.x, REF_ORDER ? y.z : y.y, REF_ORDER ? x.w : y.z, y.w};
#pragma unroll
        for (int i = 0; i < 8; i++) v[8 * j + i] = w[i];
    }
}

// The lane's one piece of a row of f32 activations (kTermsOneRowF32): piece cl on 16 columns; on 32 columns the lanes
// of MFMA block b (cl / 4) hold pieces 2 b and 2 b + 1 in turn.  The eight values stay as they were loaded, in a[0][0]
// and a_lo[0] (nothing here waits for them); gemv4s_compute checks their range and splits them.
template <int SUB, bool REF_ORDER, int RG>
__device__ __forceinline__ void gemv4s_load_a_f32_piece(ChunkS<SUB, RG> &r, const void *a_any, uint32_t arow, uint32_t kc,
                                                        uint32_t cl, uint32_t k)
{
    const uint32_t piece = SUB == 16 ? cl : (cl >> 2) * 2u + (cl & 1u);
    uint32_t k0 = kc * 128u + piece * 8u;
    if (k0 > k - 8u) k0 = k - 8u;  // only the zero-padded groups of a last partial chunk get here
    const uint4v *p = (const uint4v *)((const float *)a_any + (size_t)arow * k + k0);
    r.a[0][0] = p[0];
    r.a_lo[0] = p[1];
}

// ... and the split, when the values are needed: two f16 terms of the eight values in the k order of the unpack
template <bool REF_ORDER>
__device__ __forceinline__ void gemv4s_split_a_f32_piece(uint4v x, uint4v y, uint4v &hi, uint4v &lo, float (&inv)[4])
{
    float v[8] = {__uint_as_float(x[0]), __uint_as_float(REF_ORDER ? y[0] : x[1]), __uint_as_float(REF_ORDER ? x[1] : x[2]),
                  __uint_as_float(REF_ORDER ? y[1] : x[3]), __uint_as_float(REF_ORDER ? x[2] : y[0]),
                  __uint_as_float(REF_ORDER ? y[2] : y[1]), __uint_as_float(REF_ORDER ? x[3] : y[2]), __uint_as_float(y[3])};
    f32_terms_range<8, true>(v, inv);
    // Both terms rounded toward zero, two values per instruction: the first term need not be the nearest f16, only
    // near enough for the residual a - hi to be exact in f32 (it is: below one f16 step of a), and a residual cut by
    // one of its own steps is 2^-21 of a.  A value that is an f16 gets hi = a, lo = 0 either way.
    typedef __fp16 pk2 __attribute__((ext_vector_type(2)));
    union { pk2 p[4]; uint4v u; } ch, cl;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        ch.p[i] = __builtin_amdgcn_cvt_pkrtz(v[2 * i], v[2 * i + 1]);
        cl.p[i] = __builtin_amdgcn_cvt_pkrtz(v[2 * i] - (float)ch.p[i][0], v[2 * i + 1] - (float)ch.p[i][1]);
    }
    hi = ch.u;
    lo = cl.u;
}

template <int SUB, int TERMS, int RG>
__device__ __forceinline__ void gemv4s_split_a_f32(ChunkS<SUB, RG> &r, float (&v)[64 / SUB * 8], bool lane_is_lo)
{
    f32_terms_range(v, r.a_inv);
#pragma unroll
    for (int j = 0; j < 64 / SUB; j++) {
        float w[8];
#pragma unroll
        for (int i = 0; i < 8; i++) w[i] = v[8 * j + i];
        split_f32x8(w, r.a[0][j], r.a_lo[j]);
        if (TERMS == kTermsRowPacked) {
#pragma unroll
            for (int i = 0; i < 4; i++) r.a[0][j][i] = lane_is_lo ? r.a_lo[j][i] : r.a[0][j][i];
        }
    }
}

// The lane's activations of chunk kc: 64 / SUB pieces of eight, row arow (term modes as gemv4_load_chunk).
// ref_order: the weights' nibbles are in the reference's natural order, which the mask-and-magic unpack turns
// into the k order (0,4,1,5 | 2,6,3,7) per eight; the (f32) activations take the same order.
// With RG row groups, group rg reads row min(4*rg + arow, m_rows - 1).
template <int SUB, bool AF32, int TERMS, bool REF_ORDER = false, int RG = 1>
__device__ __forceinline__ void gemv4s_load_a(ChunkS<SUB, RG> &r, const void *a_any, uint32_t arow, uint32_t kc, uint32_t cl,
                                              uint32_t k, bool lane_is_lo, uint32_t m_rows = 0)
{
    static_assert(RG == 1 || !AF32, "more than four rows: f16 activations only");
    if (TERMS == kTermsOneRow) {
        // One row: only row 0 of an MFMA block's A operand counts, so the 16 pieces of a chunk need 16 lanes, once.
        // 16 columns: lane cl holds piece cl (the chunk's 256 bytes, contiguous over the lane group); 32 columns: the
        // lanes of MFMA block b (cl / 4) hold pieces 2 b and 2 b + 1 in turn.
        static_assert(TERMS != kTermsOneRow || (!AF32 && RG == 1), "one row of f16 activations");
        const uint32_t piece = SUB == 16 ? cl : (cl >> 2) * 2u + (cl & 1u);
        uint32_t k0 = kc * 128u + piece * 8u;
        if (k0 > k - 8u) k0 = k - 8u;  // only the zero-padded groups of a last partial chunk get here
        r.a[0][0] = *(const uint4v *)((const _Float16 *)a_any + (size_t)arow * k + k0);
        return;
    }
    if (TERMS == kTermsOneRowF32) {
        static_assert(TERMS != kTermsOneRowF32 || (AF32 && RG == 1), "one row of f32 activations");
        gemv4s_load_a_f32_piece<SUB, REF_ORDER, RG>(r, a_any, arow, kc, cl, k);
        return;
    }
    if (AF32) {
        float v[64 / SUB * 8];
        gemv4s_load_a_f32<SUB, REF_ORDER>(v, a_any, arow, kc, cl, k);
        gemv4s_split_a_f32<SUB, TERMS, RG>(r, v, lane_is_lo);
        return;
    }
#pragma unroll
    for (int j = 0; j < 64 / SUB; j++) {
        uint32_t k0 = kc * 128u + j * (2u * SUB) + (cl >> 2) * 8u;
        if (k0 > k - 8u) k0 = k - 8u;  // only the zero-padded groups of a last partial chunk get here
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            uint32_t row = arow + 4u * rg;
            if (RG > 1 && row > m_rows - 1u) row = m_rows - 1u;
            r.a[rg][j] = *(const uint4v *)((const _Float16 *)a_any + (size_t)row * k + k0);
        }
    }
}

// The lane's weights from the column-lane copy: blk = the block of the lane's chunk, col = column in the
// 64-column tile; live = false: a chunk past the k-range replays a valid one, gemv4s_compute takes its scales as 0.
// (Nothing here may touch a loaded value: any use makes the compiler wait for the load where it is issued, and
// the next pass's loads would no longer be in flight while this pass is unpacked.)
template <int SUB, int RG, bool DEFER = false>
__device__ __forceinline__ void gemv4s_load_w(ChunkS<SUB, RG> &r, const char *blk, uint32_t col, bool live)
{
    if (DEFER) {
        r.sc = ld_once((const uint2v *)(blk + 4096u + col * 8u));
        __builtin_amdgcn_sched_barrier(0);  // (the scheduler would put it last, and the first group's sum waits for it)
#pragma unroll
        for (int g = 0; g < 4; g++) r.wq[g] = ld_once((const uint4v *)(blk + g * 1024u + col * 16u));  // (in the order of their use)
        r.live = live;
    } else {
        // a single pass per wave: nothing is in flight behind these loads, the scales may be masked right here
#pragma unroll
        for (int g = 0; g < 4; g++) r.wq[g] = ld_once((const uint4v *)(blk + g * 1024u + col * 16u));
        uint2v s = ld_once((const uint2v *)(blk + 4096u + col * 8u));
        r.sc = live ? s : uint2v{0u, 0u};
        r.live = true;
    }
}

// The lane's weights and f32 activations of chunk kc from the reference's own arrays (packed u8 [G][N][16], scales f16
// [G][N]; crates/kernels/src/quantize.rs:1219-1238): a sub-tile's records of one group are SUB * 16 contiguous bytes.
// col = the lane's column, already clamped to n - 1; col_ok = false gives the lane weight 0, as do live = false (a chunk
// past the k-range, replayed) and the groups past K / 32 of a last partial chunk.
// Order of issue: the activations first (their range check, f32_terms_range, needs them all, loads complete in the order
// of their issue, and these come from the cache); all eight weight loads into locals before anything is written to r
// (written straight into r, each pair was followed by a full wait); the four scales before the records (the first
// group's sum needs them); the scales of dead groups masked after the four have been packed (a select on a freshly
// loaded value is turned into a branch around the load, with a full wait behind it).
template <int SUB, int TERMS, int RG>
__device__ __forceinline__ void gemv4s_load_pass_ref(ChunkS<SUB, RG> &r, const char *packed, const uint16_t *scales,
                                                     const void *a_any, uint32_t arow, uint32_t kc, bool live, uint32_t col,
                                                     bool col_ok, uint32_t n, uint32_t groups, uint32_t cl, uint32_t k,
                                                     bool lane_is_lo)
{
    constexpr bool PIECE = TERMS == kTermsOneRowF32;
    float av[64 / SUB * 8];
    if constexpr (PIECE) gemv4s_load_a_f32_piece<SUB, true, RG>(r, a_any, arow, kc, cl, k);
    else gemv4s_load_a_f32<SUB, true>(av, a_any, arow, kc, cl, k);
    __builtin_amdgcn_sched_barrier(0);
    uint4v wq[4];
    uint32_t sb[4];
    uint32_t keep[4];
    size_t idx[4];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const uint32_t gg = kc * 4u + g;
        idx[g] = (size_t)(gg < groups ? gg : groups - 1u) * n + col;
        keep[g] = (live && gg < groups && col_ok) ? 0xFFFFu : 0u;  // weight exactly 0 otherwise
        sb[g] = scales[idx[g]];  // (cached: the line holds the scales of the neighbouring sub-tiles, which run on the same XCD)
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < 4; g++) wq[g] = ld_once((const uint4v *)(packed + idx[g] * 16u));
#pragma unroll
    for (int g = 0; g < 4; g++) r.wq[g] = wq[g];
    r.sc = uint2v{(sb[0] | (sb[1] << 16)) & (keep[0] | (keep[1] << 16)), (sb[2] | (sb[3] << 16)) & (keep[2] | (keep[3] << 16))};
    r.live = true;  // (masked group by group above)
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!PIECE) gemv4s_split_a_f32<SUB, TERMS, RG>(r, av, lane_is_lo);
}

// lanes (A, B, C, D) of every quad of lanes, in its lanes 0 .. 3
template <int A, int B, int C, int D>
__device__ __forceinline__ uint4v quad_perm(uint4v v)
{
    uint4v o;
#pragma unroll
    for (int w = 0; w < 4; w++) o[w] = (uint32_t)__builtin_amdgcn_mov_dpp((int)v[w], A | (B << 2) | (C << 4) | (D << 6), 0xF, 0xF, true);
    return o;
}
// lane I of every quad of lanes, in all four lanes of the quad
template <int I>
__device__ __forceinline__ uint4v quad_bcast(uint4v v)
{
    return quad_perm<I, I, I, I>(v);
}

// acc[row] += f32(scale) * (sum over the group of A * (q - 8)) for the four groups of the lane's chunk
// (REF_ORDER: kTermsOneRowF32 on the reference's nibble order, whose unpack yields k (0,4,1,5 | 2,6,3,7) per eight)
template <int SUB, int RL, int TERMS, bool REF_ORDER = false>
__device__ __forceinline__ void gemv4s_compute(const ChunkS<SUB, (RL + 3) / 4> &r, const Gemv4Consts &dq, float (&acc)[RL])
{
    constexpr int PIECES = SUB / 4;  // 8-wide k pieces per A register
    constexpr int RG = (RL + 3) / 4;
    static_assert(TERMS != kTermsRowPacked || RL <= 2, "row-packed terms hold at most two rows");
    static_assert(RG == 1 || TERMS == kTermsOne, "more than four rows: one f16 term");
    static_assert((TERMS != kTermsOneRow && TERMS != kTermsOneRowF32) || RL == 1, "the shared-piece forms hold one row");
    union { uint2v u; _Float16 h[4]; } sv;
    sv.u = r.sc;
    // kTermsOneRow: the piece held by lane i of every quad, in all four lanes of the quad (row 0 is the one that counts)
    constexpr bool SHARED = TERMS == kTermsOneRow || TERMS == kTermsOneRowF32;
    constexpr int QN = SHARED ? (SUB == 16 ? 4 : 2) : 1;
    uint4v quad[QN];
    if (TERMS == kTermsOneRow) {
        quad[0] = r.a[0][0];
        if (QN > 1) quad[1 % QN] = quad_bcast<1>(r.a[0][0]);
        if (QN > 2) {
            quad[2 % QN] = quad_bcast<2>(r.a[0][0]);
            quad[3 % QN] = quad_bcast<3>(r.a[0][0]);
        }
    }
    float inv1[4] = {1.f, 1.f, 1.f, 1.f};
    if (TERMS == kTermsOneRowF32) {
        uint4v hi, lo;
        gemv4s_split_a_f32_piece<REF_ORDER>(r.a[0][0], r.a_lo[0], hi, lo, inv1);
        // Rows 0 and 1 of an A block (lanes 0 and 1 of a quad) must be the two terms of one piece; rows 2 and 3 do not
        // count.  Lanes (0, 1) and (2, 3) swap one term each: z holds (first, residual) of the even lanes' pieces in
        // lanes (0, 1) and (2, 3), z2 those of the odd lanes' pieces.  On 16 columns a quad holds four pieces (lane i
        // piece i of its block's four); on 32 columns two (lanes 0, 2 and 1, 3 hold the same).
        const bool odd = (threadIdx.x & 1u) != 0;
        const uint4v hs = quad_perm<1, 0, 3, 2>(hi), ls = quad_perm<1, 0, 3, 2>(lo);
        uint4v z, z2;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            z[w] = odd ? ls[w] : hi[w];
            z2[w] = odd ? lo[w] : hs[w];
        }
        quad[0] = z;
        if (QN > 1) quad[1 % QN] = z2;
        if (QN > 2) {
            quad[2 % QN] = quad_perm<2, 3, 2, 3>(z);
            quad[3 % QN] = quad_perm<2, 3, 2, 3>(z2);
        }
    }
#pragma unroll
    for (int g = 0; g < 4; g++) {
        float4v d[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) d[rg] = float4v{0.f, 0.f, 0.f, 0.f};
        half4v lo4, hi4;
        // word W of group g is the 8-wide piece 4g + W of the chunk: register (4g + W) / PIECES, block
        // (4g + W) % PIECES of the lane group
#define TWM_SUB_PIECE(W)                                                                   \
    {                                                                                      \
        constexpr int PG = 4 * G + W, ONE_ROW = SHARED;                                    \
        constexpr int J = ONE_ROW ? 0 : PG / PIECES;                                       \
        /* one row: piece PG sits in MFMA block PG / 4, lane PG % 4 (16 columns) or block PG / 2, lane PG % 2 */ \
        constexpr int ABID = ONE_ROW ? (SUB == 16 ? PG / 4 : PG / 2) : PG % PIECES;        \
        constexpr int QI = ONE_ROW ? (SUB == 16 ? PG % 4 : PG % 2) : 0;                    \
        union { uint4v u; half4v h[2]; } av, al;                                           \
        gemv4_dequant_word(r.wq[G][W], dq, lo4, hi4);                                      \
        _Pragma("unroll") for (int rg = 0; rg < RG; rg++) {                                \
            av.u = ONE_ROW ? quad[QI] : r.a[rg][J];                                        \
            d[rg] = mfma_sub<SUB, ABID>(av.h[0], lo4, d[rg]);                              \
            d[rg] = mfma_sub<SUB, ABID>(av.h[1], hi4, d[rg]);                              \
        }                                                                                  \
        if (TERMS == kTermsTwoPasses) {                                                    \
            al.u = r.a_lo[J];                                                              \
            d[0] = mfma_sub<SUB, ABID>(al.h[0], lo4, d[0]);                                \
            d[0] = mfma_sub<SUB, ABID>(al.h[1], hi4, d[0]);                                \
        }                                                                                  \
    }
#define TWM_SUB_GROUP(GV)                                                                  \
    if (g == GV) {                                                                         \
        constexpr int G = GV;                                                              \
        TWM_SUB_PIECE(0) TWM_SUB_PIECE(1) TWM_SUB_PIECE(2) TWM_SUB_PIECE(3)                \
    }
        TWM_SUB_GROUP(0) TWM_SUB_GROUP(1) TWM_SUB_GROUP(2) TWM_SUB_GROUP(3)
#undef TWM_SUB_GROUP
#undef TWM_SUB_PIECE
        const float s = r.live ? (float)sv.h[g] : 0.f;
#pragma unroll
        for (int rr = 0; rr < RL; rr++) {
            // (a_inv: 1 unless the f32 activations of that row were scaled into the f16 range)
            if (TERMS == kTermsOneRowF32) acc[rr] = fmaf(d[0][0] + d[0][1], s * inv1[0], acc[rr]);
            else if (TERMS == kTermsRowPacked) acc[rr] = fmaf(d[0][2 * rr] + d[0][2 * rr + 1], s * r.a_inv[2 * rr], acc[rr]);
            else if (TERMS == kTermsTwoPasses) acc[rr] = fmaf(d[0][rr], s * r.a_inv[rr], acc[rr]);
            else acc[rr] = fmaf(d[rr / 4][rr % 4], s, acc[rr]);
        }
    }
}

// NP passes per wave - first, first + stride, ... - with every load of the wave issued before the first unpack: NP
// register sets, no loop.  The loads are unconditional (a pass past the last one replays the k-range's last chunk and
// nobody unpacks it), so the wait in front of each unpack is an exact count of the loads issued after its own.
template <int SUB, int NP, int RG = 1, class Load, class Compute>
__device__ __forceinline__ void gemv4s_run_upfront(uint32_t first, uint32_t stride, uint32_t passes, Load load, Compute compute)
{
    ChunkS<SUB, RG> r[NP];
#pragma unroll
    for (int i = 0; i < NP; i++) {
        load(r[i], first + i * stride);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < NP; i++) {
        if (first + i * stride < passes) compute(r[i]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The sum of v over the lanes l, l + W, l + 2 W, ... of the wave (W = 16, 32; 64: v itself), returned in every one of
// them: v_permlane32_swap puts the lower half's values beside the upper half's, v_permlane16_swap the even rows of 16
// lanes beside the odd ones; an add after each.  The order of the additions is fixed: (g0 + g2) + (g1 + g3).
template <int W>
__device__ __forceinline__ float sum_lane_groups(float v)
{
    static_assert(W == 16 || W == 32 || W == 64, "lane groups of 16, 32 or 64");
    if (W <= 32) {
        auto h = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(h[0]) + __uint_as_float(h[1]);
    }
    if (W == 16) {
        auto q = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(q[0]) + __uint_as_float(q[1]);
    }
    return v;
}

// The passes first, first + stride, ... < passes with two register sets.  ONE: the caller knows that no wave has a
// second pass.
// PIPE: the next pass's loads are in flight while this one is unpacked.  The loop body is one basic block - prefetch,
// unpack, prefetch, unpack - and a prefetch past the wave's last pass is issued all the same (load() replays the
// k-range's last chunk for it, marked dead, and nobody unpacks it): with a prefetch under a condition of its own the
// compiler either moves the loads down into the block that uses them, or assumes at the join that they were not issued
// and waits for the newest loads before the unpack may read the older ones - which is what the plain form below
// does: its second register set only saves the address arithmetic.  The pipelined form needs both sets live through
// the unpack; the variants with more rows or f32 activations would spill, and stay with the plain form.
template <int SUB, bool ONE, int RG = 1, bool PIPE = false, class Load, class Compute>
__device__ __forceinline__ void gemv4s_run_passes(uint32_t first, uint32_t stride, uint32_t passes, Load load, Compute compute)
{
    if (ONE) {
        ChunkS<SUB, RG> r0;
        if (first < passes) {
            load(r0, first);
            compute(r0);
        }
        return;
    }
    if (first >= passes) return;
    ChunkS<SUB, RG> r0, r1;
    uint32_t p = first;
    load(r0, p);
    if (PIPE) {
        const uint32_t mine = (passes - first + stride - 1u) / stride;  // this wave's passes
        for (uint32_t i = 1; i < mine; i += 2) {
            load(r1, p + stride);
            __builtin_amdgcn_sched_barrier(0);  // (the scheduler would sink the prefetch below the unpack)
            compute(r0);
            __builtin_amdgcn_sched_barrier(0);
            load(r0, p + 2u * stride);
            __builtin_amdgcn_sched_barrier(0);
            compute(r1);
            p += 2u * stride;
        }
        if (mine & 1u) compute(r0);
        return;
    }
    while (true) {
        uint32_t pn = p + stride;
        if (pn < passes) load(r1, pn);
        compute(r0);
        if (pn >= passes) break;
        p = pn + stride;
        if (p < passes) load(r0, p);
        compute(r1);
        if (p >= passes) break;
    }
}

}  // namespace twm

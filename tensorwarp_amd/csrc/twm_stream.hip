// Batched-decode kernel (M = 5 .. 32): streams the 16-column tile copy once for up to 32 rows.
//
// Semantics: as the M = 1 kernels (reference order, crates/kernels/src/quantize.rs:1219-1238): per 32-deep
// group the products a * (q - 8) are summed in f32 (here by one v_mfma_f32_16x16x32_f16 with a zero
// accumulator; (q - 8) and the f16 activations are exact operands), then the group sum is scaled once by
// f32(scale) and added to the running f32 sum.  M > 1 has the meaning of gemm_q4_0 (quantize.rs:1825-1858).
//
// Workgroup = 4 waves on one quad of tiles (64 columns) and one k-range (blockIdx.y = split).  The waves
// take the chunks of that range in turn (wave w: chunks w, w + 4, ...), each with its own registers:
//   B : 4 x 16 B nibbles + 4 x 8 B scales per lane and chunk (one tile each), straight from HBM;
//   A : MT x 4 x 16 B per lane and chunk (row = lane % 16 of row block mt, eight k per group), from L2;
//       f32 activations are split once per launch into two f16 arrays (hi, lo) and both terms are multiplied;
// one chunk ahead in a second register set (the loop is unrolled by two, loads are unconditional with
// clamped chunk indices so that the compiler can count them).  At the end the four waves add their sums
// through LDS and the workgroup stores 16 MT x 64 outputs, or parks them as split-K partials for
// k_splitk_reduce.  Bound: HBM (weights are read once); the vector ALU is second (14 instructions per
// tile and group).
#include "twm_device.h"

namespace twm {

namespace {

#define TWM_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ const TWM_GLOBAL char *st_scalar_base(const void *p, size_t byte_offset)
{
    uint64_t v = (uint64_t)p + byte_offset;
    asm("" : "+s"(v));  // a uniform base kept in scalar registers: loads take saddr + 32-bit lane offset
    return (const TWM_GLOBAL char *)v;
}

struct StConsts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};

// eight nibbles of word w -> eight f16 values (q - 8), exact
__device__ __forceinline__ half8 st_unpack(uint32_t w, const StConsts &c)
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

// One lane's eight activations of one group.  TWO: the activations came as f32 and were split beforehand into
// two f16 arrays, hi = f16(a) and lo = f16(a - hi) (about 22 bits together); both terms go through the MFMA.
template <bool TWO>
struct AFrag;
template <>
struct AFrag<false> {
    uint4v v;
    __device__ __forceinline__ void load(const TWM_GLOBAL char *p, uint32_t) { v = *(const TWM_GLOBAL uint4v *)p; }
    __device__ __forceinline__ half8 get() const
    {
        union { uint4v u; half8 h; } cv;
        cv.u = v;
        return cv.h;
    }
};
template <>
struct AFrag<true> {
    uint4v v, w;
    __device__ __forceinline__ void load(const TWM_GLOBAL char *p, uint32_t lo_offset)
    {
        v = *(const TWM_GLOBAL uint4v *)p;
        w = *(const TWM_GLOBAL uint4v *)(p + lo_offset);
    }
    __device__ __forceinline__ half8 get() const
    {
        union { uint4v u; half8 h; } cv;
        cv.u = v;
        return cv.h;
    }
    __device__ __forceinline__ half8 get_lo() const
    {
        union { uint4v u; half8 h; } cv;
        cv.u = w;
        return cv.h;
    }
};

template <int MT, bool AF32>
struct ChunkRegs {
    uint4v bq[4];
    uint2v bs[4];
    AFrag<AF32> a[MT][4];
};

}  // namespace

template <int MT, bool AF32, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_stream(const uint4v *__restrict__ qw, const uint2v *__restrict__ sc,
                                                 const void *__restrict__ a_any, uint32_t m_rows, uint32_t k, uint32_t n,
                                                 uint32_t n_tiles, uint32_t k_chunks, uint32_t chunks_per_split,
                                                 uint32_t lo_offset, float *__restrict__ partials, OutSpec out)
{
    constexpr uint32_t kABytes = 2u;  // f16 rows; with AF32 a_any holds the hi rows and, lo_offset bytes on, the lo rows
    __shared__ float red[WAVES][16 * MT][64];

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t c = lane & 15u, kb = lane >> 4;
    const uint32_t nt0 = blockIdx.x * 4u;  // n_tiles is a multiple of 4
    const uint32_t kc_begin = blockIdx.y * chunks_per_split;
    const uint32_t kc_end = kc_begin + chunks_per_split < k_chunks ? kc_begin + chunks_per_split : k_chunks;

    StConsts dq = {0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(dq.mask_lo), "+s"(dq.mask_hi), "+v"(dq.magic_lo), "+v"(dq.magic_hi));

    float4v acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int t = 0; t < 4; t++) acc[mt][t] = float4v{0.f, 0.f, 0.f, 0.f};

    // per-lane byte offsets that never change: rows past m_rows replay the last row (never stored)
    uint32_t a_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        uint32_t row = mt * 16u + c;
        row = row < m_rows ? row : m_rows - 1;
        a_off[mt] = (row * k + kb * 8u) * kABytes;
    }
    const uint32_t q_off = lane * 16u, s_off = c * 8u;

    auto load_chunk = [&](ChunkRegs<MT, AF32> &r, uint32_t kc) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            size_t tile = (size_t)kc * n_tiles + nt0 + t;
            // (weights are read once per launch: non-temporal)
            r.bq[t] = __builtin_nontemporal_load((const TWM_GLOBAL uint4v *)(st_scalar_base(qw, tile * 1024u) + q_off));
            r.bs[t] = __builtin_nontemporal_load((const TWM_GLOBAL uint2v *)(st_scalar_base(sc, tile * 128u) + s_off));
        }
#pragma unroll
        for (int g = 0; g < 4; g++) {
            // groups past K (only in the last chunk when K is not a multiple of 128) have zero weights:
            // they replay the row's first group instead of reading past the row
            uint32_t kk = kc * 128u + g * 32u;
            kk = kk < k ? kk : 0u;
            const TWM_GLOBAL char *base = st_scalar_base(a_any, (size_t)kk * kABytes);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) r.a[mt][g].load(base + a_off[mt], lo_offset);
        }
    };
    auto compute = [&](const ChunkRegs<MT, AF32> &r) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
            half8 af[MT], al[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                af[mt] = r.a[mt][g].get();
                if constexpr (AF32) al[mt] = r.a[mt][g].get_lo();
            }
#pragma unroll
            for (int t = 0; t < 4; t++) {
                half8 bf = st_unpack(r.bq[t][g], dq);
                uint32_t pair = r.bs[t][g >> 1];
                union { uint16_t u; _Float16 h; } s16;
                s16.u = (uint16_t)((g & 1) ? (pair >> 16) : (pair & 0xFFFFu));
                const float scale = (float)s16.h;
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    float4v d = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[mt], bf, float4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    if constexpr (AF32) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[mt], bf, d, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[mt][t][i] += d[i] * scale;
                }
            }
        }
    };

    // this wave's chunks: kc_begin + wave, + WAVES, ...; two register sets, one chunk ahead
    const uint32_t first = kc_begin + wave;
    if (first < kc_end) {
        const uint32_t count = (kc_end - first + WAVES - 1u) / WAVES;
        const uint32_t last = first + (count - 1u) * WAVES;
        ChunkRegs<MT, AF32> r0, r1;
        load_chunk(r0, first);
        uint32_t kc = first;
        for (uint32_t i = 0; i + 1 < count; i += 2) {
            load_chunk(r1, kc + WAVES);  // i + 1 < count: a chunk of this wave
            compute(r0);
            uint32_t nx = kc + 2u * WAVES < last ? kc + 2u * WAVES : last;  // past the end: the last chunk again, unused
            load_chunk(r0, nx);
            compute(r1);
            kc += 2u * WAVES;
        }
        if (count & 1u) compute(r0);
    }

    // ---- add the four waves' sums: value (mt, t, r) of lane (c, kb) is row 16 mt + 4 kb + r, column 16 t + c
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[wave][(mt * 4 + t) * 4 + r][lane] = acc[mt][t][r];
    __syncthreads();
    const uint32_t col = threadIdx.x & 63u;                 // column inside the quad, fastest over threads
    const uint32_t on = nt0 * 16u + col;
    const uint32_t n_ld = n_tiles * 16u;
#pragma unroll
    for (int j = 0; j < 16 * MT / WAVES; j++) {
        const uint32_t row = (threadIdx.x >> 6) + (uint32_t)WAVES * j;  // 0 .. 16 MT - 1
        const uint32_t reg = ((row >> 4) * 4u + (col >> 4)) * 4u + (row & 3u);
        const uint32_t src_lane = ((row & 15u) >> 2) * 16u + (col & 15u);
        float s = red[0][reg][src_lane];
#pragma unroll
        for (int w = 1; w < WAVES; w++) s += red[w][reg][src_lane];
        if (row >= m_rows) continue;
        const float rs = out.row_scale && !partials ? out.row_scale[row] : 1.f;  // (f32 rows scaled into the f16 range)
        s *= rs;
        if (partials) {
            partials[((size_t)blockIdx.y * m_rows + row) * n_ld + on] = s;
        } else if (out.swiglu) {
            // paired gate/up weight: columns 0..31 of the quad are gate columns, 32..63 the up columns of the same
            // features (two tiles = eight registers further in the same lane)
            if (col < 32u) {
                float u = red[0][reg + 8][src_lane];
#pragma unroll
                for (int w = 1; w < WAVES; w++) u += red[w][reg + 8][src_lane];
                const uint32_t ffn = n >> 1, feat = paired_feature(on);
                if (feat < ffn) out.swiglu[(size_t)row * ffn + feat] = gated_mul(out.gate_act, s, u * rs);
            }
        } else if (on < n) {
#pragma unroll
            for (uint32_t sg = 0; sg < kMaxSegs; sg++) {
                if (sg < out.count) {
                    uint32_t rel = on - out.seg[sg].start;
                    if (rel < out.seg[sg].width) out.seg[sg].ptr[(size_t)row * out.seg[sg].width + rel] = out.seg[sg].bias ? s + out.seg[sg].bias[rel] : s;
                }
            }
        }
    }
}

// f32 activations -> f16 terms, a workgroup per row: hi = f16(x), lo = f16(x - hi) (the subtraction is exact) of
// x = a * 2^-s, where s brings the row's largest magnitude to [2^13, 2^14) when it lies outside [2^-2, 2^14] (any finite
// f32 row keeps about 21 bits per value relative to the row's largest, as the reference's f32 product would; in range
// s = 0 and nothing changes), and row_scale[row] = 2^s, which the GEMM's store multiplies the row's sums by (exact).
// TWO = false: the one rounded term only (the prefill GEMM's operand).
template <bool TWO>
__global__ __launch_bounds__(1024) void k_f32_rows_to_f16(const float *__restrict__ a, _Float16 *__restrict__ hi,
                                                           _Float16 *__restrict__ lo, float *__restrict__ row_scale, uint32_t k)
{
    __shared__ float s_max[16];
    const float *src = a + (size_t)blockIdx.x * k;
    float m = 0.f;
    bool odd = false;  // an infinity or a NaN in the row
    for (uint32_t i = threadIdx.x; i < k; i += 1024u) {
        const float v = fabsf(src[i]);
        odd = odd || !(v <= 3.4028234e38f);
        m = fmaxf(m, v);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (__builtin_amdgcn_ballot_w64(odd) != 0) m = __builtin_inff();
    if ((threadIdx.x & 63u) == 0) s_max[threadIdx.x >> 6] = m;
    __syncthreads();
    m = s_max[0];
#pragma unroll
    for (int w = 1; w < 16; w++) m = fmaxf(m, s_max[w]);
    float down = 1.f, back = 1.f;
    const uint32_t e = (__float_as_uint(m) >> 23) & 0xFFu;   // biased exponent of the row's largest magnitude
    if (e != 0xFFu && e >= 16u && (m > 16384.f || m < 0.25f)) {
        down = __uint_as_float((254u + 13u - e) << 23);       // 2^(13 - (e - 127))
        back = __uint_as_float((e - 13u) << 23);              // 2^((e - 127) - 13)
    }
    if (threadIdx.x == 0) row_scale[blockIdx.x] = back;
    _Float16 *dh = hi + (size_t)blockIdx.x * k, *dl = TWO ? lo + (size_t)blockIdx.x * k : nullptr;
    for (uint32_t i = threadIdx.x; i < k; i += 1024u) {
        const float v = src[i] * down;
        const _Float16 h = (_Float16)v;
        dh[i] = h;
        if (TWO) dl[i] = (_Float16)(v - (float)h);
    }
}

hipError_t launch_f32_rows_to_f16(hipStream_t s, const float *a, _Float16 *hi, _Float16 *lo, float *row_scale, uint32_t rows,
                                  uint32_t k)
{
    if (rows == 0 || k == 0) return hipSuccess;
    if (lo) hipLaunchKernelGGL(k_f32_rows_to_f16<true>, dim3(rows), dim3(1024), 0, s, a, hi, lo, row_scale, k);
    else hipLaunchKernelGGL(k_f32_rows_to_f16<false>, dim3(rows), dim3(1024), 0, s, a, hi, lo, row_scale, k);
    return hipGetLastError();
}

template <int MT, bool AF32, int WAVES>
static hipError_t launch_stream_t(hipStream_t s, const WeightView &w, const void *a, uint32_t m, const OutSpec &out,
                                  uint32_t splits, float *partials, uint32_t lo_offset)
{
    uint32_t cps = (w.k_chunks + splits - 1) / splits;
    splits = (w.k_chunks + cps - 1) / cps;  // no empty split
    dim3 grid(w.n_tiles / 4, splits);
    hipLaunchKernelGGL((k_stream<MT, AF32, WAVES>), grid, dim3(WAVES * 64), 0, s, (const uint4v *)w.qw, (const uint2v *)w.sc, a,
                       m, w.k, w.n, w.n_tiles, w.k_chunks, cps, lo_offset, splits > 1 ? partials : nullptr, out);
    if (splits > 1) {
        hipError_t e = launch_splitk_reduce(s, partials, out, m, w.n, w.n_tiles * 16, splits);
        if (e != hipSuccess) return e;
    }
    return hipGetLastError();
}

// M <= 32.  `scratch` holds, for f32 activations, their two f16 terms (2 x M x K halves) and after them the
// split-K partials (splits x M x (n_tiles * 16) floats); the split factor is cut to what fits.
hipError_t launch_stream(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out_in,
                         uint32_t splits, uint32_t waves, float *scratch, size_t scratch_bytes)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    if (m > 32 || w.k_chunks == 0) return hipErrorInvalidValue;
    if (waves != 4 && waves != 8) return hipErrorInvalidValue;
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
#define TWM_STREAM_CASE(MT, F32, W) return launch_stream_t<MT, F32, W>(s, w, a, m, out, splits, partials, lo_offset)
    if (m <= 16) {
        if (waves == 8) { if (a_f32) TWM_STREAM_CASE(1, true, 8); TWM_STREAM_CASE(1, false, 8); }
        if (a_f32) TWM_STREAM_CASE(1, true, 4);
        TWM_STREAM_CASE(1, false, 4);
    }
    if (waves == 8) { if (a_f32) TWM_STREAM_CASE(2, true, 8); TWM_STREAM_CASE(2, false, 8); }
    if (a_f32) TWM_STREAM_CASE(2, true, 4);
    TWM_STREAM_CASE(2, false, 4);
#undef TWM_STREAM_CASE
}

}  // namespace twm

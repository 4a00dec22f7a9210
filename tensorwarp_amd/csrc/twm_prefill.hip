// Prefill kernel (M > 32): C[M,N] = A[M,K] * dequant(W), FP16 MFMA with FP32 accumulation.
//
// Semantics: gemm_q4_0 (crates/kernels/src/quantize.rs:1825-1858 / kernel :186-246 in the reference),
// i.e. C[m][n] = sum_k A[m][k] * w[k][n].  Here w is the reference's Q4 unpack to FP16,
// f16_rne(f32(scale) * (q - 8)) (quantize.rs:534-571), produced in registers: (q - 8) is exact in f16 and
// one packed f16 multiply by the scale rounds exactly like the reference's __float2half(scale * q).
//
// Block = 16*MT rows x 256 columns (MT = 8 or 4), 4 waves; wave w owns 64 columns (four 16-column tiles of
// the tile-order copy) for all rows of the block, so no weight is unpacked twice inside a block.  Per
// 128-deep k-chunk and wave:
//   A tile (16*MT x 128 f16): global -> LDS directly (global_load_lds_dwordx4), double buffered, 256-byte rows
//                             whose 16-byte slots are XOR-swizzled so that the sixteen rows of an operand
//                             read hit distinct banks;
//   B : 16 bytes of nibbles + four scales per lane per tile, straight from HBM/L2 into registers, one
//       chunk ahead (two register slots), unpacked to MFMA B operands one 32-deep group ahead;
//   16*MT v_mfma_f32_16x16x32_f16 (MT row blocks x 4 column tiles x 4 groups), 16*MT accumulator registers.
// One v_mfma issue slot hides about two other vector instructions, so the unpack (14 instructions per
// tile and group, shared by MT row blocks) is only free from MT = 8 on.
#include "twm_prefill_core.h"

#include <type_traits>

// (two workgroups of four waves per CU: the compiler keeps the kernel within 256 registers)
#define TWM_PF_OCC(TWO) __attribute__((amdgpu_waves_per_eu((TWO) ? 2 : 1)))

namespace twm {

// MT = 16-row blocks per workgroup tile (BM = 16 * MT rows); NTW = 16-column tiles per wave: 4 (256-column blocks) or
// 3 (192-column blocks, for shapes whose 256-column blocks leave a round of workgroups mostly empty)
// HALF: the MFMAs of a 32-deep group run as two half steps of MT / 2 row blocks, and the A operands are read half a step
// ahead instead of a whole one: MT / 2 x 2 operand registers less, which with NTW = 3 brings the kernel under 256
// registers, so that two workgroups share a CU and one's MFMAs fill the issue gaps of the other.
template <int MT, int NTW = 4, bool HALF = false>
__global__ __launch_bounds__(256) TWM_PF_OCC(HALF) void k_prefill(const uint4v *__restrict__ qw, const uint2v *__restrict__ sc,
                                                  const _Float16 *__restrict__ a_any, OutSpec out, uint32_t m_rows,
                                                  uint32_t k, uint32_t n, uint32_t n_tiles, uint32_t k_chunks,
                                                  uint32_t chunks_per_split, float *__restrict__ partials,
                                                  uint32_t row_store, uint32_t col_blocks, uint32_t row_blocks)
{
    constexpr int kPfTileHalves = 16 * MT * kPfRowStride;
    constexpr int NV = MT;       // direct-to-LDS load instructions per wave and A tile (16 MT rows / 16)
    constexpr int HP = 2 * NTW;  // half fragments of B operands per 32-deep group
    extern __shared__ _Float16 a_lds[];  // two tiles of kPfTileHalves (64 KB at MT = 8)

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t c = lane & 15u, kb = lane >> 4;
    // Tile of this workgroup.  Workgroups go to the eight XCDs (each with its own L2) in turn by linear id, so id
    // L runs on XCD L % 8 as that XCD's workgroup L / 8.  The tiles are listed band by band (kBand row blocks high),
    // inside a band column by column, and XCD x takes the x-th eighth of that list
    // (a contiguous range): the 32 (or 64) workgroups an
    // XCD runs at a time then cover a patch of about 8 column blocks x kBand row blocks, which shares every weight
    // slice among kBand and every activation slice among 8 of them in that L2 -- with id = column + columns * row
    // an XCD held two column blocks for ALL row blocks and pulled the whole activation matrix through its L2.
    // (With fewer than 128 tiles per K-split there is no patch to speak of, and the plain order column + columns *
    // row measured 4 - 12 % faster there.)
    constexpr uint32_t kBand = MT == 8 ? 4u : 8u;
    uint32_t bx, by;
    if (col_blocks * row_blocks < 128u) {
        bx = blockIdx.x % col_blocks;
        by = blockIdx.x / col_blocks;
    } else {
        // (shares differ by at most one tile: the first tiles % 8 XCDs take one more)
        const uint32_t tiles = col_blocks * row_blocks, share = tiles >> 3, rest = tiles & 7u, x8 = blockIdx.x & 7u;
        const uint32_t t = x8 * share + (x8 < rest ? x8 : rest) + (blockIdx.x >> 3);
        const uint32_t band_tiles = kBand * col_blocks;
        const uint32_t band = t / band_tiles, u = t - band * band_tiles;
        const uint32_t hb = row_blocks - band * kBand < kBand ? row_blocks - band * kBand : kBand;
        bx = u / hb;
        by = band * kBand + u % hb;
    }
    const uint32_t m0 = by * (16u * MT);
    const uint32_t nt0 = (bx * 4u + wave) * NTW;  // first of this wave's NTW 16-column tiles
    // split-K: blockIdx.z takes chunks [kc0, kc0 + nchunks); chunk indices below are relative to kc0
    const uint32_t kc0 = blockIdx.z * chunks_per_split;
    const uint32_t nchunks = k_chunks - kc0 < chunks_per_split ? k_chunks - kc0 : chunks_per_split;
    const uint32_t last = nchunks - 1;

    const PfConsts dq = make_pf_consts();

    // this wave's tiles; tiles past the end replay the last tile and are never stored
    uint32_t nt[NTW];
#pragma unroll
    for (int t = 0; t < NTW; t++) nt[t] = nt0 + t < n_tiles ? nt0 + t : n_tiles - 1;

    // Accumulators live in AGPRs.  The empty asm pins them there across the loop back edge; without it the
    // compiler carries them in VGPRs and copies all of them to AGPRs and back every iteration.
    float4v acc[MT][NTW];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int t = 0; t < NTW; t++) acc[mt][t] = float4v{0.f, 0.f, 0.f, 0.f};
    auto pin_acc = [&]() {
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int t = 0; t < NTW; t++) asm volatile("" : "+a"(acc[mt][t]));
    };
    pin_acc();

    // ---- A tile: global -> LDS directly (global_load_lds_dwordx4: lane L's 16 bytes land at the instruction's
    // LDS base + 16 L, no registers, no LDS store instruction).  Instruction j of wave w fills rows
    // 16 j + 4 w .. + 3 (256 bytes each).  Slot s of row r holds the row's vector s ^ (r % 16) (8 halves
    // each): lane L = (row 4 w + L / 16 of the instruction, slot L % 16) therefore fetches vector
    // (L % 16) ^ ((4 w + L / 16) % 16), and the sixteen rows of an operand read (one slot each, chosen by the
    // same XOR) fall on distinct banks.  Loads are unconditional: rows past m_rows replay the last row and
    // are never stored; vectors past k replay the row's first vector, where the padded weights are zero.
    const char *a_blk = (const char *)a_any + (size_t)m0 * k * 2u;
    const uint32_t a_vec = (lane & 15u) ^ ((4u * wave + (lane >> 4)) & 15u);
    uint32_t a_off[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        uint32_t row = m0 + 16u * j + 4u * wave + (lane >> 4);
        row = (row < m_rows ? row : m_rows - 1) - m0;
        a_off[j] = (row * k + a_vec * 8u) * 2u;
    }
    auto load_a = [&](uint32_t buf, uint32_t kc, int j) {  // part j of tile kc (relative) into LDS buffer buf
        const char *src = a_blk + (size_t)(kc0 + kc) * 256u;
        const uint32_t back = (kc0 + kc) * 128u + a_vec * 8u < k ? 0u : a_vec * 16u;
        __builtin_amdgcn_global_load_lds((const TWM_GLOBAL void *)(src + (a_off[j] - back)),
                                         (__attribute__((address_space(3))) void *)(a_lds + buf * kPfTileHalves +
                                                                                    (16 * j + 4 * wave) * kPfRowStride),
                                         16, 0, 0);
    };
    // everything this wave has loaded (its parts of the A tile among it) has arrived: before a barrier
    auto wait_loads = [&]() { __builtin_amdgcn_s_waitcnt(0x0F70); };  // vmcnt(0), other counters untouched

    // ---- B: chunk kc lives in register slot kc % 2
    uint4v bq[2][NTW];
    uint2v bs[2][NTW];
    const uint32_t q_off = lane * 16u, s_off = c * 8u;
    auto load_bq = [&](int slot, uint32_t kc, int t) {
        bq[slot][t] = *(const TWM_GLOBAL uint4v *)(scalar_base(qw, (size_t)((kc0 + kc) * n_tiles + nt[t]) * 1024u) + q_off);
    };
    auto load_bs = [&](int slot, uint32_t kc, int t) {
        bs[slot][t] = *(const TWM_GLOBAL uint2v *)(scalar_base(sc, (size_t)((kc0 + kc) * n_tiles + nt[t]) * 128u) + s_off);
    };
    // half fragment hp (tile hp / 2, half hp % 2) of group g
    auto unpack = [&](int slot, int g, PfFrag (&bf)[NTW], int hp) {
        const int t = hp >> 1;
        pf_unpack_half(bf[t], hp & 1, bq[slot][t][g], bs[slot][t][g >> 1], g & 1, dq);
    };

    uint32_t rd_off[4];  // row c of a row block, vector 4 g + kb of the chunk -> slot (4 g + kb) ^ c
#pragma unroll
    for (int g = 0; g < 4; g++) rd_off[g] = c * kPfRowStride + (((4u * g + kb) ^ c) * 8u);
    auto read_a = [&](uint32_t buf, int g, int mt) {
        return *(const half8 *)(a_lds + buf * kPfTileHalves + rd_off[g] + mt * 16 * kPfRowStride);
    };

    constexpr int AF = HALF ? MT / 2 : MT;   // row blocks whose A operands are held at a time
    half8 af0[AF], af1[AF];
    PfFrag bf0[NTW], bf1[NTW];

    // One step = the MFMAs of one 32-deep group, in MT units of NTW (one row block x NTW tiles).  Unit mt
    // also fetches the next group's A operand for its row block, unpacks its share of the next group's B
    // operands and issues `extra(mt)`, its share of the traffic for later chunks.  The scheduling barrier
    // after each unit keeps this interleaving: one MFMA issue slot hides about two other instructions,
    // but only if they sit next to it.
    auto step = [&](const half8 (&af_cur)[AF], const PfFrag (&bf_cur)[NTW], half8 (&af_nxt)[AF], PfFrag (&bf_nxt)[NTW],
                    uint32_t rd_buf, int rd_g, int uq_slot, int uq_g, auto extra) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            af_nxt[mt % AF] = read_a(rd_buf, rd_g, mt);
            extra(mt);
            // the 2 NTW half fragments of the next group, dealt over the MT units
#pragma unroll
            for (int hp = mt * HP / MT; hp < (mt + 1) * HP / MT; hp++) unpack(uq_slot, uq_g, bf_nxt, hp);
#pragma unroll
            for (int t = 0; t < NTW; t++)
                acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af_cur[mt % AF], bf_cur[t].h, acc[mt][t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // Half step h of group g: the MFMAs of row blocks h MT/2 .. with the operands in af_cur; unit u reads the operand of
    // row block (1 - h) MT/2 + u of group rd_g for the next half step, and unpacks its share (part h) of the next group.
    auto half_step = [&](int h, const half8 (&af_cur)[AF], const PfFrag (&bf_cur)[NTW], half8 (&af_nxt)[AF], PfFrag (&bf_nxt)[NTW],
                         uint32_t rd_buf, int rd_g, int uq_slot, int uq_g, auto extra) {
#pragma unroll
        for (int u = 0; u < AF; u++) {
            const int mt = h * AF + u;
            af_nxt[u] = read_a(rd_buf, rd_g, (1 - h) * AF + u);
            extra(u);
#pragma unroll
            for (int hp = mt * HP / MT; hp < (mt + 1) * HP / MT; hp++) unpack(uq_slot, uq_g, bf_nxt, hp);
#pragma unroll
            for (int t = 0; t < NTW; t++)
                acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af_cur[u], bf_cur[t].h, acc[mt][t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // One k-chunk (B slot S = kc & 1, LDS buffer kc & 1).  On entry af0 / bf0 hold group 0 of this chunk.
    //   step 0 .. 2: no loads; at the end of step 2 wait for this wave's loads, then the chunk's only barrier:
    //              A tile kc+1 and B of chunk kc+1 are complete (both requested a whole chunk ago, nothing newer
    //              is in flight), and every wave is done reading buffer kc & 1 (tile kc: its reads were issued
    //              up to step 2 and are waited for by the barrier)
    //   step 3   : A tile kc+2 -> buffer kc & 1 and B of chunk kc+2 -> slot S (its last group was unpacked in
    //              step 2); the step's own reads and unpack are already those of chunk kc+1, group 0
    // Past the end the last chunk is loaded again and never used.
    // HALF: eight half steps; the last reads of tile kc are those of half step 6 (group 3, second half), so the wait
    // for the loads stands before half step 6 (which already unpacks chunk kc+1), the barrier behind it, and half step 7
    // issues the loads of chunk kc+2.  On entry af0 holds the first half of group 0.
    auto chunk = [&](auto slot_c, uint32_t kc) {
        constexpr int S = decltype(slot_c)::value, S1 = S ^ 1;
        const uint32_t buf = kc & 1u;
        const uint32_t kc2 = kc + 2 < last ? kc + 2 : last;
        auto later_loads = [&](int u, int units) {
            // (the A parts and the B tiles of chunk kc + 2, dealt over `units` units)
#pragma unroll
            for (int j = 0; j < NV; j++)
                if (j * units / NV == u) load_a(buf, kc2, j);
#pragma unroll
            for (int t = 0; t < NTW; t++) {
                if (t * units / 4 == u) load_bq(S, kc2, t);
                if (t * units / 4 + (units >= 8 ? 1 : 0) == u) load_bs(S, kc2, t);
            }
        };
        if constexpr (HALF) {
            half_step(0, af0, bf0, af1, bf1, buf, 0, S, 1, [&](int) {});
            half_step(1, af1, bf0, af0, bf1, buf, 1, S, 1, [&](int) {});
            half_step(0, af0, bf1, af1, bf0, buf, 1, S, 2, [&](int) {});
            half_step(1, af1, bf1, af0, bf0, buf, 2, S, 2, [&](int) {});
            half_step(0, af0, bf0, af1, bf1, buf, 2, S, 3, [&](int) {});
            half_step(1, af1, bf0, af0, bf1, buf, 3, S, 3, [&](int) {});
            wait_loads();
            half_step(0, af0, bf1, af1, bf0, buf, 3, S1, 0, [&](int) {});
            __syncthreads();
            half_step(1, af1, bf1, af0, bf0, buf ^ 1u, 0, S1, 0, [&](int u) { later_loads(u, AF); });
        } else {
            step(af0, bf0, af1, bf1, buf, 1, S, 1, [&](int) {});
            step(af1, bf1, af0, bf0, buf, 2, S, 2, [&](int) {});
            step(af0, bf0, af1, bf1, buf, 3, S, 3, [&](int) {});
            wait_loads();
            __syncthreads();
            step(af1, bf1, af0, bf0, buf ^ 1u, 0, S1, 0, [&](int u) { later_loads(u, MT); });
        }
        pin_acc();
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;

    // prologue: tiles 0 and 1 -> LDS, B chunks 0 and 1 -> slots 0 and 1
    const uint32_t kc1p = 1 < last ? 1 : last;
#pragma unroll
    for (int j = 0; j < NV; j++) load_a(0, 0, j);
#pragma unroll
    for (int t = 0; t < NTW; t++) {
        load_bq(0, 0, t);
        load_bs(0, 0, t);
        load_bq(1, kc1p, t);
        load_bs(1, kc1p, t);
    }
#pragma unroll
    for (int j = 0; j < NV; j++) load_a(1, kc1p, j);
    wait_loads();
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < AF; mt++) af0[mt] = read_a(0, 0, mt);
#pragma unroll
    for (int hp = 0; hp < HP; hp++) unpack(0, 0, bf0, hp);
    __builtin_amdgcn_sched_barrier(0);

    uint32_t kc = 0;
    for (; kc + 2 <= nchunks; kc += 2) {
        chunk(S0{}, kc);
        chunk(S1{}, kc + 1);
    }
    if (kc < nchunks) chunk(S0{}, kc);

    // ---- store: lane (c, kb) holds rows 4*kb + r of row block mt, column 16*tile + c ----
    if (row_store) {
        // One destination (the output itself or this split's partial sums), rows 16-byte aligned: each wave turns
        // its 16 x 64 block of a row block through LDS (272-byte rows: the four row groups kb fall on different
        // banks) so that a lane stores 16 bytes and sixteen lanes cover 256 consecutive bytes of a row, instead
        // of 64-byte pieces of four rows from 4-byte stores.
        float *dst = partials ? partials + ((size_t)blockIdx.z * m_rows) * (n_tiles * 16u) : out.seg[0].ptr;
        const uint32_t ld = partials ? n_tiles * 16u : n;
        const uint32_t n_lim = partials ? n_tiles * 16u : n;  // a multiple of 4
        __syncthreads();                                       // every wave is done with the A tiles
        float *stage = (float *)a_lds + wave * (16 * 68);
        const uint32_t col = nt0 * 16u + (lane & 15u) * 4u;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
            for (int t = 0; t < NTW; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) stage[(kb * 4 + r) * 68 + t * 16 + c] = acc[mt][t][r];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t row = (lane >> 4) + 4u * i;
                const float4v v = *(const float4v *)(stage + row * 68 + (lane & 15u) * 4u);
                const uint32_t om = m0 + mt * 16u + row;
                if (om < m_rows && col < n_lim && (lane & 15u) * 4u < 16u * NTW)
                    __builtin_nontemporal_store(v, (float4v *)(dst + (size_t)om * ld + col));
            }
        }
        return;
    }
    if (partials) {
        // split-K: plain [split][row][padded column] partial sums, added up in split order by k_splitk_reduce
        const uint32_t n_ld = n_tiles * 16u;
        float *dst = partials + ((size_t)blockIdx.z * m_rows) * n_ld;
#pragma unroll
        for (int t = 0; t < NTW; t++) {
            if (nt0 + t >= n_tiles) continue;
            uint32_t on = (nt0 + t) * 16u + c;
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    uint32_t om = m0 + mt * 16u + kb * 4u + r;
                    if (om < m_rows) dst[(size_t)om * n_ld + on] = acc[mt][t][r];
                }
        }
        return;
    }
    if (NTW == 4 && out.swiglu) {
        // paired gate/up weight: this wave's tiles 0, 1 are 32 gate columns and tiles 2, 3 the up columns of the
        // same features, in the same lanes and registers.  The 16 x 32 gated block of a row block goes through
        // LDS like the plain store: a lane stores 16 bytes, eight lanes cover the wave's 128 bytes of a row.
        const uint32_t ffn = n >> 1;  // a multiple of 32
        __syncthreads();
        float *stage = (float *)a_lds + wave * (16 * 36);
        const uint32_t feat = paired_feature(nt0 * 16u) + (lane & 7u) * 4u;
        const bool aligned = ((uintptr_t)out.swiglu & 15) == 0;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    stage[(kb * 4 + r) * 36 + t * 16 + c] = gated_mul(out.gate_act, acc[mt][t][r], acc[mt][(t + 2) % NTW][r]);
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint32_t row = (lane >> 3) + 8u * i;
                const float4v v = *(const float4v *)(stage + row * 36 + (lane & 7u) * 4u);
                const uint32_t om = m0 + mt * 16u + row;
                if (om < m_rows && feat < ffn && nt0 + 3 < n_tiles) {
                    float *p = out.swiglu + (size_t)om * ffn + feat;
                    if (aligned) {
                        __builtin_nontemporal_store(v, (float4v *)p);
                    } else {
                        p[0] = v[0]; p[1] = v[1]; p[2] = v[2]; p[3] = v[3];
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < NTW; t++) {
        if (nt0 + t >= n_tiles) continue;
        uint32_t on = (nt0 + t) * 16u + c;
        if (on >= n) continue;
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                uint32_t om = m0 + mt * 16u + kb * 4u + r;
                if (om < m_rows) pf_store_out(out, om, on, acc[mt][t][r]);
            }
    }
}

// out[row][col] = sum over splits, in split order (deterministic), of partials[split][row][col]
__global__ __launch_bounds__(256) void k_splitk_reduce(const float *__restrict__ partials, OutSpec out, uint32_t m_rows, uint32_t n,
                                                         uint32_t n_ld, uint32_t splits)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // one thread per four padded columns
    uint32_t quads = n_ld / 4;
    if (idx >= (size_t)m_rows * quads) return;
    uint32_t row = (uint32_t)(idx / quads), col = (uint32_t)(idx % quads) * 4u;
    const float4 *src = (const float4 *)(partials + (size_t)row * n_ld + col);
    size_t stride4 = (size_t)m_rows * n_ld / 4;
    float4 s = src[0];
    for (uint32_t z = 1; z < splits; z++) {
        float4 v = src[z * stride4];
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    if (out.row_scale) {
        const float rs = out.row_scale[row];  // (f32 rows scaled into the f16 range)
        s.x *= rs; s.y *= rs; s.z *= rs; s.w *= rs;
    }
    if (col + 0 < n) pf_store_out(out, row, col + 0, s.x);
    if (col + 1 < n) pf_store_out(out, row, col + 1, s.y);
    if (col + 2 < n) pf_store_out(out, row, col + 2, s.z);
    if (col + 3 < n) pf_store_out(out, row, col + 3, s.w);
}

// The same sum for a paired gate/up weight: one thread per four features adds the gate and the up partials
// (32 columns apart) in split order and stores silu(gate) * up.
__global__ __launch_bounds__(256) void k_splitk_reduce_swiglu(const float *__restrict__ partials, float *__restrict__ gate_out,
                                                                uint32_t m_rows, uint32_t ffn, uint32_t n_ld, uint32_t splits,
                                                                uint32_t act, const float *__restrict__ row_scale)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    uint32_t quads = ffn / 4;  // ffn is a multiple of 32
    if (idx >= (size_t)m_rows * quads) return;
    uint32_t row = (uint32_t)(idx / quads), feat = (uint32_t)(idx % quads) * 4u;
    uint32_t col = (feat >> 5) * 64u + (feat & 31u);
    const float4 *src = (const float4 *)(partials + (size_t)row * n_ld + col);
    size_t stride4 = (size_t)m_rows * n_ld / 4;
    float4 g = src[0], u = src[8];
    for (uint32_t z = 1; z < splits; z++) {
        float4 v = src[z * stride4], w = src[z * stride4 + 8];
        g.x += v.x; g.y += v.y; g.z += v.z; g.w += v.w;
        u.x += w.x; u.y += w.y; u.z += w.z; u.w += w.w;
    }
    const float rs = row_scale ? row_scale[row] : 1.f;  // (f32 rows scaled into the f16 range)
    float4 o = {gated_mul(act, g.x * rs, u.x * rs), gated_mul(act, g.y * rs, u.y * rs), gated_mul(act, g.z * rs, u.z * rs),
                gated_mul(act, g.w * rs, u.w * rs)};
    *(float4 *)(gate_out + (size_t)row * ffn + feat) = o;
}

// out[row][:] *= row_scale[row] over every segment, for the rows whose factor is not 1 (a workgroup per row; a row that
// needs nothing costs its workgroup one load)
__global__ __launch_bounds__(256) void k_scale_rows(OutSpec out, const float *__restrict__ row_scale)
{
    const uint32_t row = blockIdx.x;
    const float rs = row_scale[row];
    if (rs == 1.f) return;
    for (uint32_t sg = 0; sg < out.count && sg < (uint32_t)kMaxSegs; sg++) {
        float *p = out.seg[sg].ptr + (size_t)row * out.seg[sg].width;
        for (uint32_t c = threadIdx.x; c < out.seg[sg].width; c += 256u) p[c] *= rs;
    }
}

hipError_t launch_splitk_reduce(hipStream_t s, const float *partials, const OutSpec &out, uint32_t m, uint32_t n,
                                uint32_t n_ld, uint32_t splits)
{
    size_t quads = (size_t)m * n_ld / 4;
    if (quads == 0) return hipSuccess;
    if (out.swiglu) {
        if (n % (2 * kPairWidth) != 0) return hipErrorInvalidValue;
        size_t fq = (size_t)m * (n / 2) / 4;
        hipLaunchKernelGGL(k_splitk_reduce_swiglu, dim3((unsigned)((fq + 255) / 256)), dim3(256), 0, s, partials, out.swiglu, m,
                           n / 2, n_ld, splits, out.gate_act, out.row_scale);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(k_splitk_reduce, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, partials, out, m, n, n_ld,
                       splits);
    return hipGetLastError();
}

// Block form and split-K factor by a small cost model fitted to per-shape sweeps on MI355X (microseconds per
// 128-deep chunk and workgroup): a 64-row block alone on a CU 1.1, two sharing a CU 2.0 each, a 128-row block 1.5
// with few workgroups in flight up to 1.8 with all 256 CUs busy; 3 per round of workgroups for the start and the
// store; a split costs the second kernel, 2.5 + its read of the partial sums at 4 TB/s.  (128-row blocks unpack
// every weight for twice the rows: per row they are the cheapest form as soon as there is a workgroup for most
// CUs, and K 4096 -> N 11008 at M = 512 runs in 50 us on 172 of them against 61 us on 344 64-row blocks.)
// Forms: 64 = 64 rows x 256 columns, 128 = 128 x 256, 192 = 128 rows x 192 columns (three tiles per wave).  Alone on a
// CU a chunk of the 192-column form takes 0.95 of a 256-column block's chunk for 0.75 of the columns; it pays where
// it fills a round of workgroups that 256-column blocks leave mostly empty (4096 -> 11008 at M = 512: 232 workgroups
// instead of 172, 46.1 against 47.8 us; kPf192 is the weight that reproduces the best form on the sweep's cases with
// up to 256 workgroups, not that ratio).  With more workgroups than CUs its two-per-CU variant runs (the kernel's HALF
// form, under 256 registers): 4096 -> 11008 at M = 1024 81.6 us against 102.5 on 256-column blocks, 3584 -> 4608 at
// M = 2048 66.9 against 90.7, 3584 -> 37888 at M = 2048 462 against 476; level at 4096 -> 11008, M = 2048 (158.7 / 158.0).
// Not with the gated store, whose waves hold gate and up tiles in pairs.
constexpr double kPf192 = 0.80;
struct PrefillPlan {
    uint32_t block_rows, splits;   // block_rows: the form (64, 128, 192)
    double us;
};
static PrefillPlan plan_prefill(uint32_t rows, uint32_t force_rows, uint32_t force_splits, uint32_t n_tiles, uint32_t k_chunks,
                                bool gated)
{
    PrefillPlan best = {force_rows ? force_rows : 64u, force_splits ? force_splits : 1u, 1e30};
    const size_t n_ld = (size_t)n_tiles * 16;
    const double partial_us = (double)rows * (double)n_ld * 4.0 / 4.0e6;  // the reduce kernel's read of one split
    for (uint32_t bm = 64; bm <= 192; bm += 64) {
        if (force_rows && bm != force_rows) continue;
        if (bm == 192 && gated) continue;
        const uint32_t col_blocks = bm == 192 ? (n_tiles + 11) / 12 : (n_tiles + 15) / 16, height = bm == 64 ? 64u : 128u;
        const double wgs = (double)((rows + height - 1) / height) * col_blocks;
        for (uint32_t sp = 1; sp <= 64; sp++) {
            if (force_splits ? sp != force_splits : sp * 2 > (k_chunks > 1 ? k_chunks : 2) && sp > 1) continue;
            const uint32_t cps = (k_chunks + sp - 1) / sp;
            if (!force_splits && (k_chunks + cps - 1) / cps != sp) continue;  // same work as a smaller factor
            const double total = wgs * sp;
            double t;
            if (bm == 192 && total > 256.0) {
                // two workgroups share a CU: 2.45 per chunk each; a last round of up to one per CU runs at 1.45
                const double full = (double)(uint64_t)(total / 512.0), rem = total - 512.0 * full;
                t = full * (cps * 2.45 + 3.0) + (rem == 0.0 ? 0.0 : (rem <= 256.0 ? cps * 1.45 : cps * 2.45) + 3.0);
            } else if (bm >= 128) {
                const double rounds = (double)(uint64_t)((total + 255.0) / 256.0);
                const double load = total >= 256.0 ? 1.0 : total / 256.0;
                t = rounds * (cps * (1.5 + 0.3 * load) * (bm == 192 ? kPf192 : 1.0) + 3.0);
            } else if (total <= 256.0) {
                t = cps * 1.1 + 3.0;
            } else {
                const double full = (double)(uint64_t)(total / 512.0), rem = total - 512.0 * full;
                t = full * (cps * 2.0 + 3.0) + (rem == 0.0 ? 0.0 : (rem <= 256.0 ? cps * 1.1 : cps * 2.0) + 3.0);
            }
            if (sp > 1) t += 2.5 + sp * partial_us;
            // a larger factor, and the narrower block, have to pay for themselves
            const double margin = (sp > best.splits && bm == best.block_rows) || bm == 192 ? 0.97 : 1.0;
            if (t < best.us * margin) {
                best.block_rows = bm;
                best.splits = sp;
                best.us = t;
            }
        }
    }
    return best;
}

// The plan within what the scratch can hold of partial sums (ws_bytes = 0: no scratch, unsplit).
static PrefillPlan plan_prefill_within(uint32_t rows, uint32_t block_rows, uint32_t splits, uint32_t n_tiles, uint32_t k_chunks,
                                       size_t ws_bytes, bool gated)
{
    const size_t n_ld = (size_t)n_tiles * 16;
    PrefillPlan plan = plan_prefill(rows, block_rows, splits, n_tiles, k_chunks, gated);
    const size_t per_split = (size_t)rows * n_ld * 4;
    if (plan.splits > 1 && (ws_bytes == 0 || per_split == 0 || plan.splits > ws_bytes / per_split)) {
        // the scratch cannot hold that many partial sums: plan again within what it holds (at least unsplit)
        uint32_t cap = (ws_bytes == 0 || per_split == 0) ? 1u : (uint32_t)(ws_bytes / per_split);
        if (cap < 2) cap = 1;
        if (splits) plan.splits = cap;  // a forced factor is cut, the forced height kept
        else {
            PrefillPlan capped = {0, 0, 1e30};
            for (uint32_t sp = 1; sp <= cap; sp++) {
                PrefillPlan c = plan_prefill(rows, block_rows, sp, n_tiles, k_chunks, gated);
                if (c.us < capped.us) capped = c;
            }
            plan = capped;
        }
    }
    return plan;
}

void prefill_plan_of(uint32_t rows, uint32_t block_rows, uint32_t splits, uint32_t n_tiles, uint32_t k_chunks, size_t ws_bytes,
                     bool gated, uint32_t *block_rows_out, uint32_t *splits_out)
{
    const PrefillPlan plan = plan_prefill_within(rows, block_rows, splits, n_tiles, k_chunks, ws_bytes, gated);
    *block_rows_out = plan.block_rows;
    *splits_out = plan.splits;
}

template <int MT, int NTW = 4, bool HALF = false>
static hipError_t launch_prefill_t(hipStream_t s, const WeightView &w, const _Float16 *a, uint32_t m, const OutSpec &out,
                                   uint32_t splits, float *partials, bool via_partials = false)
{
    size_t lds = (size_t)2 * 16 * MT * kPfRowStride * sizeof(_Float16);
    uint32_t cps = (w.k_chunks + splits - 1) / splits;
    splits = (w.k_chunks + cps - 1) / cps;  // no empty split
    const uint32_t col_blocks = (w.n_tiles + 4 * NTW - 1) / (4 * NTW), row_blocks = (m + 16 * MT - 1) / (16 * MT);
    dim3 grid(col_blocks * row_blocks, 1, splits);  // the kernel turns the linear id into an XCD-aware tile
    // 16-byte row stores: into the partial sums always (padded width, a multiple of 64); into the output when it
    // is one plain [M, N] matrix with N a multiple of 4 at a 16-byte aligned address
    // (via_partials: the sums of a single split go through the partial-sum buffer too and k_splitk_reduce stores them:
    // it is the store that applies the rows' power-of-two factors of f32 activations ahead of a bias or a gate)
    via_partials = via_partials && partials != nullptr;
    uint32_t row_store = 1;
    if (splits == 1 && !via_partials)
        row_store = !out.swiglu && out.count == 1 && out.seg[0].start == 0 && out.seg[0].width == w.n && !out.seg[0].bias &&
                    w.n % 4 == 0 && ((uintptr_t)out.seg[0].ptr & 15) == 0;
    if (NTW != 4 && out.swiglu) return hipErrorInvalidValue;
    hipLaunchKernelGGL((k_prefill<MT, NTW, HALF>), grid, dim3(256), lds, s, (const uint4v *)w.qw, (const uint2v *)w.sc, a, out, m, w.k,
                       w.n, w.n_tiles, w.k_chunks, cps, splits > 1 || via_partials ? partials : nullptr, row_store, col_blocks, row_blocks);
    if (splits > 1 || via_partials) return launch_splitk_reduce(s, partials, out, m, w.n, w.n_tiles * 16, splits);
    return hipGetLastError();
}

// Once per device, outside any stream capture: the 128-row variant asks for all 64 KB of dynamic LDS.
hipError_t init_prefill()
{
    hipError_t e = hipFuncSetAttribute((const void *)k_prefill<8>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       2 * 16 * 8 * kPfRowStride * (int)sizeof(_Float16));
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute((const void *)k_prefill<8, 3>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            2 * 16 * 8 * kPfRowStride * (int)sizeof(_Float16));
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute((const void *)k_prefill<8, 3, true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               2 * 16 * 8 * kPfRowStride * (int)sizeof(_Float16));
}

// block_rows: the block form (64 = 64 rows x 256 columns, 128 = 128 x 256, 192 = 128 rows x 192 columns), splits: k-split
// factor; 0 = choose (plan_prefill), within what `scratch` can hold as f32 partial sums.
// `scratch` (scratch_bytes) holds the f16 copy of f32 activations and / or the split-K partials; when it
// cannot hold all M rows the rows are processed in slabs.
hipError_t launch_prefill(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                          uint32_t block_rows, uint32_t splits, void *scratch, size_t scratch_bytes)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    if (block_rows != 0 && block_rows != 64 && block_rows != 128 && block_rows != 192) return hipErrorInvalidValue;
    auto run = [&](const _Float16 *a16, uint32_t rows, const OutSpec &o, void *ws, size_t ws_bytes, bool via = false) {
        // (a forced 192-column form with the gated store: the 256-column one)
        const uint32_t form = block_rows == 192 && o.swiglu ? 128u : block_rows;
        const PrefillPlan plan = plan_prefill_within(rows, form, splits, w.n_tiles, w.k_chunks, ws ? ws_bytes : 0, o.swiglu != nullptr);
        if (plan.block_rows == 64) return launch_prefill_t<4>(s, w, a16, rows, o, plan.splits, (float *)ws, via);
        if (plan.block_rows == 192) {
            // more workgroups than CUs: the variant of which two share a CU (4096 -> 11008 at M = 1024, 464 workgroups:
            // 81.6 against 89.5 us; at M = 512, 232 workgroups, 49.0 against 46.4)
            const uint64_t wgs = (uint64_t)((w.n_tiles + 11) / 12) * ((rows + 127) / 128) * plan.splits;
            return wgs > 256 ? launch_prefill_t<8, 3, true>(s, w, a16, rows, o, plan.splits, (float *)ws, via)
                             : launch_prefill_t<8, 3>(s, w, a16, rows, o, plan.splits, (float *)ws, via);
        }
        return launch_prefill_t<8>(s, w, a16, rows, o, plan.splits, (float *)ws, via);
    };
    if (!a_f32) return run((const _Float16 *)a, m, out, scratch, scratch_bytes);
    // f16 copy of the activations (each row scaled by a power of two where it would leave the f16 range, the factors in
    // front of the copy) at the front of the scratch, partials behind it.  The factors go back onto the sums in the
    // K-split's sum kernel where there is one; a launch without a K-split stores plain sums and a small kernel scales
    // the rows that need it afterwards (most launches: none) -- unless a bias or a gate follows the sum, which the
    // factor has to come before: then the single split's sums go through the partial-sum buffer and the sum kernel too.
    bool after_sum = out.swiglu != nullptr;
    for (uint32_t i = 0; i < out.count; i++) after_sum = after_sum || out.seg[i].bias != nullptr;
    size_t row_bytes = (size_t)w.k * 2 + 4 + (after_sum ? (size_t)w.n_tiles * 16 * 4 : 0);
    if (!scratch || scratch_bytes < row_bytes + 512) return hipErrorInvalidValue;
    uint32_t slab = (uint32_t)((scratch_bytes - 512) / 2 / row_bytes < m ? (scratch_bytes - 512) / 2 / row_bytes : m);
    if (slab == 0) slab = 1;
    if (slab >= 128) slab -= slab % 128;
    for (uint32_t r0 = 0; r0 < m; r0 += slab) {
        uint32_t rows = m - r0 < slab ? m - r0 : slab;
        float *row_scale = (float *)scratch;
        _Float16 *a16 = (_Float16 *)((char *)scratch + (((size_t)rows * 4 + 255) & ~(size_t)255));
        hipError_t ce = launch_f32_rows_to_f16(s, (const float *)a + (size_t)r0 * w.k, a16, nullptr, row_scale, rows, w.k);
        if (ce != hipSuccess) return ce;
        OutSpec o = out;
        o.row_scale = row_scale;
        for (uint32_t i = 0; i < o.count; i++) o.seg[i].ptr += (size_t)r0 * o.seg[i].width;
        if (o.swiglu) o.swiglu += (size_t)r0 * (w.n / 2);
        size_t used = (size_t)((char *)a16 - (char *)scratch) + (((size_t)rows * w.k * 2 + 255) & ~(size_t)255);
        hipError_t e = run(a16, rows, o, (char *)scratch + used, scratch_bytes - used, after_sum);
        if (e != hipSuccess) return e;
        if (!after_sum) {
            const PrefillPlan plan = plan_prefill_within(rows, block_rows == 192 && o.swiglu ? 128u : block_rows, splits, w.n_tiles, w.k_chunks,
                                                         scratch_bytes - used, false);
            const uint32_t cps = (w.k_chunks + plan.splits - 1) / plan.splits;
            if ((w.k_chunks + cps - 1) / cps == 1) {  // (with a K-split the sum kernel has applied the factors)
                hipLaunchKernelGGL(k_scale_rows, dim3(rows), dim3(256), 0, s, o, (const float *)row_scale);
                e = hipGetLastError();
                if (e != hipSuccess) return e;
            }
        }
    }
    return hipGetLastError();
}

}  // namespace twm

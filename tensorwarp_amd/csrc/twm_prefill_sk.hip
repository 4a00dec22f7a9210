// Prefill GEMM for large M with stream-K scheduling: C[M,N] = A[M,K] * dequant(W), FP16 MFMA, FP32 accumulation.
//
// Semantics and arithmetic as k_prefill (twm_prefill.hip): gemm_q4_0 (crates/kernels/src/quantize.rs:1825-1858) on the
// reference's Q4 unpack to FP16, f16_rne(f32(scale) * (q - 8)) (quantize.rs:534-571), one f32 accumulator over K.
//
// What differs is the decomposition.  A workgroup tile is 16 MT rows x 256 columns (MT = 16: 256 rows, so every unpacked
// weight feeds sixteen row blocks and the unpack costs half as many vector instructions per MFMA as with 128 rows; a
// single wave per SIMD issues everything, and those instructions are what keeps the MFMA pipe waiting).  Such tiles are
// few (M = 2048, N = 11008: 344), so the work is not dealt out by tile: the (tile, 128-deep k-chunk) units are numbered
// tile-major, and each of the `workers` workgroups (one per CU) takes an equal, contiguous range of units.  A range
// covers the tail of one tile, whole tiles, and the head of another; a tile cut between workers is finished by the
// last of them to arrive: the others park their partial sums in scratch memory and bump the tile's counter, the last
// one adds the parked sums to its own and stores the tile.  With two contributors (the usual case) the sum does not
// depend on who is last (a + b = b + a); with more, everybody parks and the last one adds the parts in worker order:
// results are run-to-run identical.  Nobody ever waits for another workgroup.
//
// Parked sums and counters cross XCDs inside one launch: they are written and read with agent-scope relaxed atomics
// (coherent at the device level by themselves), a workgroup bumps the counter only after s_waitcnt vmcnt(0) has seen
// its stores complete, and the finisher reads only after it has seen the count.
//
// Inner loop per chunk and wave (4 waves, wave w owns 64 columns for all rows): the A tile goes global -> LDS directly
// (double buffered, XOR-swizzled rows), B nibbles and scales go to registers one chunk ahead (two slots), A operands are
// read from LDS three units ahead into a ring of four registers sets (a unit = one row block's four MFMAs), which keeps
// 16 MT accumulators + about 150 other registers inside the 512 a lone wave may use.
#include "twm_prefill_core.h"

#include <type_traits>

namespace twm {

namespace {

__host__ __device__ __forceinline__ uint32_t sk_unit_begin(uint32_t w, uint32_t workers, uint32_t units)
{
    return (uint32_t)(((uint64_t)w * units) / workers);
}

// the worker whose range holds `unit`: the largest w with floor(w * units / workers) <= unit
__device__ __forceinline__ uint32_t sk_worker_of(uint32_t unit, uint32_t workers, uint32_t units)
{
    return (uint32_t)((((uint64_t)unit + 1u) * workers - 1u) / units);
}

}  // namespace

template <int MT>
__global__ __launch_bounds__(256) void k_prefill_sk(const uint4v *__restrict__ qw, const uint2v *__restrict__ sc,
                                                     const _Float16 *__restrict__ a_any, OutSpec out, uint32_t m_rows,
                                                     uint32_t k, uint32_t n, uint32_t n_tiles, uint32_t k_chunks,
                                                     uint32_t row_blocks, uint32_t col_blocks, uint32_t units, float *__restrict__ partials,
                                                     unsigned *__restrict__ counters)
{
    constexpr int kTileHalves = 16 * MT * kPfRowStride;  // one A tile in LDS
    constexpr int NV = MT;                               // direct-to-LDS loads per wave and A tile
    constexpr int kRegs = MT * 4;                        // float4 accumulators per lane
    // two A tiles, then one word for the fix-up's flag (no static LDS beside it: the dynamic block must start at
    // offset 0, 16-byte aligned, for the 16-byte LDS accesses below)
    extern __shared__ __attribute__((aligned(16))) _Float16 a_lds[];
    int &s_flag = *(int *)(a_lds + 2 * kTileHalves);

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t c = lane & 15u, kb = lane >> 4;

    // Worker id: workgroups reach the eight XCDs in turn by linear id; XCD x takes the x-th eighth of the workers, i.e.
    // a contiguous stretch of the unit list, so that the tiles it works on at any time are neighbours (tiles are
    // numbered down the rows first: neighbours share the weights' column block and walk through K together).
    const uint32_t workers = gridDim.x;
    const uint32_t share = workers >> 3, rest = workers & 7u, x8 = blockIdx.x & 7u;
    const uint32_t wid = x8 * share + (x8 < rest ? x8 : rest) + (blockIdx.x >> 3);
    const uint32_t u_begin = sk_unit_begin(wid, workers, units), u_end = sk_unit_begin(wid + 1u, workers, units);

    const PfConsts dq = make_pf_consts();
    const uint32_t a_vec = (lane & 15u) ^ ((4u * wave + (lane >> 4)) & 15u);
    const uint32_t q_off = lane * 16u, s_off = c * 8u;
    uint32_t rd_off[4];  // row c of a row block, vector 4 g + kb of the chunk -> slot (4 g + kb) ^ c
#pragma unroll
    for (int g = 0; g < 4; g++) rd_off[g] = c * kPfRowStride + (((4u * g + kb) ^ c) * 8u);

    for (uint32_t u = u_begin; u < u_end;) {
        const uint32_t tile = u / k_chunks, kc0 = u - tile * k_chunks;
        const uint32_t nchunks = k_chunks - kc0 < u_end - u ? k_chunks - kc0 : u_end - u;
        const uint32_t last = nchunks - 1;
        const bool first_segment = u == u_begin;
        // tiles are numbered band by band (four row blocks high), inside a band column by column: an XCD's stretch of
        // the list is a patch a few row blocks high, whose weights and activations its L2 shares
        const uint32_t band_tiles = 4u * col_blocks, band = tile / band_tiles, ub = tile - band * band_tiles;
        const uint32_t hb = row_blocks - band * 4u < 4u ? row_blocks - band * 4u : 4u;
        const uint32_t bx = ub / hb, by = band * 4u + ub % hb;
        const uint32_t m0 = by * (16u * MT);
        const uint32_t nt0 = (bx * 4u + wave) * 4u;  // first of this wave's four 16-column tiles

        uint32_t nt[4];  // tiles past the end replay the last tile and are never stored
#pragma unroll
        for (int t = 0; t < 4; t++) nt[t] = nt0 + t < n_tiles ? nt0 + t : n_tiles - 1;

        float4v acc[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int t = 0; t < 4; t++) acc[mt][t] = float4v{0.f, 0.f, 0.f, 0.f};
        auto pin_acc = [&]() {  // keeps the accumulators in AGPRs across the loop back edge
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int t = 0; t < 4; t++) asm volatile("" : "+a"(acc[mt][t]));
        };
        pin_acc();

        // A tile: instruction j of wave w fills rows 16 j + 4 w .. + 3 (256 bytes each); slot s of row r holds the row's
        // vector s ^ (r % 16).  Rows past m_rows replay the last row (never stored); vectors past K replay the row's first
        // vector of the chunk, where the padded weights are zero.
        // Group j (16 rows) of a full tile lies j * 16 rows further in A: a uniform offset.  Only the last group that holds
        // a valid row needs its own lane offsets (its rows past m_rows replay its last valid row); groups after it
        // replay it.
        const char *a_blk = (const char *)a_any + (size_t)m0 * k * 2u;
        const uint32_t rows_here = m_rows - m0 < 16u * MT ? m_rows - m0 : 16u * MT;  // >= 1
        const uint32_t jlim = (rows_here - 1u) >> 4, rows_last = rows_here - 16u * jlim;
        const uint32_t lr = 4u * wave + (lane >> 4);
        const uint32_t a_off0 = (lr * k + a_vec * 8u) * 2u;
        const uint32_t a_off_e = ((lr < rows_last ? lr : rows_last - 1u) * k + a_vec * 8u) * 2u;
        auto load_a = [&](uint32_t buf, uint32_t kc, int j) {  // part j of tile kc (relative to kc0) into LDS buffer buf
            const bool inner = (uint32_t)j < jlim;  // (uniform)
            const char *src = a_blk + (size_t)(kc0 + kc) * 256u + (size_t)(inner ? (uint32_t)j : jlim) * 32u * k;
            const uint32_t back = (kc0 + kc) * 128u + a_vec * 8u < k ? 0u : a_vec * 16u;
            __builtin_amdgcn_global_load_lds((const TWM_GLOBAL void *)(src + ((inner ? a_off0 : a_off_e) - back)),
                                             (__attribute__((address_space(3))) void *)(a_lds + buf * kTileHalves +
                                                                                        (16 * j + 4 * wave) * kPfRowStride),
                                             16, 0, 0);
        };
        auto wait_loads = [&]() { __builtin_amdgcn_s_waitcnt(0x0F70); };  // vmcnt(0)

        uint4v bq[2][4];
        uint2v bs[2][4];
        auto load_bq = [&](int slot, uint32_t kc, int t) {
            bq[slot][t] = *(const TWM_GLOBAL uint4v *)(scalar_base(qw, (size_t)((kc0 + kc) * n_tiles + nt[t]) * 1024u) + q_off);
        };
        auto load_bs = [&](int slot, uint32_t kc, int t) {
            bs[slot][t] = *(const TWM_GLOBAL uint2v *)(scalar_base(sc, (size_t)((kc0 + kc) * n_tiles + nt[t]) * 128u) + s_off);
        };
        auto unpack = [&](int slot, int g, PfFrag (&bf)[4], int hp) {  // half fragment hp (tile hp / 2, half hp % 2) of group g
            const int t = hp >> 1;
            pf_unpack_half(bf[t], hp & 1, bq[slot][t][g], bs[slot][t][g >> 1], g & 1, dq);
        };
        auto read_a = [&](uint32_t buf, int g, int mt) {
            return *(const half8 *)(a_lds + buf * kTileHalves + rd_off[g] + mt * 16 * kPfRowStride);
        };
        half8 af0[MT], af1[MT];
        PfFrag bf0[4], bf1[4];
        constexpr int PPU = 8 / MT;  // half fragments unpacked per unit (a unit = one row block's four MFMAs)

        // One step = the MFMAs of one 32-deep group, in MT units of four.  Unit mt also fetches the next group's A operand
        // for its row block, unpacks its share of the next group's B operands and issues `extra(mt)`.
        auto step = [&](const half8 (&af_cur)[MT], const PfFrag (&bf_cur)[4], half8 (&af_nxt)[MT], PfFrag (&bf_nxt)[4],
                        uint32_t rd_buf, int rd_g, int uq_slot, int uq_g, auto extra) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                af_nxt[mt] = read_a(rd_buf, rd_g, mt);
                extra(mt);
#pragma unroll
                for (int p = 0; p < PPU; p++) unpack(uq_slot, uq_g, bf_nxt, mt * PPU + p);
#pragma unroll
                for (int t = 0; t < 4; t++)
                    acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af_cur[mt], bf_cur[t].h, acc[mt][t], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // One chunk (B slot and LDS buffer kc % 2), the schedule of k_prefill: three steps without loads; then wait for
        // this wave's loads (A tile kc + 1 and B of chunk kc + 1, both requested a chunk ago) and the chunk's only
        // barrier; the fourth step already reads the next tile and requests A tile kc + 2 and B of chunk kc + 2.
        auto chunk = [&](auto slot_c, uint32_t kc) {
            constexpr int S = decltype(slot_c)::value, S1 = S ^ 1;
            const uint32_t buf = kc & 1u;
            const uint32_t kc2 = kc + 2 < last ? kc + 2 : last;  // (past the end the last chunk is requested again, unused)
            step(af0, bf0, af1, bf1, buf, 1, S, 1, [&](int) {});
            step(af1, bf1, af0, bf0, buf, 2, S, 2, [&](int) {});
            step(af0, bf0, af1, bf1, buf, 3, S, 3, [&](int) {});
            wait_loads();
            __syncthreads();
            step(af1, bf1, af0, bf0, buf ^ 1u, 0, S1, 0, [&](int u) {
                if (u < NV) load_a(buf, kc2, u);
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    if (t * MT / 4 == u) load_bq(S, kc2, t);
                    if (t * MT / 4 + 1 == u) load_bs(S, kc2, t);
                }
            });
            pin_acc();
        };
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;

        // prologue: tiles 0 and 1 -> LDS, B chunks 0 and 1 -> slots 0 and 1
        const uint32_t kc1p = 1 < last ? 1 : last;
#pragma unroll
        for (int j = 0; j < NV; j++) load_a(0, 0, j);
#pragma unroll
        for (int t = 0; t < 4; t++) {
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
        for (int mt = 0; mt < MT; mt++) af0[mt] = read_a(0, 0, mt);
#pragma unroll
        for (int hp = 0; hp < 8; hp++) unpack(0, 0, bf0, hp);
        __builtin_amdgcn_sched_barrier(0);

        uint32_t kc = 0;
        for (; kc + 2 <= nchunks; kc += 2) {
            chunk(S0{}, kc);
            chunk(S1{}, kc + 1);
        }
        if (kc < nchunks) chunk(S0{}, kc);
        __syncthreads();  // every wave is done with the A tiles: the stores below stage through the same LDS
        pin_acc();

        u += nchunks;

        // ---- a tile cut between workers: park the partial sums, or finish the tile ----
        if (nchunks != k_chunks) {
            const uint32_t w_first = sk_worker_of(tile * k_chunks, workers, units);
            const uint32_t w_last = sk_worker_of(tile * k_chunks + k_chunks - 1u, workers, units);
            constexpr size_t kSlotFloats = (size_t)256 * kRegs * 4;
            auto slot_of = [&](uint32_t w) {  // a worker's first segment parks in its slot 0, its last one in slot 1
                const bool is_first = sk_unit_begin(w, workers, units) >= tile * k_chunks;
                return partials + ((size_t)w * 2u + (is_first ? 0u : 1u)) * kSlotFloats;
            };
            auto park = [&]() {
                uint64_t *dst = (uint64_t *)(first_segment ? partials + (size_t)wid * 2u * kSlotFloats
                                                           : partials + ((size_t)wid * 2u + 1u) * kSlotFloats);
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        union { float4v f; uint64_t q[2]; } v;
                        v.f = acc[mt][t];
                        uint64_t *p = dst + ((size_t)(mt * 4 + t) * 256u + threadIdx.x) * 2u;
                        __hip_atomic_store(p, v.q[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(p + 1, v.q[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                pin_acc();
            };
            auto add_parked = [&](const float *slot) {
                const uint64_t *src = (const uint64_t *)slot;
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        union { float4v f; uint64_t q[2]; } v;
                        const uint64_t *p = src + ((size_t)(mt * 4 + t) * 256u + threadIdx.x) * 2u;
                        v.q[0] = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        v.q[1] = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        acc[mt][t] += v.f;
                    }
            };
            // have all the others parked already?  (Two contributors only: then this workgroup's own sums need not be parked.)
            if (threadIdx.x == 0) s_flag = (int)__hip_atomic_load(&counters[tile], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            bool finish = s_flag == 1;
            __syncthreads();
            if (!finish) {
                park();
                __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have completed
                __syncthreads();
                if (threadIdx.x == 0)
                    s_flag = (int)__hip_atomic_fetch_add(&counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __syncthreads();
                finish = s_flag == 1;  // the second to arrive: both parts are parked
                __syncthreads();
                if (!finish) continue;
                add_parked(slot_of(wid == w_first ? w_last : w_first));
            } else {
                add_parked(slot_of(wid == w_first ? w_last : w_first));
            }
            if (threadIdx.x == 0) __hip_atomic_store(&counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }

        // ---- store the tile: lane (c, kb) holds rows 4 kb + r of row block mt, column 16 tile + c ----
        {
            // one plain [M, N] output, rows 16-byte aligned: each wave turns its 16 x 64 block of a row block through LDS
            // (272-byte rows) so that a lane stores 16 bytes and sixteen lanes cover 256 consecutive bytes of a row
            float *dst = out.seg[0].ptr;
            float *stage = (float *)a_lds + wave * (16 * 68);
            const uint32_t col = nt0 * 16u + (lane & 15u) * 4u;
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
#pragma unroll
                for (int t = 0; t < 4; t++)
#pragma unroll
                    for (int r = 0; r < 4; r++) stage[(kb * 4 + r) * 68 + t * 16 + c] = acc[mt][t][r];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t row = (lane >> 4) + 4u * i;
                    const float4v v = *(const float4v *)(stage + row * 68 + (lane & 15u) * 4u);
                    const uint32_t om = m0 + mt * 16u + row;
                    if (om < m_rows && col < n) __builtin_nontemporal_store(v, (float4v *)(dst + (size_t)om * n + col));
                }
            }
        }
        __syncthreads();  // the staging area is LDS the next segment's tiles land in
    }
}

// Once per device, outside any stream capture: the kernels ask for 64 KB / 128 KB of dynamic LDS.
hipError_t init_prefill_sk()
{
    const int tile = 16 * kPfRowStride * (int)sizeof(_Float16);  // one 16-row block of an A tile
    return hipFuncSetAttribute((const void *)k_prefill_sk<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 8 * tile + 16);
}

size_t prefill_sk_scratch_bytes(uint32_t block_rows, uint32_t workers)
{
    return (size_t)workers * 2u * 256u * (block_rows / 16u) * 4u * 16u;  // two slots per worker, 16 bytes per lane and accumulator
}

// a16: f16 activations [m, K].  block_rows 128 or 256; workers = workgroups (one per CU).  `partials` must hold
// prefill_sk_scratch_bytes(block_rows, workers); counters: one per tile, zero between launches.
hipError_t launch_prefill_sk(hipStream_t s, const WeightView &w, const _Float16 *a16, uint32_t m, const OutSpec &out,
                             uint32_t block_rows, uint32_t workers, float *partials, size_t partial_bytes,
                             unsigned *counters, uint32_t n_counters)
{
    if (m == 0 || w.n == 0) return hipSuccess;
    if (block_rows != 128 || workers == 0 || out.swiglu || !a16) return hipErrorInvalidValue;
    const uint32_t col_blocks = (w.n_tiles + 15) / 16, row_blocks = (m + block_rows - 1) / block_rows;
    const uint64_t tiles = (uint64_t)col_blocks * row_blocks, units = tiles * w.k_chunks;
    if (tiles > n_counters || units > 0x7FFFFFFFu || w.k_chunks == 0) return hipErrorInvalidValue;
    // one plain [M, N] output with 16-byte aligned rows (anything else takes the plain kernel)
    const bool row_store = out.count == 1 && out.seg[0].start == 0 && out.seg[0].width == w.n && !out.seg[0].bias &&
                           w.n % 4 == 0 && ((uintptr_t)out.seg[0].ptr & 15) == 0;
    if (!row_store) return hipErrorInvalidValue;
    // A tile may be cut between two workers at most (the kernel's fix-up adds exactly one parked part): ranges at least
    // a tile long (workers <= tiles), or exactly two workers per tile.
    if (tiles < workers) workers = 2 * tiles <= workers ? (uint32_t)(2 * tiles) : (uint32_t)tiles;
    if (!partials || partial_bytes < prefill_sk_scratch_bytes(block_rows, workers)) return hipErrorInvalidValue;
    const size_t lds = (size_t)2 * block_rows * kPfRowStride * sizeof(_Float16) + 16;
    hipLaunchKernelGGL((k_prefill_sk<8>), dim3(workers), dim3(256), lds, s, (const uint4v *)w.qw, (const uint2v *)w.sc, a16, out,
                           m, w.k, w.n, w.n_tiles, w.k_chunks, row_blocks, col_blocks, (uint32_t)units, partials, counters);
    return hipGetLastError();
}

}  // namespace twm

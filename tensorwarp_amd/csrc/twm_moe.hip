// Expert-bank GEMVs for mixture-of-experts decode: every expert of a layer shares (K, N) and lives in one
// allocation in the column-lane order of twm_gemv4.hip; the expert of a launch slot is read from device
// memory (the router's top-k ids, stored as f32 like the reference's), so no id ever travels to the host.
//
//   k_bank_gemv      C[slot][n] = A x W[ids[slot]]              (batched_marlin_gate_up,
//                    crates/kernels/src/moe_batched_marlin.rs:20-74; with one slot it is the device-indexed
//                    GEMV of quantize_indirect.rs:185-253).  On a bank built in the paired gate/up column
//                    order the store applies gelu_tanh(gate) * up (batched_marlin_split_geglu, :137-151) or
//                    silu(gate) * up, and the [slot][2*dim] intermediate never reaches memory.
//   k_bank_down_axpy acc[n] += sum over slots, in slot order, of weight[slot] * (A[slot] x W[ids[slot]])
//                    (batched_marlin_down_axpy, :78-134, whose float atomics add in no fixed order).
//
// Arithmetic per output as in the dense kernel: f16 activations (f32 ones are rounded on load), exact
// q - 8, f32 sum per 32-wide group times f32(scale).  An id outside [0, experts) contributes zeros.
#include "twm_gemv4_core.h"

namespace twm {

template <int ACT>
__device__ __forceinline__ float gate_mul(float g, float u)
{
    return ACT == 1 ? gelu_mul_f32(g, u) : silu_mul_f32(g, u);
}

// float id -> expert index, or experts (= "none") when it is not a valid index
__device__ __forceinline__ uint32_t expert_of(float id, uint32_t experts)
{
    return (id >= 0.f && id < (float)experts) ? (uint32_t)id : experts;
}

// Both kernels work on sub-tiles of SUB = 16 or 32 columns (see twm_gemv4_core.h): a wave covers 64 / SUB
// consecutive chunks of them in one pass, so that the short K of an expert matrix (a few chunks) still gives
// every wave of a workgroup one pass and the launch many workgroups.

// Workgroup = `waves` waves on one sub-tile of one slot's expert; wave w takes passes w, w + waves, ...
// grid = (sub-tiles, slots).  ACT 0: out[slot][n]; 1 / 2: paired bank (each 64-column tile is 32 gate columns,
// then the up columns of the same features; the workgroup takes SUB / 2 of each),
// out[slot][n/2] = gelu_tanh / silu (gate) * up.
template <int SUB, bool AF32, int ACT, bool ONE>
__global__ __launch_bounds__(1024) void k_bank_gemv(const char *__restrict__ bank, size_t expert_bytes, uint32_t experts,
                                                     const void *__restrict__ a_any, uint32_t a_slot_stride,
                                                     const float *__restrict__ ids, float *__restrict__ out,
                                                     uint32_t k, uint32_t n, uint32_t k_chunks, uint32_t sub_tiles)
{
    constexpr int CPP = 64 / SUB;
    constexpr int TERMS = AF32 ? kTermsOneRowF32 : kTermsOne;   // one row: f32 activations as two f16 terms of one shared piece per lane
    extern __shared__ float red[];  // [waves][64]
    // (gridDim.x is a multiple of 8, workgroups reach the eight XCDs in turn: a contiguous run of sub-tiles per XCD, so
    // that the sub-tiles of a 64-column tile, whose pieces interleave inside the copy's blocks, stream through one L2)
    const uint32_t st = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3), slot = blockIdx.y;
    if (st >= sub_tiles) return;
    const uint32_t waves = blockDim.x >> 6;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u, cl = lane % SUB, cg = lane / SUB;
    const uint32_t tile = st / CPP, part = st % CPP;
    const uint32_t eid = __builtin_amdgcn_readfirstlane(expert_of(ids[slot], experts));
    const uint32_t col = ACT ? (cl / (SUB / 2)) * 32u + part * (SUB / 2) + cl % (SUB / 2) : part * SUB + cl;
    const uint32_t passes = (k_chunks + CPP - 1) / CPP;

    float acc[1] = {0.f};
    if (eid < experts) {
        const char *tbase = bank + (size_t)eid * expert_bytes + (size_t)tile * k_chunks * kColBlockBytes;
        const void *a_row = (const char *)a_any + (size_t)slot * a_slot_stride * (AF32 ? 4 : 2);
        const Gemv4Consts dq = make_gemv4_consts();
        const bool is_lo = (cl & 1u) != 0;
        gemv4s_run_passes<SUB, ONE>(
            wave, waves, passes,
            [&](ChunkS<SUB> &r, uint32_t pass) {
                uint32_t kc = pass * CPP + cg;
                const bool live = kc < k_chunks;
                kc = live ? kc : k_chunks - 1u;
                gemv4s_load_w<SUB>(r, tbase + (size_t)kc * kColBlockBytes, col, live);
                gemv4s_load_a<SUB, AF32, TERMS>(r, a_row, 0, kc, cl, k, is_lo);
            },
            [&](const ChunkS<SUB> &r) { gemv4s_compute<SUB, 1, TERMS>(r, dq, acc); });
    }
    red[wave * 64 + lane] = acc[0];
    __syncthreads();
    auto summed = [&](uint32_t c) {
        float v = 0.f;
        for (uint32_t w = 0; w < waves; w++)
#pragma unroll
            for (int q = 0; q < CPP; q++) v += red[w * 64 + q * SUB + c];
        return v;
    };
    if (ACT == 0) {
        if (threadIdx.x < SUB) {
            uint32_t on = st * SUB + threadIdx.x;
            if (on < n) out[(size_t)slot * n + on] = summed(threadIdx.x);
        }
    } else if (threadIdx.x < SUB / 2) {
        uint32_t dim = n >> 1, feat = tile * 32u + part * (SUB / 2) + threadIdx.x;
        if (feat < dim) out[(size_t)slot * dim + feat] = gate_mul<ACT>(summed(threadIdx.x), summed(SUB / 2 + threadIdx.x));
    }
}

// Workgroup = slots * wps waves on one sub-tile: wave (slot, j) takes passes j, j + wps, ... of its slot's
// expert with its slot's activation row; one thread per column then adds weight[slot] * dot to the accumulator
// slot by slot.
template <int SUB, bool AF32, bool ONE>
__global__ __launch_bounds__(1024) void k_bank_down_axpy(const char *__restrict__ bank, size_t expert_bytes, uint32_t experts,
                                                          const void *__restrict__ a_all, const float *__restrict__ ids,
                                                          const float *__restrict__ weights, float *__restrict__ accum,
                                                          uint32_t k, uint32_t n, uint32_t k_chunks, uint32_t sub_tiles,
                                                          uint32_t slots, uint32_t wps)
{
    constexpr int CPP = 64 / SUB;
    constexpr int TERMS = AF32 ? kTermsOneRowF32 : kTermsOne;
    extern __shared__ float red[];  // [slots * wps][64]
    const uint32_t st = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);  // (a contiguous run per XCD, as in k_bank_gemv)
    if (st >= sub_tiles) return;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u, cl = lane % SUB, cg = lane / SUB;
    const uint32_t tile = st / CPP, part = st % CPP;
    const uint32_t slot = wave / wps, j = wave % wps;
    const uint32_t eid = __builtin_amdgcn_readfirstlane(expert_of(ids[slot], experts));
    const uint32_t passes = (k_chunks + CPP - 1) / CPP;

    float acc[1] = {0.f};
    if (eid < experts) {
        const char *tbase = bank + (size_t)eid * expert_bytes + (size_t)tile * k_chunks * kColBlockBytes;
        const void *a_row = (const char *)a_all + (size_t)slot * k * (AF32 ? 4 : 2);
        const Gemv4Consts dq = make_gemv4_consts();
        const bool is_lo = (cl & 1u) != 0;
        gemv4s_run_passes<SUB, ONE>(
            j, wps, passes,
            [&](ChunkS<SUB> &r, uint32_t pass) {
                uint32_t kc = pass * CPP + cg;
                const bool live = kc < k_chunks;
                kc = live ? kc : k_chunks - 1u;
                gemv4s_load_w<SUB>(r, tbase + (size_t)kc * kColBlockBytes, part * SUB + cl, live);
                gemv4s_load_a<SUB, AF32, TERMS>(r, a_row, 0, kc, cl, k, is_lo);
            },
            [&](const ChunkS<SUB> &r) { gemv4s_compute<SUB, 1, TERMS>(r, dq, acc); });
    }
    red[wave * 64 + lane] = acc[0];
    __syncthreads();
    if (threadIdx.x < SUB) {
        uint32_t on = st * SUB + threadIdx.x;
        if (on < n) {
            float total = accum[on];
            for (uint32_t s = 0; s < slots; s++) {
                float dot = 0.f;
                for (uint32_t q = 0; q < wps; q++)
#pragma unroll
                    for (int c = 0; c < CPP; c++) dot += red[(s * wps + q) * 64 + c * SUB + threadIdx.x];
                total += weights[s] * dot;
            }
            accum[on] = total;
        }
    }
}

// ---- the same two launches on the reference's own slabs (no bank, nothing repacked) --------------------------
// batched_marlin_gate_up / batched_marlin_down_axpy (moe_batched_marlin.rs:20-74, 78-134) take the slab of all experts'
// packed arrays u8 [G][N][16], the slab of their scales f16 [G][N], and per-expert strides; the expert of a slot is
// (int)ids[slot].  gemm_tw_marlin_m1_indirect (quantize_indirect.rs:185-253) takes two u32 offset tables on the device
// and a fixed expert index instead.  Both forms come down to two base addresses per slot.  An id below zero (or NaN),
// where the reference would read before the slab, contributes zeros.  f32 activations as two f16 terms, like the
// dense entry point on the reference's arrays.
struct RawSlab {
    const char *packed;
    const uint16_t *scales;
    uint32_t packed_stride, scales_stride;        // bytes, f16 elements per expert (strided form)
    const uint32_t *packed_offs, *scales_offs;     // device tables: bytes, f16 elements (offset form; null otherwise)
    int index;                                     // offset form: the expert
};

__device__ __forceinline__ bool raw_expert(const RawSlab &e, const float *ids, uint32_t slot, const char *&packed,
                                           const uint16_t *&scales)
{
    if (e.packed_offs) {
        packed = e.packed + e.packed_offs[e.index];
        scales = e.scales + e.scales_offs[e.index];
        return true;
    }
    const float id = ids[slot];
    const bool ok = id >= 0.f;
    const uint64_t x = ok ? (uint64_t)id : 0u;
    packed = e.packed + x * e.packed_stride;
    scales = e.scales + x * e.scales_stride;
    return ok;
}

// grid = (sub-tiles, slots); workgroup = `waves` waves on SUB columns of one slot's expert, wave w takes passes
// w, w + waves, ...; out[slot][n] = A[slot * a_slot_stride ...] x W[expert]
template <int SUB, bool ONE>
__global__ __launch_bounds__(1024) void k_raw_gemv(RawSlab e, const float *__restrict__ a, uint32_t a_slot_stride,
                                                    const float *__restrict__ ids, float *__restrict__ out, uint32_t k,
                                                    uint32_t n, uint32_t k_chunks)
{
    constexpr int CPP = 64 / SUB;
    constexpr int TERMS = kTermsOneRowF32;
    extern __shared__ float red[];  // [waves][64]
    // gridDim.x is a multiple of 8 and workgroups reach the eight XCDs in turn: each XCD takes a contiguous run of
    // sub-tiles, so that the 128-byte lines of the scale rows, which neighbouring sub-tiles share, meet in one L2
    const uint32_t st = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3), slot = blockIdx.y;
    if (st * SUB >= n) return;
    const uint32_t waves = blockDim.x >> 6;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u, cl = lane % SUB, cg = lane / SUB;
    const uint32_t passes = (k_chunks + CPP - 1) / CPP;
    const uint32_t on = st * SUB + cl, col = on < n ? on : n - 1u;
    const char *packed;
    const uint16_t *scales;
    const bool have = raw_expert(e, ids, slot, packed, scales);

    float acc[1] = {0.f};
    if (have) {
        const float *a_row = a + (size_t)slot * a_slot_stride;
        const Gemv4Consts dq = make_gemv4_consts();
        const bool is_lo = (cl & 1u) != 0;
        gemv4s_run_passes<SUB, ONE>(
            wave, waves, passes,
            [&](ChunkS<SUB> &r, uint32_t pass) {
                uint32_t kc = pass * CPP + cg;
                const bool live = kc < k_chunks;
                kc = live ? kc : k_chunks - 1u;
                gemv4s_load_pass_ref<SUB, TERMS, 1>(r, packed, scales, a_row, 0, kc, live, col, on < n, n, k / 32u, cl, k, is_lo);
            },
            [&](const ChunkS<SUB> &r) { gemv4s_compute<SUB, 1, TERMS, true>(r, dq, acc); });
    }
    red[wave * 64 + lane] = acc[0];
    __syncthreads();
    if (threadIdx.x < SUB) {
        const uint32_t o = st * SUB + threadIdx.x;
        if (o < n) {
            float v = 0.f;
            for (uint32_t w = 0; w < waves; w++)
#pragma unroll
                for (int q = 0; q < CPP; q++) v += red[w * 64 + q * SUB + threadIdx.x];
            out[(size_t)slot * n + o] = v;
        }
    }
}

// grid = sub-tiles; workgroup = slots * wps waves: wave (slot, j) takes passes j, j + wps, ... of its slot's expert on
// row slot0 + slot of a_all; one thread per column then adds weight * dot to the accumulator slot by slot.
template <int SUB, bool ONE>
__global__ __launch_bounds__(1024) void k_raw_down_axpy(RawSlab e, const float *__restrict__ a_all, const float *__restrict__ ids,
                                                         const float *__restrict__ weights, float *__restrict__ accum, uint32_t k,
                                                         uint32_t n, uint32_t k_chunks, uint32_t slots, uint32_t wps)
{
    constexpr int CPP = 64 / SUB;
    constexpr int TERMS = kTermsOneRowF32;
    extern __shared__ float red[];  // [slots * wps][64]
    const uint32_t st = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);  // (a contiguous run per XCD, as in k_raw_gemv)
    if (st * SUB >= n) return;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u, cl = lane % SUB, cg = lane / SUB;
    const uint32_t slot = wave / wps, j = wave % wps;
    const uint32_t passes = (k_chunks + CPP - 1) / CPP;
    const uint32_t on = st * SUB + cl, col = on < n ? on : n - 1u;
    const char *packed;
    const uint16_t *scales;
    const bool have = raw_expert(e, ids, slot, packed, scales);

    float acc[1] = {0.f};
    if (have) {
        const float *a_row = a_all + (size_t)slot * k;
        const Gemv4Consts dq = make_gemv4_consts();
        const bool is_lo = (cl & 1u) != 0;
        gemv4s_run_passes<SUB, ONE>(
            j, wps, passes,
            [&](ChunkS<SUB> &r, uint32_t pass) {
                uint32_t kc = pass * CPP + cg;
                const bool live = kc < k_chunks;
                kc = live ? kc : k_chunks - 1u;
                gemv4s_load_pass_ref<SUB, TERMS, 1>(r, packed, scales, a_row, 0, kc, live, col, on < n, n, k / 32u, cl, k, is_lo);
            },
            [&](const ChunkS<SUB> &r) { gemv4s_compute<SUB, 1, TERMS, true>(r, dq, acc); });
    }
    red[wave * 64 + lane] = acc[0];
    __syncthreads();
    if (threadIdx.x < SUB) {
        const uint32_t o = st * SUB + threadIdx.x;
        if (o < n) {
            float total = accum[o];
            for (uint32_t s = 0; s < slots; s++) {
                float dot = 0.f;
                for (uint32_t q = 0; q < wps; q++)
#pragma unroll
                    for (int c = 0; c < CPP; c++) dot += red[(s * wps + q) * 64 + c * SUB + threadIdx.x];
                total += weights[s] * dot;
            }
            accum[o] = total;
        }
    }
}

template <bool PAIRED, int ACT>
__global__ __launch_bounds__(256) void k_gate_rows(const float *__restrict__ gu, float *__restrict__ out, uint32_t dim,
                                                    uint32_t batch)
{
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)batch * dim) return;
    uint32_t b = (uint32_t)(idx / dim), j = (uint32_t)(idx % dim);
    const float *row = gu + (size_t)b * 2 * dim;
    uint32_t cg = PAIRED ? paired_col(j) : j, cu = PAIRED ? cg + kPairWidth : dim + j;
    out[idx] = gate_mul<ACT>(row[cg], row[cu]);
}

hipError_t launch_geglu_rows(hipStream_t s, const float *gu, float *out, uint32_t dim, uint32_t batch, bool paired)
{
    size_t total = (size_t)batch * dim;
    if (total == 0) return hipSuccess;
    dim3 grid((unsigned)((total + 255) / 256));
    if (paired) hipLaunchKernelGGL((k_gate_rows<true, 1>), grid, dim3(256), 0, s, gu, out, dim, batch);
    else hipLaunchKernelGGL((k_gate_rows<false, 1>), grid, dim3(256), 0, s, gu, out, dim, batch);
    return hipGetLastError();
}

// Sub-tile width of the bank kernels (force_sub = 16 or 32 overrides: a tuning knob of the context).  The
// per-slot GEMV runs best on 32 columns once that gives a workgroup per CU (Gemma, Qwen and Mixtral expert
// shapes: 7.0 against 7.6, 5.5 against 5.9, 26.9 against 29.7 us); the down projection, whose workgroups hold
// every slot, on 16 (6.6 against 7.9, 5.6 against 7.6, 15.4 against 18.6 us).
static uint32_t bank_sub(uint32_t n_pad, uint32_t slots, bool per_slot, int force_sub)
{
    if (force_sub == 16 || force_sub == 32) return (uint32_t)force_sub;
    return per_slot && (uint64_t)(n_pad / 32) * slots >= 256 ? 32 : 16;
}

hipError_t launch_bank_gemv(hipStream_t s, const BankView &b, const void *a, bool a_f32, uint32_t a_slot_stride,
                            const float *ids, uint32_t slots, int act, float *out, int force_sub, int force_waves)
{
    if (slots == 0 || b.n == 0) return hipSuccess;
    if (!b.cq || act < 0 || act > 2 || slots > 65535u) return hipErrorInvalidValue;
    if (act != 0 && b.n % (2 * kPairWidth) != 0) return hipErrorInvalidValue;
    const uint32_t sub = bank_sub(b.n_pad, slots, true, force_sub), sub_tiles = b.n_pad / sub;
    const uint32_t passes = (b.k_chunks + 64 / sub - 1) / (64 / sub);
    uint32_t waves = passes < 16 ? passes : 16;
    if (force_waves >= 1 && force_waves <= 16) waves = (uint32_t)force_waves;
    const bool one = passes <= waves;
    dim3 grid(((sub_tiles + 7) / 8) * 8, slots), block(waves * 64);  // (whole rounds of the eight XCDs: see k_bank_gemv)
    size_t lds = (size_t)waves * 64 * sizeof(float);
#define TWM_BANK_LAUNCH(SUBV, F32, A, ONEV)                                                                            \
    hipLaunchKernelGGL((k_bank_gemv<SUBV, F32, A, ONEV>), grid, block, lds, s, (const char *)b.cq, b.expert_bytes,      \
                       b.experts, a, a_slot_stride, ids, out, b.k, b.n, b.k_chunks, sub_tiles)
#define TWM_BANK_ONE(SUBV, F32, A)                  \
    if (one) TWM_BANK_LAUNCH(SUBV, F32, A, true);   \
    else TWM_BANK_LAUNCH(SUBV, F32, A, false)
#define TWM_BANK_ACT(SUBV, F32)                     \
    if (act == 0) { TWM_BANK_ONE(SUBV, F32, 0); }   \
    else if (act == 1) { TWM_BANK_ONE(SUBV, F32, 1); } \
    else { TWM_BANK_ONE(SUBV, F32, 2); }
    if (sub == 16) {
        if (a_f32) { TWM_BANK_ACT(16, true) } else { TWM_BANK_ACT(16, false) }
    } else {
        if (a_f32) { TWM_BANK_ACT(32, true) } else { TWM_BANK_ACT(32, false) }
    }
#undef TWM_BANK_ACT
#undef TWM_BANK_ONE
#undef TWM_BANK_LAUNCH
    return hipGetLastError();
}

hipError_t launch_bank_down_axpy(hipStream_t s, const BankView &b, const void *a_all, bool a_f32, const float *ids,
                                 const float *weights, uint32_t slots, float *accum, int force_sub, int force_waves)
{
    if (slots == 0 || b.n == 0) return hipSuccess;
    if (!b.cq || slots > (uint32_t)kMaxBankSlots) return hipErrorInvalidValue;
    const uint32_t sub = bank_sub(b.n_pad, slots, false, force_sub), sub_tiles = b.n_pad / sub;
    const uint32_t passes = (b.k_chunks + 64 / sub - 1) / (64 / sub);
    uint32_t wps = 16 / slots;                // waves per slot: up to one per pass, sixteen waves in all
    if (wps > passes) wps = passes;
    if (force_waves >= 1 && (uint32_t)force_waves * slots <= 16) wps = (uint32_t)force_waves;
    if (wps == 0) wps = 1;
    const bool one = passes <= wps;
    const uint32_t waves = slots * wps;
    size_t lds = (size_t)waves * 64 * sizeof(float);
#define TWM_DOWN_LAUNCH(SUBV, F32, ONEV)                                                                               \
    hipLaunchKernelGGL((k_bank_down_axpy<SUBV, F32, ONEV>), dim3(((sub_tiles + 7) / 8) * 8), dim3(waves * 64), lds, s, (const char *)b.cq, \
                       b.expert_bytes, b.experts, a_all, ids, weights, accum, b.k, b.n, b.k_chunks, sub_tiles, slots, wps)
#define TWM_DOWN_ONE(SUBV, F32)                  \
    if (one) TWM_DOWN_LAUNCH(SUBV, F32, true);   \
    else TWM_DOWN_LAUNCH(SUBV, F32, false)
    if (sub == 16) {
        if (a_f32) { TWM_DOWN_ONE(16, true); } else { TWM_DOWN_ONE(16, false); }
    } else {
        if (a_f32) { TWM_DOWN_ONE(32, true); } else { TWM_DOWN_ONE(32, false); }
    }
#undef TWM_DOWN_ONE
#undef TWM_DOWN_LAUNCH
    return hipGetLastError();
}

static RawSlab raw_slab(const RawView &v)
{
    RawSlab e;
    e.packed = (const char *)v.packed;
    e.scales = v.scales;
    e.packed_stride = v.packed_stride;
    e.scales_stride = v.scales_stride;
    e.packed_offs = v.packed_offs;
    e.scales_offs = v.scales_offs;
    e.index = v.index;
    return e;
}

hipError_t launch_raw_gemv(hipStream_t s, const RawView &v, const float *a, uint32_t a_slot_stride, const float *ids,
                           uint32_t slots, float *out, int force_sub, int force_waves)
{
    if (slots == 0 || v.n == 0) return hipSuccess;
    if (v.k == 0 || v.k % 32 != 0 || slots > 65535u) return hipErrorInvalidValue;
    const uint32_t n_pad = ((v.n + 63) / 64) * 64, k_chunks = (v.k / 32 + 3) / 4;
    const uint32_t sub = bank_sub(n_pad, slots, true, force_sub), sub_tiles = (v.n + sub - 1) / sub;
    const uint32_t passes = (k_chunks + 64 / sub - 1) / (64 / sub);
    uint32_t waves = passes < 16 ? passes : 16;
    if (force_waves >= 1 && force_waves <= 16) waves = (uint32_t)force_waves;
    const bool one = passes <= waves;
    dim3 grid(((sub_tiles + 7) / 8) * 8, slots), block(waves * 64);  // (whole rounds of the eight XCDs: see k_raw_gemv)
    const size_t lds = (size_t)waves * 64 * sizeof(float);
    const RawSlab e = raw_slab(v);
#define TWM_RAW_LAUNCH(SUBV, ONEV) \
    hipLaunchKernelGGL((k_raw_gemv<SUBV, ONEV>), grid, block, lds, s, e, a, a_slot_stride, ids, out, v.k, v.n, k_chunks)
    if (sub == 16) {
        if (one) TWM_RAW_LAUNCH(16, true);
        else TWM_RAW_LAUNCH(16, false);
    } else {
        if (one) TWM_RAW_LAUNCH(32, true);
        else TWM_RAW_LAUNCH(32, false);
    }
#undef TWM_RAW_LAUNCH
    return hipGetLastError();
}

// slots beyond kMaxBankSlots: one launch per sixteen, in slot order on the stream, so the sum keeps its order
hipError_t launch_raw_down_axpy(hipStream_t s, const RawView &v, const float *a_all, const float *ids, const float *weights,
                                uint32_t slots, float *accum, int force_sub, int force_waves)
{
    if (slots == 0 || v.n == 0) return hipSuccess;
    if (v.k == 0 || v.k % 32 != 0) return hipErrorInvalidValue;
    const uint32_t n_pad = ((v.n + 63) / 64) * 64, k_chunks = (v.k / 32 + 3) / 4;
    const RawSlab e = raw_slab(v);
    for (uint32_t s0 = 0; s0 < slots; s0 += kMaxBankSlots) {
        const uint32_t now = slots - s0 < (uint32_t)kMaxBankSlots ? slots - s0 : (uint32_t)kMaxBankSlots;
        const uint32_t sub = bank_sub(n_pad, now, false, force_sub), sub_tiles = (v.n + sub - 1) / sub;
        const uint32_t passes = (k_chunks + 64 / sub - 1) / (64 / sub);
        uint32_t wps = 16 / now;
        if (wps > passes) wps = passes;
        if (force_waves >= 1 && (uint32_t)force_waves * now <= 16) wps = (uint32_t)force_waves;
        if (wps == 0) wps = 1;
        const bool one = passes <= wps;
        const uint32_t waves = now * wps;
        const size_t lds = (size_t)waves * 64 * sizeof(float);
#define TWM_RAW_DOWN(SUBV, ONEV)                                                                                           \
    hipLaunchKernelGGL((k_raw_down_axpy<SUBV, ONEV>), dim3(((sub_tiles + 7) / 8) * 8), dim3(waves * 64), lds, s, e, a_all + (size_t)s0 * v.k, \
                       ids + s0, weights + s0, accum, v.k, v.n, k_chunks, now, wps)
        if (sub == 16) {
            if (one) TWM_RAW_DOWN(16, true);
            else TWM_RAW_DOWN(16, false);
        } else {
            if (one) TWM_RAW_DOWN(32, true);
            else TWM_RAW_DOWN(32, false);
        }
#undef TWM_RAW_DOWN
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    return hipSuccess;
}

}  // namespace twm

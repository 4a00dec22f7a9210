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

// This wave's chunks first, first + stride, ... of one 64-column tile with three register sets: for the short
// K loops of expert matrices (two or three chunks per wave) every load is in flight before the first unpack.
template <bool AF32>
__device__ __forceinline__ void bank_accumulate(const char *tile_base, const void *a_row, uint32_t first, uint32_t stride,
                                                uint32_t k_chunks, uint32_t k, uint32_t lane, float (&acc)[1][1])
{
    const char *wbase[1] = {tile_base};
    const uint32_t lane16 = lane * 16u, lane8 = 4096u + lane * 8u, apiece = (lane >> 2) * 8u;
    const Gemv4Consts dq = make_gemv4_consts();
    constexpr int TERMS = gemv4_terms<AF32, 1>();   // one row: f32 activations as two row-packed terms
    const bool is_lo = (lane & 1u) != 0;
    Chunk4<1> r0, r1, r2;
    uint32_t c0 = first, c1 = first + stride, c2 = first + 2u * stride;
    if (c0 < k_chunks) gemv4_load_chunk<1, AF32, TERMS>(r0, wbase, c0, lane16, lane8, a_row, 0, apiece, k, is_lo);
    if (c1 < k_chunks) gemv4_load_chunk<1, AF32, TERMS>(r1, wbase, c1, lane16, lane8, a_row, 0, apiece, k, is_lo);
    if (c2 < k_chunks) gemv4_load_chunk<1, AF32, TERMS>(r2, wbase, c2, lane16, lane8, a_row, 0, apiece, k, is_lo);
    for (;;) {
        if (c0 >= k_chunks) break;
        gemv4_compute_chunk<1, 1, TERMS>(r0, dq, acc);
        c0 += 3u * stride;
        if (c0 < k_chunks) gemv4_load_chunk<1, AF32, TERMS>(r0, wbase, c0, lane16, lane8, a_row, 0, apiece, k, is_lo);
        if (c1 >= k_chunks) break;
        gemv4_compute_chunk<1, 1, TERMS>(r1, dq, acc);
        c1 += 3u * stride;
        if (c1 < k_chunks) gemv4_load_chunk<1, AF32, TERMS>(r1, wbase, c1, lane16, lane8, a_row, 0, apiece, k, is_lo);
        if (c2 >= k_chunks) break;
        gemv4_compute_chunk<1, 1, TERMS>(r2, dq, acc);
        c2 += 3u * stride;
        if (c2 < k_chunks) gemv4_load_chunk<1, AF32, TERMS>(r2, wbase, c2, lane16, lane8, a_row, 0, apiece, k, is_lo);
    }
}

// Workgroup = `waves` waves on one 64-column tile of one slot's expert; wave w takes chunks w, w + waves, ...
// grid = (tiles64 rounded up to the 8 XCDs, slots).  ACT 0: out[slot][n]; 1 / 2: paired bank,
// out[slot][n/2] = gelu_tanh / silu (gate) * up.
template <bool AF32, int ACT>
__global__ __launch_bounds__(1024) void k_bank_gemv(const char *__restrict__ bank, size_t expert_bytes, uint32_t experts,
                                                     const void *__restrict__ a_any, uint32_t a_slot_stride,
                                                     const float *__restrict__ ids, float *__restrict__ out,
                                                     uint32_t k, uint32_t n, uint32_t k_chunks, uint32_t tiles64)
{
    extern __shared__ float red[];  // [waves][64]
    const uint32_t tile = blockIdx.x, slot = blockIdx.y;
    if (tile >= tiles64) return;
    const uint32_t waves = blockDim.x >> 6;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t eid = __builtin_amdgcn_readfirstlane(expert_of(ids[slot], experts));

    float acc[1][1] = {{0.f}};
    if (eid < experts)
        bank_accumulate<AF32>(bank + (size_t)eid * expert_bytes + (size_t)tile * k_chunks * kColBlockBytes,
                              (const char *)a_any + (size_t)slot * a_slot_stride * (AF32 ? 4 : 2), wave, waves, k_chunks, k,
                              lane, acc);
    red[wave * 64 + lane] = acc[0][0];
    __syncthreads();
    if (ACT == 0) {
        if (threadIdx.x < 64) {
            uint32_t on = tile * 64u + lane;
            if (on < n) {
                float v = 0.f;
                for (uint32_t w = 0; w < waves; w++) v += red[w * 64 + lane];
                out[(size_t)slot * n + on] = v;
            }
        }
    } else {
        // paired order: lanes 0..31 of the tile are gate columns, lanes 32..63 the up columns of the same features
        if (threadIdx.x < 32) {
            uint32_t dim = n >> 1, feat = tile * 32u + lane;
            if (feat < dim) {
                float g = 0.f, u = 0.f;
                for (uint32_t w = 0; w < waves; w++) {
                    g += red[w * 64 + lane];
                    u += red[w * 64 + 32 + lane];
                }
                out[(size_t)slot * dim + feat] = gate_mul<ACT>(g, u);
            }
        }
    }
}

// Workgroup = slots * wps waves on one 64-column tile: wave (slot, j) takes chunks j, j + wps, ... of its
// slot's expert with its slot's activation row; one thread per column then adds weight[slot] * dot to the
// accumulator slot by slot.
template <bool AF32>
__global__ __launch_bounds__(1024) void k_bank_down_axpy(const char *__restrict__ bank, size_t expert_bytes, uint32_t experts,
                                                          const void *__restrict__ a_all, const float *__restrict__ ids,
                                                          const float *__restrict__ weights, float *__restrict__ accum,
                                                          uint32_t k, uint32_t n, uint32_t k_chunks, uint32_t tiles64,
                                                          uint32_t slots, uint32_t wps)
{
    extern __shared__ float red[];  // [slots * wps][64]
    const uint32_t tile = blockIdx.x;
    if (tile >= tiles64) return;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t slot = wave / wps, j = wave % wps;
    const uint32_t eid = __builtin_amdgcn_readfirstlane(expert_of(ids[slot], experts));

    float acc[1][1] = {{0.f}};
    if (eid < experts)
        bank_accumulate<AF32>(bank + (size_t)eid * expert_bytes + (size_t)tile * k_chunks * kColBlockBytes,
                              (const char *)a_all + (size_t)slot * k * (AF32 ? 4 : 2), j, wps, k_chunks, k, lane, acc);
    red[wave * 64 + lane] = acc[0][0];
    __syncthreads();
    if (threadIdx.x < 64) {
        uint32_t on = tile * 64u + lane;
        if (on < n) {
            float total = accum[on];
            for (uint32_t s = 0; s < slots; s++) {
                float dot = 0.f;
                for (uint32_t q = 0; q < wps; q++) dot += red[(s * wps + q) * 64 + lane];
                total += weights[s] * dot;
            }
            accum[on] = total;
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

static uint32_t bank_waves(uint32_t k_chunks)
{
    uint32_t waves = 8;
    while (waves > 1 && k_chunks <= waves / 2) waves /= 2;  // as the dense M <= 4 plan: idle waves only below half
    return waves;
}

hipError_t launch_bank_gemv(hipStream_t s, const BankView &b, const void *a, bool a_f32, uint32_t a_slot_stride,
                            const float *ids, uint32_t slots, int act, float *out)
{
    if (slots == 0 || b.n == 0) return hipSuccess;
    if (!b.cq || act < 0 || act > 2 || slots > 65535u) return hipErrorInvalidValue;
    if (act != 0 && b.n % (2 * kPairWidth) != 0) return hipErrorInvalidValue;
    uint32_t tiles64 = b.n_pad / 64, waves = bank_waves(b.k_chunks);
    dim3 grid(tiles64, slots), block(waves * 64);
    size_t lds = (size_t)waves * 64 * sizeof(float);
#define TWM_BANK_LAUNCH(F32, A)                                                                                        \
    hipLaunchKernelGGL((k_bank_gemv<F32, A>), grid, block, lds, s, (const char *)b.cq, b.expert_bytes, b.experts, a,   \
                       a_slot_stride, ids, out, b.k, b.n, b.k_chunks, tiles64)
    if (a_f32) {
        if (act == 0) TWM_BANK_LAUNCH(true, 0);
        else if (act == 1) TWM_BANK_LAUNCH(true, 1);
        else TWM_BANK_LAUNCH(true, 2);
    } else {
        if (act == 0) TWM_BANK_LAUNCH(false, 0);
        else if (act == 1) TWM_BANK_LAUNCH(false, 1);
        else TWM_BANK_LAUNCH(false, 2);
    }
#undef TWM_BANK_LAUNCH
    return hipGetLastError();
}

hipError_t launch_bank_down_axpy(hipStream_t s, const BankView &b, const void *a_all, bool a_f32, const float *ids,
                                 const float *weights, uint32_t slots, float *accum)
{
    if (slots == 0 || b.n == 0) return hipSuccess;
    if (!b.cq || slots > (uint32_t)kMaxBankSlots) return hipErrorInvalidValue;
    uint32_t wps = 1;
    while (slots * wps * 2 <= 16 && b.k_chunks >= wps * 4) wps *= 2;  // at least two chunks per wave
    uint32_t tiles64 = b.n_pad / 64, waves = slots * wps;
    size_t lds = (size_t)waves * 64 * sizeof(float);
    if (a_f32)
        hipLaunchKernelGGL((k_bank_down_axpy<true>), dim3(tiles64), dim3(waves * 64), lds, s, (const char *)b.cq,
                           b.expert_bytes, b.experts, a_all, ids, weights, accum, b.k, b.n, b.k_chunks, tiles64, slots, wps);
    else
        hipLaunchKernelGGL((k_bank_down_axpy<false>), dim3(tiles64), dim3(waves * 64), lds, s, (const char *)b.cq,
                           b.expert_bytes, b.experts, a_all, ids, weights, accum, b.k, b.n, b.k_chunks, tiles64, slots, wps);
    return hipGetLastError();
}

}  // namespace twm

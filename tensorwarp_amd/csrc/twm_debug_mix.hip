// Profiling aid (twm_debug_mfma_mix): what the matrix pipes of this GPU deliver under the instruction mixes of a W4A16
// prefill block, on constant data -- the ceilings the prefill kernel's design choices were made against.  Nothing of
// the product path calls these kernels.
//
// Form A, "one wave does everything" (the shipped k_prefill): a wave issues 32 v_mfma_f32_16x16x32_f16 per 32-deep
// step (8 row blocks x 4 column tiles) and, between them, the step's other work, selected by bits of `parts`:
//   1 = the Q4 unpack of the next step's four B operands (13 vector instructions per 32-bit word of nibbles),
//   2 = eight ds_read_b128 (the A operands), 4 = four global_load_dwordx4, 8 = four ds_write_b128.
// 256 threads per workgroup; launched on one or two workgroups per CU (one or two waves per SIMD).
//
// Form B, "producers and consumers": 512 threads; waves 0-3 only read their operands from LDS (bit 2: the eight A
// operands, bit 4: also the four B operands) and issue the MFMAs, waves 4-7 load nibbles, unpack them (bit 1) and write
// the f16 B operands to LDS for the next 64-deep interval; one barrier per interval, both operand tiles double buffered
// (96 KB).  This is the arrangement in which the unpack leaves the MFMA-issuing waves.
#include "twm_api_impl.h"
#include "twm_device.h"

using namespace twm;

namespace {

union Frag { uint4v u; half8 h; };

struct MixConsts { uint32_t mask_lo, mask_hi, magic_lo, magic_hi; };
__device__ __forceinline__ MixConsts mix_consts()
{
    MixConsts c = {0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(c.mask_lo), "+s"(c.mask_hi), "+v"(c.magic_lo), "+v"(c.magic_hi));
    return c;
}
// the prefill kernel's unpack of one word: eight nibbles -> eight f16 weights f16(scale * (q - 8))
__device__ __forceinline__ uint4v mix_unpack(uint32_t x, uint32_t scale2, const MixConsts &c)
{
    const half2v b_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f}, b_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    union { uint32_t u[4]; half2v h2[4]; uint4v v; } r;
    union { uint32_t u; half2v h; } s2;
    s2.u = scale2;
    const uint32_t x8 = x >> 8;
    r.u[0] = (x & c.mask_lo) | c.magic_lo;
    r.u[1] = (x & c.mask_hi) | c.magic_hi;
    r.u[2] = (x8 & c.mask_lo) | c.magic_lo;
    r.u[3] = (x8 & c.mask_hi) | c.magic_hi;
    r.h2[0] = (r.h2[0] + b_lo) * s2.h;
    r.h2[1] = (r.h2[1] + b_hi) * s2.h;
    r.h2[2] = (r.h2[2] + b_lo) * s2.h;
    r.h2[3] = (r.h2[3] + b_hi) * s2.h;
    return r.v;
}

template <int PARTS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void k_mix_one_wave(float *out, const uint4v *in, int steps)
{
    __shared__ uint4v lds[4096];   // 64 KB
    constexpr bool UNP = (PARTS & 1) != 0, DR = (PARTS & 2) != 0, GL = (PARTS & 4) != 0, DW = (PARTS & 8) != 0;
    for (int i = threadIdx.x; i < 4096; i += 256) lds[i] = uint4v{(uint32_t)i, 1u, 2u, 3u};
    __syncthreads();
    const MixConsts c = mix_consts();
    half8 a[8];
#pragma unroll
    for (int m = 0; m < 8; m++) {
        const _Float16 v = (_Float16)(threadIdx.x * 0.001f + m);
        a[m] = half8{v, v, v, v, v, v, v, v};
    }
    float4v acc[8][4];
#pragma unroll
    for (int m = 0; m < 8; m++)
#pragma unroll
        for (int t = 0; t < 4; t++) {
            acc[m][t] = float4v{0.f, 0.f, 0.f, 0.f};
            asm volatile("" : "+a"(acc[m][t]));
        }
    uint32_t w[4], sc[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        w[t] = in[threadIdx.x][t];
        sc[t] = in[256 + threadIdx.x][t] | 0x20002000u;
    }
    Frag bf[2][4];
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
        for (int t = 0; t < 4; t++) bf[s][t].u = uint4v{w[t] + s, w[t] + 1u, w[t] + 2u, w[t] + 3u};
    uint4v gl[4] = {}, dr[8] = {};
    const uint4v *gsrc = in + 512 + threadIdx.x;
    for (int it = 0; it < steps; it += 2) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            if (UNP) {
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    bf[s ^ 1][t].u = mix_unpack(w[t], sc[t], c);
                    w[t] += 0x11111111u;
                }
            }
            if (GL) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if ((PARTS & 32) && i < 2) {
                        // (two of the four as direct-to-LDS loads, as k_prefill's A tile: no data comes back to registers)
                        __builtin_amdgcn_global_load_lds((const TWM_GLOBAL void *)(gsrc + ((it >> 1) & 7) * 256 + i * 2048),
                                                         (__attribute__((address_space(3))) void *)(lds + 3072 + (threadIdx.x >> 6) * 64 + i * 256), 16, 0, 0);
                        continue;
                    }
                    w[i] ^= gl[i][0] & 1u;
                    gl[i] = gsrc[((it >> 1) & 7) * 256 + i * 2048];
                }
            }
            if (DR) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    w[i & 3] ^= dr[i][1] & 1u;
                    dr[i] = lds[threadIdx.x + i * 256];
                }
            }
            if (DW) {
#pragma unroll
                for (int i = 0; i < 4; i++) lds[2048 + threadIdx.x + i * 256] = uint4v{w[0], w[1], w[2], w[3]};
            }
#pragma unroll
            for (int m = 0; m < 8; m++)
#pragma unroll
                for (int t = 0; t < 4; t++) acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m], bf[s][t].h, acc[m][t], 0, 0, 0);
            // the other work dealt out between the MFMAs, as k_prefill's units do
            constexpr int Q = UNP ? 7 : 0;  // vector instructions per four MFMAs
            constexpr int q0 = (Q + 3) / 4, q1 = (Q + 2) / 4, q2 = (Q + 1) / 4, q3 = Q / 4;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (GL && i < 4) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                if (DW && i < 4) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                if (DR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (q0 > 0) __builtin_amdgcn_sched_group_barrier(0x002, q0, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (q1 > 0) __builtin_amdgcn_sched_group_barrier(0x002, q1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (q2 > 0) __builtin_amdgcn_sched_group_barrier(0x002, q2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (q3 > 0) __builtin_amdgcn_sched_group_barrier(0x002, q3, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int m = 0; m < 8; m++)
#pragma unroll
            for (int t = 0; t < 4; t++) asm volatile("" : "+a"(acc[m][t]));
    }
    float s = 0.f;
    for (int m = 0; m < 8; m++)
        for (int t = 0; t < 4; t++) s += acc[m][t][0] + acc[m][t][1] + acc[m][t][2] + acc[m][t][3];
    out[blockIdx.x * 512 + threadIdx.x] = s + (float)(w[0] + gl[0][1] + gl[3][1] + dr[0][0] + dr[7][0] + lds[threadIdx.x + 2048][0]);
}

template <int PARTS>
__global__ __launch_bounds__(512) void k_mix_split(float *out, const uint4v *in, int steps)
{
    constexpr int STEPS = 2;               // 32-deep steps per interval (64 deep)
    constexpr int A_STEP = 8 * 64, B_STEP = 16 * 64;   // uint4 per step: 8 row blocks / 16 column tiles x 64 lanes
    extern __shared__ uint4v mix_lds[];    // [2][STEPS][A_STEP], then [2][STEPS][B_STEP]: 96 KB
    uint4v *a_lds = mix_lds, *b_lds = mix_lds + 2 * STEPS * A_STEP;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 2 * STEPS * (A_STEP + B_STEP); i += 512) mix_lds[i] = uint4v{0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
    __syncthreads();
    const int intervals = steps / STEPS;
    if (wave < 4) {
        float4v acc[8][4];
#pragma unroll
        for (int m = 0; m < 8; m++)
#pragma unroll
            for (int t = 0; t < 4; t++) {
                acc[m][t] = float4v{0.f, 0.f, 0.f, 0.f};
                asm volatile("" : "+a"(acc[m][t]));
            }
        Frag af[2][8], bf[2][4];
#pragma unroll
        for (int m = 0; m < 8; m++) af[0][m].u = a_lds[m * 64 + lane];
#pragma unroll
        for (int t = 0; t < 4; t++) bf[0][t].u = b_lds[(wave * 4 + t) * 64 + lane];
        for (int it = 0; it < intervals; it++) {
            const int buf = it & 1;
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                const int cur = s & 1, nxt = cur ^ 1;
                const int ns = (s + 1) % STEPS, nb = (s + 1 == STEPS) ? buf ^ 1 : buf;
                if (s + 1 == STEPS) __syncthreads();   // the next interval's tiles are complete
                const uint4v *ap = a_lds + (nb * STEPS + ns) * A_STEP, *bp = b_lds + (nb * STEPS + ns) * B_STEP;
#pragma unroll
                for (int m = 0; m < 8; m++) {
                    if (PARTS & 2) af[nxt][m].u = ap[m * 64 + lane];
                    if ((PARTS & 16) && m < 4) bf[nxt][m].u = bp[(wave * 4 + m) * 64 + lane];
#pragma unroll
                    for (int t = 0; t < 4; t++) acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[cur][m].h, bf[cur][t].h, acc[m][t], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (!(PARTS & 2)) {
#pragma unroll
                    for (int m = 0; m < 8; m++) af[nxt][m] = af[cur][m];
                }
                if (!(PARTS & 16)) {
#pragma unroll
                    for (int t = 0; t < 4; t++) bf[nxt][t] = bf[cur][t];
                }
            }
#pragma unroll
            for (int m = 0; m < 8; m++)
#pragma unroll
                for (int t = 0; t < 4; t++) asm volatile("" : "+a"(acc[m][t]));
        }
        float s = 0.f;
        for (int m = 0; m < 8; m++)
            for (int t = 0; t < 4; t++) s += acc[m][t][0] + acc[m][t][1] + acc[m][t][2] + acc[m][t][3];
        out[blockIdx.x * 512 + threadIdx.x] = s;
    } else {
        // producer wave p owns the column tiles 4 p .. 4 p + 3; four intervals of nibble loads in flight
        const int p = wave - 4;
        const MixConsts c = mix_consts();
        constexpr int D = 4;
        const uint4v *src = in + p * 256 + lane;
        uint4v w[D][4];
#pragma unroll
        for (int d = 0; d < D - 1; d++)
#pragma unroll
            for (int t = 0; t < 4; t++) w[d][t] = src[d * 1024 + t * 64];
        for (int it0 = 0; it0 < intervals; it0 += D) {
#pragma unroll
            for (int dd = 0; dd < D; dd++) {
                const int it = it0 + dd, nb = (it & 1) ^ 1;
#pragma unroll
                for (int t = 0; t < 4; t++) w[(dd + D - 1) % D][t] = src[((it + D - 1) & 7) * 1024 + t * 64];
                if (PARTS & 1) {
#pragma unroll
                    for (int s = 0; s < STEPS; s++)
#pragma unroll
                        for (int t = 0; t < 4; t++)
                            b_lds[(nb * STEPS + s) * B_STEP + (p * 4 + t) * 64 + lane] = mix_unpack(w[dd][t][s & 3], w[dd][t][3] | 0x20002000u, c);
                }
                __syncthreads();
            }
        }
        out[blockIdx.x * 512 + threadIdx.x] = (float)(w[0][0][0] + w[1][1][1] + w[2][2][2] + w[3][3][3]);
    }
}

template <class K>
int time_mix(twm_ctx *ctx, K kernel, uint32_t blocks, uint32_t threads, size_t lds, int steps, float *out, const uint4v *in, float *tflops)
{
    hipEvent_t e0, e1;
    HIP_TRY(hipEventCreate(&e0), TWM_DEVICE_ERROR, "hipEventCreate");
    HIP_TRY(hipEventCreate(&e1), TWM_DEVICE_ERROR, "hipEventCreate");
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), lds, ctx->stream, out, in, 64);   // (loads the code object, settles the clock)
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), lds, ctx->stream, out, in, steps);
    HIP_TRY(hipEventRecord(e0, ctx->stream), TWM_DEVICE_ERROR, "hipEventRecord");
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), lds, ctx->stream, out, in, steps);
    HIP_TRY(hipEventRecord(e1, ctx->stream), TWM_DEVICE_ERROR, "hipEventRecord");
    HIP_TRY(hipEventSynchronize(e1), TWM_DEVICE_ERROR, "hipEventSynchronize");
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, e0, e1), TWM_DEVICE_ERROR, "hipEventElapsedTime");
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    HIP_TRY(hipGetLastError(), TWM_DEVICE_ERROR, "instruction-mix kernel");
    // MFMA-issuing waves: four per workgroup in both forms; 32 MFMAs of 16 x 16 x 32 per step each
    *tflops = (float)((double)blocks * 4.0 * steps * 32.0 * 16 * 16 * 32 * 2 / (ms * 1e-3) / 1e12);
    return TWM_OK;
}

}  // namespace

extern "C" int twm_debug_mfma_mix(twm_ctx *ctx, int form, int parts, int workgroups_per_cu, int steps, float *tflops)
{
    const char *who = "twm_debug_mfma_mix";
    if (!ctx || !tflops) return api_fail(TWM_INVALID_HANDLE, "%s: null argument", who);
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "%s: a graph capture is open", who);
    if (steps < 64 || steps > (1 << 20) || steps % 16 != 0) return api_fail(TWM_SHAPE_ERROR, "%s: steps must be a multiple of 16 in 64 .. 2^20", who);
    if (workgroups_per_cu < 1 || workgroups_per_cu > 2) return api_fail(TWM_SHAPE_ERROR, "%s: one or two workgroups per CU", who);
    const uint32_t blocks = (uint32_t)ctx->prop.multiProcessorCount * (uint32_t)workgroups_per_cu;
    // inputs and outputs in the context's scratch: 64 KB of words to unpack per interval slot, one float per thread
    const size_t in_bytes = (size_t)(512 + 8 * 2048 + 2048 * 4) * 16, out_bytes = (size_t)blocks * 512 * 4;
    if (ctx->ws_bytes < in_bytes + out_bytes) return api_fail(TWM_MEMORY_ERROR, "%s: the context's scratch is too small", who);
    const uint4v *in = (const uint4v *)ctx->ws;
    float *out = (float *)((char *)ctx->ws + in_bytes);
    HIP_TRY(hipMemsetAsync(ctx->ws, 0x35, in_bytes, ctx->stream), TWM_DEVICE_ERROR, "hipMemsetAsync");
#define TWM_MIX_A(P) case P: return time_mix(ctx, k_mix_one_wave<P>, blocks, 256, 0, steps, out, in, tflops)
#define TWM_MIX_B(P)                                                                                                           \
    case P: {                                                                                                                  \
        HIP_TRY(hipFuncSetAttribute((const void *)k_mix_split<P>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 << 10),        \
                TWM_DEVICE_ERROR, "hipFuncSetAttribute");                                                                      \
        return time_mix(ctx, k_mix_split<P>, blocks, 512, 96 << 10, steps, out, in, tflops);                                    \
    }
    if (form == 0) {
        switch (parts) {
            TWM_MIX_A(0); TWM_MIX_A(1); TWM_MIX_A(3); TWM_MIX_A(5); TWM_MIX_A(7); TWM_MIX_A(15); TWM_MIX_A(39);
        default: break;
        }
    } else if (form == 1) {
        if (workgroups_per_cu != 1) return api_fail(TWM_SHAPE_ERROR, "%s: the split form is one workgroup of eight waves per CU", who);
        switch (parts) {
            TWM_MIX_B(0); TWM_MIX_B(2); TWM_MIX_B(18); TWM_MIX_B(19);
        default: break;
        }
    }
#undef TWM_MIX_A
#undef TWM_MIX_B
    return api_fail(TWM_UNSUPPORTED_OP, "%s: no such form / parts (form 0: 0, 1, 3, 5, 7, 15; form 1: 0, 2, 18, 19)", who);
}

// Device-side vector types shared by the kernel files.
#pragma once
#include "twm_internal.h"

namespace twm {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));

#define TWM_GLOBAL __attribute__((address_space(1)))   // a pointer into device memory, for the builtins that ask for one

// SwiGLU gate of the reference (warp_fused_silu_mul, crates/kernels/src/ops.rs:966-976):
// silu(g) * u with silu(g) = g / (1 + exp(-g)), every step in f32.  One definition for the
// elementwise kernels and for the GEMV epilogue, so that both give the same bits.
__device__ __forceinline__ float silu_mul_f32(float g, float u)
{
    float silu_g = g / (1.0f + expf(-g));
    return silu_g * u;
}

// warp_fused_gelu_mul's gate (crates/kernels/src/ops.rs:1161-1170, the tanh form), used by the reference's
// batched_marlin_split_geglu as well
__device__ __forceinline__ float gelu_mul_f32(float g, float u)
{
    float gelu_g = 0.5f * g * (1.0f + tanhf(0.7978845608f * (g + 0.044715f * g * g * g)));
    return gelu_g * u;
}

// the gate of a paired store: act 1 = gelu_tanh(g) * u, otherwise silu(g) * u (act is uniform over the launch)
__device__ __forceinline__ float gated_mul(uint32_t act, float g, float u)
{
    return act == 1u ? gelu_mul_f32(g, u) : silu_mul_f32(g, u);
}

}  // namespace twm

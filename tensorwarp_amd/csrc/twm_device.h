// Device-side vector types shared by the kernel files.
#pragma once
#include "twm_internal.h"

namespace twm {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));

// SwiGLU gate of the reference (warp_fused_silu_mul, crates/kernels/src/ops.rs:966-976):
// silu(g) * u with silu(g) = g / (1 + exp(-g)), every step in f32.  One definition for the
// elementwise kernels and for the GEMV epilogue, so that both give the same bits.
__device__ __forceinline__ float silu_mul_f32(float g, float u)
{
    float silu_g = g / (1.0f + expf(-g));
    return silu_g * u;
}

}  // namespace twm

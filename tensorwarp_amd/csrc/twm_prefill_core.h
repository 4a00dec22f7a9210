// Building blocks of the prefill GEMM kernel (twm_prefill.hip): the Q4 unpack to MFMA B
// operands, the scalar-base load helper, the generic output store.
#pragma once
#include "twm_device.h"

namespace twm {

constexpr int kPfRowStride = 128;  // halves per LDS row (256 bytes, unpadded: the 16-byte slots of a row are XOR-swizzled)

struct PfConsts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};

__device__ __forceinline__ PfConsts make_pf_consts()
{
    PfConsts c = {0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(c.mask_lo), "+s"(c.mask_hi), "+v"(c.magic_lo), "+v"(c.magic_hi));
    return c;
}

// Pins a uniform address in a scalar register pair so that the load takes it as its scalar base with the
// per-lane part as a 32-bit offset (otherwise the loop-invariant per-lane part is folded into a 64-bit
// vector base and every load costs a 64-bit vector add).
__device__ __forceinline__ const TWM_GLOBAL char *scalar_base(const void *p, size_t byte_offset)
{
    uint64_t v = (uint64_t)p + byte_offset;
    asm("" : "+s"(v));  // not volatile: a volatile asm would cut the scheduling region in two
    return (const TWM_GLOBAL char *)v;
}

// MFMA B operand of one tile and group: eight FP16 weights per lane
union PfFrag {
    uint32_t u[4];
    half2v h2[4];
    half8 h;
};

// Half of a fragment: nibbles 0..3 (half 0) or 4..7 (half 1) of word `w` -> f16(scale * (q - 8)).
// 1024 + q and 64 + q are built by OR-ing the nibble into an f16 mantissa; the subtraction is exact.
// scale_pair holds two groups' f16 scales; `odd` says which one counts (a splat of one half of a register is free: the
// packed multiply selects the half for both of its lanes).
__device__ __forceinline__ void pf_unpack_half(PfFrag &r, int half, uint32_t w, uint32_t scale_pair, int odd, const PfConsts &c)
{
    union { uint32_t u; half2v h; } sp, s2;
    sp.u = scale_pair;
    s2.h = odd ? half2v{sp.h[1], sp.h[1]} : half2v{sp.h[0], sp.h[0]};
    const half2v b_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
    const half2v b_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    if (half) w >>= 8;
    r.u[2 * half] = (w & c.mask_lo) | c.magic_lo;
    r.u[2 * half + 1] = (w & c.mask_hi) | c.magic_hi;
    r.h2[2 * half] = (r.h2[2 * half] + b_lo) * s2.h;
    r.h2[2 * half + 1] = (r.h2[2 * half + 1] + b_hi) * s2.h;
}

__device__ __forceinline__ void pf_store_out(const OutSpec &out, uint32_t m, uint32_t col, float v)
{
#pragma unroll
    for (uint32_t s = 0; s < kMaxSegs; s++) {
        if (s < out.count) {
            uint32_t rel = col - out.seg[s].start;
            if (rel < out.seg[s].width) out.seg[s].ptr[(size_t)m * out.seg[s].width + rel] = out.seg[s].bias ? v + out.seg[s].bias[rel] : v;
        }
    }
}

}  // namespace twm

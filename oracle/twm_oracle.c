/*
 * CPU oracle for the TW-Marlin W4A16 quantized-linear path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the arithmetic of
 * the reference's quantized-linear path so that the HIP kernels can be checked
 * against it.  Only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg may link or call it; the shipped library never does.
 *
 * Every function names the reference source lines it follows.  Paths are
 * relative to the reference checkout (crates/...).
 *
 * Pinning status (what independently checks each function lives in
 * tests/test_oracle.py):
 *   f16<->f32 conversion ........ exhaustive / randomized against numpy's IEEE binary16
 *   quantizers .................. reference generators + nearest-grid-point property
 *   reorder / fuse .............. permutation invariants, numpy twin
 *   dequant f32 / f16 ........... exhaustive 65536 x 16 table against numpy
 *   gemv / gemm ................. closed forms (one-hot, all-8, scale=1), numpy matmul,
 *                                 reference known-answer 4x3x2 matmul
 *   split-K heuristic ........... known-answer table for eleven shapes
 *   split_qkv / split_gate_up ... numpy slicing
 * The reference holds no test of its own for the TW-Marlin GEMV, the reorder,
 * the fuse or the split-K heuristic, so for those "parity" means agreement with
 * the closed forms above, not with a reference-produced vector.
 *
 * Build: see oracle/Makefile (-O2 -ffp-contract=off so that a*b+c is only
 * fused where fmaf() is written).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define TWM_GROUP 32
#define TWM_Q4_0_BLOCK_BYTES 20

/* ------------------------------------------------------------------ */
/* IEEE binary16 <-> binary32                                          */
/* ------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* binary16 -> binary32, exact.  Mirrors `cvt.f32.f16` (quantize.rs:1223) and
 * half::f16::to_f32 (crate half 2.7.1, not vendored in the reference). */
float twmo_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return bits_f32(f32_bits(v) | sign);
    }
    if (exp == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest even, subnormals kept, overflow to
 * inf, NaN stays NaN (quiet).  Mirrors half::f16::from_f32 as called at
 * quantize.rs:944 and gemma_moe_q4.rs:240. */
uint16_t twmo_f32_to_f16(float f)
{
    uint32_t x = f32_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) {                       /* inf / nan */
        if (ax == 0x7F800000u) return sign | 0x7C00u;
        return sign | 0x7E00u | (uint16_t)((ax >> 13) & 0x3FFu);
    }
    if (ax >= 0x477FF000u) return sign | 0x7C00u;  /* >= 65520 rounds to inf */
    if (ax < 0x33000001u) return sign;             /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;     /* 24-bit significand */
    uint32_t shift;
    uint32_t base;
    if (e < -14) {                                 /* subnormal result */
        shift = (uint32_t)(13 + (-14 - e));
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7FFFFFu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    /* a carry out of the mantissa correctly bumps the exponent field */
    return sign | (uint16_t)(base + q);
}

/* ------------------------------------------------------------------ */
/* Quantizers                                                          */
/* ------------------------------------------------------------------ */

/* One group of 32 values -> scale (f32) + 16 packed bytes.
 * quantize.rs:444-463 and gemma_moe_q4.rs:235-250 are the same arithmetic:
 *   amax = fold(0, max) of |v|   (NaN-ignoring, like f32::max)
 *   scale = amax / 7 ; inv = scale != 0 ? 7 / amax : 0
 *   q = clamp((int)roundf(v * inv) + 8, 0, 15)   roundf = half away from zero
 *   byte i = q[2i] | q[2i+1] << 4 */
static void quantize_group(const float *vals, float *scale_out, uint8_t *bytes)
{
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) {
        float a = fabsf(vals[i]);
        if (a > amax) amax = a;       /* NaN compares false: ignored, as f32::max does */
    }
    float scale = amax / 7.0f;
    float inv = (scale != 0.0f) ? 7.0f / amax : 0.0f;
    *scale_out = scale;
    for (int i = 0; i < 16; i++) {
        float r0 = roundf(vals[2 * i] * inv);
        float r1 = roundf(vals[2 * i + 1] * inv);
        /* Rust `as i32` saturates and maps NaN to 0 */
        int q0 = (r0 != r0) ? 0 : (r0 > 2147483520.0f ? 2147483647 : (r0 < -2147483648.0f ? (-2147483647 - 1) : (int)r0));
        int q1 = (r1 != r1) ? 0 : (r1 > 2147483520.0f ? 2147483647 : (r1 < -2147483648.0f ? (-2147483647 - 1) : (int)r1));
        long long t0 = (long long)q0 + 8, t1 = (long long)q1 + 8;
        if (t0 < 0) t0 = 0; if (t0 > 15) t0 = 15;
        if (t1 < 0) t1 = 0; if (t1 > 15) t1 = 15;
        bytes[i] = (uint8_t)((uint8_t)t0 | ((uint8_t)t1 << 4));
    }
}

/* cpu_quantize_tw_marlin, gemma_moe_q4.rs:218-254.
 * data: row-major [N, K] f32.  packed: u8[G][N][16].  scales: f16[G][N]. */
void twmo_quantize_tw_marlin_nk(const float *data, uint32_t k, uint32_t n,
                                uint8_t *packed, uint16_t *scales)
{
    uint32_t G = k / TWM_GROUP;
    for (uint32_t col = 0; col < n; col++) {
        for (uint32_t g = 0; g < G; g++) {
            float vals[32];
            for (int i = 0; i < 32; i++)
                vals[i] = data[(size_t)col * k + (size_t)g * 32 + i];
            float scale;
            quantize_group(vals, &scale, packed + ((size_t)g * n + col) * 16);
            scales[(size_t)g * n + col] = twmo_f32_to_f16(scale);
        }
    }
}

/* cpu_quantize_q4_col_major, gemma_moe_q4.rs:259-294.
 * data: row-major [N, K].  out: 20-byte blocks at (col*G + b)*20. */
void twmo_quantize_q4_col_major_nk(const float *data, uint32_t k, uint32_t n, uint8_t *out)
{
    uint32_t G = k / TWM_GROUP;
    for (uint32_t col = 0; col < n; col++) {
        for (uint32_t b = 0; b < G; b++) {
            float vals[32];
            for (int i = 0; i < 32; i++)
                vals[i] = data[(size_t)col * k + (size_t)b * 32 + i];
            uint8_t *blk = out + ((size_t)col * G + b) * TWM_Q4_0_BLOCK_BYTES;
            float scale;
            quantize_group(vals, &scale, blk + 4);
            memcpy(blk, &scale, 4);
        }
    }
}

/* quantize_weights_q4_0, quantize.rs:414-474, with the block placement its own
 * doc comment (quantize.rs:410-413) and every consumer (quantize.rs:217, 554,
 * 932) use: column-major, (j*G + b)*20.  The function body at quantize.rs:435
 * writes (b*N + j)*20 instead; `block_major != 0` selects that placement.
 * weights: row-major [K, N] f32. */
void twmo_quantize_weights_q4_0_kn(const float *w, uint32_t k, uint32_t n,
                                   uint8_t *out, int block_major)
{
    uint32_t G = k / TWM_GROUP;
    for (uint32_t j = 0; j < n; j++) {
        for (uint32_t b = 0; b < G; b++) {
            float vals[32];
            for (int i = 0; i < 32; i++)
                vals[i] = w[((size_t)b * 32 + i) * n + j];
            size_t off = block_major ? ((size_t)b * n + j) : ((size_t)j * G + b);
            uint8_t *blk = out + off * TWM_Q4_0_BLOCK_BYTES;
            float scale;
            quantize_group(vals, &scale, blk + 4);
            memcpy(blk, &scale, 4);
        }
    }
}

/* Linear-block Q4_0 quantize + dequantize of a flat vector; the CPU
 * restatement the reference's own test holds (cpu_q4_0_roundtrip,
 * quantize.rs:2938-2954). */
void twmo_q4_0_roundtrip(const float *in, float *out, size_t len)
{
    for (size_t blk = 0; blk + 32 <= len; blk += 32) {
        float scale;
        uint8_t bytes[16];
        quantize_group(in + blk, &scale, bytes);
        for (int i = 0; i < 32; i++) {
            int nib = (i & 1) ? (bytes[i / 2] >> 4) : (bytes[i / 2] & 0xF);
            out[blk + i] = scale * (float)(nib - 8);
        }
    }
}

/* ------------------------------------------------------------------ */
/* Format transforms                                                   */
/* ------------------------------------------------------------------ */

/* reorder_to_tw_marlin, quantize.rs:912-956. */
void twmo_reorder_to_tw_marlin(const uint8_t *q4, uint32_t k, uint32_t n,
                               uint8_t *packed, uint16_t *scales)
{
    uint32_t G = k / TWM_GROUP;
    for (uint32_t col = 0; col < n; col++) {
        for (uint32_t g = 0; g < G; g++) {
            const uint8_t *src = q4 + ((size_t)col * G + g) * TWM_Q4_0_BLOCK_BYTES;
            float scale;
            memcpy(&scale, src, 4);
            scales[(size_t)g * n + col] = twmo_f32_to_f16(scale);
            memcpy(packed + ((size_t)g * n + col) * 16, src + 4, 16);
        }
    }
}

/* fuse_tw_marlin_n, quantize.rs:1018-1063.  `count` matrices sharing K. */
void twmo_fuse_tw_marlin_n(const uint8_t *const *packed_in, const uint16_t *const *scales_in,
                           uint32_t k, const uint32_t *ns, uint32_t count,
                           uint8_t *packed_out, uint16_t *scales_out)
{
    uint32_t G = k / TWM_GROUP;
    size_t total = 0;
    for (uint32_t i = 0; i < count; i++) total += ns[i];
    for (uint32_t g = 0; g < G; g++) {
        size_t off = 0;
        for (uint32_t i = 0; i < count; i++) {
            size_t ni = ns[i];
            memcpy(packed_out + ((size_t)g * total + off) * 16,
                   packed_in[i] + (size_t)g * ni * 16, ni * 16);
            memcpy(scales_out + (size_t)g * total + off,
                   scales_in[i] + (size_t)g * ni, ni * 2);
            off += ni;
        }
    }
}

/* split_qkv / split_gate_up, ops.rs:2255-2297. */
void twmo_split_qkv(const float *qkv, float *q, float *kk, float *v,
                    uint32_t h, uint32_t kv, uint32_t batch)
{
    size_t per = (size_t)h + kv + kv;
    for (uint32_t b = 0; b < batch; b++) {
        memcpy(q + (size_t)b * h, qkv + b * per, (size_t)h * 4);
        memcpy(kk + (size_t)b * kv, qkv + b * per + h, (size_t)kv * 4);
        memcpy(v + (size_t)b * kv, qkv + b * per + h + kv, (size_t)kv * 4);
    }
}

void twmo_split_gate_up(const float *gu, float *gate, float *up, uint32_t ffn, uint32_t batch)
{
    for (uint32_t b = 0; b < batch; b++) {
        memcpy(gate + (size_t)b * ffn, gu + (size_t)b * 2 * ffn, (size_t)ffn * 4);
        memcpy(up + (size_t)b * ffn, gu + (size_t)b * 2 * ffn + ffn, (size_t)ffn * 4);
    }
}

/* warp_fused_silu_mul (crates/kernels/src/ops.rs:966-976): g / (1 + expf(-g)) * up, in f32 */
void twmo_silu_mul(const float *gate, const float *up, float *out, size_t count)
{
    for (size_t i = 0; i < count; i++) {
        float g = gate[i];
        float silu_g = g / (1.0f + expf(-g));
        out[i] = silu_g * up[i];
    }
}

/* The GEGLU gate of batched_marlin_split_geglu (crates/kernels/src/moe_batched_marlin.rs:137-151; the same
 * expression as warp_fused_gelu_mul, ops.rs:1161-1170): 0.5 g (1 + tanhf(0.7978845608 (g + 0.044715 g^3))) * up */
void twmo_gelu_mul(const float *gate, const float *up, float *out, size_t count)
{
    for (size_t i = 0; i < count; i++) {
        float g = gate[i];
        float gelu_g = 0.5f * g * (1.0f + tanhf(0.7978845608f * (g + 0.044715f * g * g * g)));
        out[i] = gelu_g * up[i];
    }
}

/* The paired column order of a gate_up weight (no counterpart in the reference, which keeps
 * [gate | up]): output column 64*(j/32) + j%32 is gate column j, the up column j sits 32 further.
 * Stated here as a plain gather so the device kernel has an independent twin. */
void twmo_pair_gate_up(const uint8_t *gate_packed, const uint16_t *gate_scales,
                       const uint8_t *up_packed, const uint16_t *up_scales, uint32_t k, uint32_t ffn,
                       uint8_t *packed_out, uint16_t *scales_out)
{
    uint32_t G = k / TWM_GROUP;
    size_t n2 = (size_t)2 * ffn;
    for (uint32_t g = 0; g < G; g++) {
        for (uint32_t j = 0; j < ffn; j++) {
            size_t src = (size_t)g * ffn + j;
            size_t dg = (size_t)g * n2 + (size_t)(j / 32) * 64 + j % 32;
            size_t du = dg + 32;
            memcpy(packed_out + dg * 16, gate_packed + src * 16, 16);
            memcpy(packed_out + du * 16, up_packed + src * 16, 16);
            scales_out[dg] = gate_scales[src];
            scales_out[du] = up_scales[src];
        }
    }
}

/* warp_argmax (crates/kernels/src/missing_ops.rs:24-39): sequential scan, strict '>' from -1e30 at index 0 */
void twmo_argmax(const float *in, uint32_t rows, uint32_t cols, int32_t *out)
{
    for (uint32_t r = 0; r < rows; r++) {
        float max_val = -1e30f;
        int32_t max_idx = 0;
        for (uint32_t c = 0; c < cols; c++) {
            float v = in[(size_t)r * cols + c];
            if (v > max_val) {
                max_val = v;
                max_idx = (int32_t)c;
            }
        }
        out[r] = max_idx;
    }
}

/* ------------------------------------------------------------------ */
/* Dequant                                                             */
/* ------------------------------------------------------------------ */

static inline int nibble_at(const uint8_t *rec, int i)
{
    /* byte i/2: low nibble = even k, high nibble = odd k (quantize.rs:1209-1216,
     * gemma_moe_q4.rs:249) */
    return (i & 1) ? (rec[i >> 1] >> 4) : (rec[i >> 1] & 0xF);
}

/* w[k][n] = f32(scale[g][n]) * (nib - 8), dense row-major [K, N] f32.
 * The per-element value the GEMV kernels use (quantize.rs:1209-1238). */
void twmo_dequant_f32(const uint8_t *packed, const uint16_t *scales,
                      uint32_t k, uint32_t n, float *out)
{
    uint32_t G = k / TWM_GROUP;
    for (uint32_t g = 0; g < G; g++)
        for (uint32_t col = 0; col < n; col++) {
            float s = twmo_f16_to_f32(scales[(size_t)g * n + col]);
            const uint8_t *rec = packed + ((size_t)g * n + col) * 16;
            for (int i = 0; i < 32; i++)
                out[((size_t)g * 32 + i) * n + col] = s * (float)(nibble_at(rec, i) - 8);
        }
}

/* "Q4 unpack" to FP16: out[k][n] = f16_rne(scale * (nib - 8)), row-major [K, N]
 * (warp_dequant_q4_to_f16, quantize.rs:534-571, with the TW-Marlin FP16 scale
 * widened to f32 in place of the Q4_0 block's f32 scale). */
void twmo_dequant_f16(const uint8_t *packed, const uint16_t *scales,
                      uint32_t k, uint32_t n, uint16_t *out)
{
    uint32_t G = k / TWM_GROUP;
    for (uint32_t g = 0; g < G; g++)
        for (uint32_t col = 0; col < n; col++) {
            float s = twmo_f16_to_f32(scales[(size_t)g * n + col]);
            const uint8_t *rec = packed + ((size_t)g * n + col) * 16;
            for (int i = 0; i < 32; i++)
                out[((size_t)g * 32 + i) * n + col] =
                    twmo_f32_to_f16(s * (float)(nibble_at(rec, i) - 8));
        }
}

/* Same from a Q4_0 column-major buffer with its f32 scale: the function the
 * reference test dequant_q4_to_f16_correctness (quantize.rs:3607-3668) checks. */
void twmo_dequant_q4_0_to_f16(const uint8_t *q4, uint32_t k, uint32_t n, uint16_t *out)
{
    uint32_t G = k / TWM_GROUP;
    for (uint32_t row = 0; row < k; row++)
        for (uint32_t col = 0; col < n; col++) {
            const uint8_t *blk = q4 + ((size_t)col * G + row / 32) * TWM_Q4_0_BLOCK_BYTES;
            float scale;
            memcpy(&scale, blk, 4);
            int q = nibble_at(blk + 4, (int)(row % 32)) - 8;
            out[(size_t)row * n + col] = twmo_f32_to_f16(scale * (float)q);
        }
}

/* ------------------------------------------------------------------ */
/* GEMV / GEMM                                                         */
/* ------------------------------------------------------------------ */

/* cpu_gemm, gemm.rs:162-172: C[i][j] = sum_p A[i][p] * B[p][j], f32, p
 * ascending, separate multiply and add (Rust does not contract). */
void twmo_cpu_gemm(const float *a, const float *b, float *c, size_t m, size_t n, size_t k)
{
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            float sum = 0.0f;
            for (size_t p = 0; p < k; p++)
                sum += a[i * k + p] * b[p * n + j];
            c[i * n + j] = sum;
        }
}

/* The reference GEMV kernels' own order (quantize.rs:1219-1243 split-K,
 * 1274-1296 direct): per group gdot = sequential fused multiply-add over the
 * 32 elements (nvcc/NVRTC contract a*b+c by default), dot += gdot*scale fused,
 * groups ascending inside a split; splits combined in ascending order here
 * (the GPU combines them with atomicAdd in arbitrary order).
 * a: f32 [M][K]; c: f32 [M][N]; row m is an independent GEMV. */
void twmo_gemv_ref_order(const float *a, const uint8_t *packed, const uint16_t *scales,
                         float *c, uint32_t m_rows, uint32_t k, uint32_t n,
                         uint32_t splits)
{
    uint32_t G = k / TWM_GROUP;
    if (splits == 0) splits = 1;
    uint32_t kbps = (G + splits - 1) / splits;
    for (uint32_t m = 0; m < m_rows; m++) {
        const float *arow = a + (size_t)m * k;
        for (uint32_t col = 0; col < n; col++) {
            float total = 0.0f;
            for (uint32_t sp = 0; sp < splits; sp++) {
                uint32_t g0 = sp * kbps, g1 = g0 + kbps;
                if (g1 > G) g1 = G;
                float dot = 0.0f;
                for (uint32_t g = g0; g < g1; g++) {
                    float s = twmo_f16_to_f32(scales[(size_t)g * n + col]);
                    const uint8_t *rec = packed + ((size_t)g * n + col) * 16;
                    float gdot = 0.0f;
                    for (int i = 0; i < 32; i++)
                        gdot = fmaf(arow[g * 32 + i], (float)(nibble_at(rec, i) - 8), gdot);
                    dot = fmaf(gdot, s, dot);
                }
                if (splits == 1) total = dot; else total += dot;
            }
            c[(size_t)m * n + col] = total;
        }
    }
}

/* The M>1 semantic reference (warp_gemm_q4_0, quantize.rs:186-246): per output
 * element one f32 accumulator, k ascending, fused multiply-add of
 * A[m][k] * (scale*q) where scale*q is exact in f32. */
void twmo_gemm_tile_order(const float *a, const uint8_t *packed, const uint16_t *scales,
                          float *c, uint32_t m_rows, uint32_t k, uint32_t n)
{
    uint32_t G = k / TWM_GROUP;
    for (uint32_t m = 0; m < m_rows; m++)
        for (uint32_t col = 0; col < n; col++) {
            float sum = 0.0f;
            for (uint32_t g = 0; g < G; g++) {
                float s = twmo_f16_to_f32(scales[(size_t)g * n + col]);
                const uint8_t *rec = packed + ((size_t)g * n + col) * 16;
                for (int i = 0; i < 32; i++)
                    sum = fmaf(a[(size_t)m * k + g * 32 + i], s * (float)(nibble_at(rec, i) - 8), sum);
            }
            c[(size_t)m * n + col] = sum;
        }
}

/* Truth for error bounds: same sum in f64, rounded once at the end is NOT
 * applied; returns f64 so callers can measure error against it.  Threaded over
 * columns when built with OpenMP. */
void twmo_gemm_f64(const float *a, const uint8_t *packed, const uint16_t *scales,
                   double *c, uint32_t m_rows, uint32_t k, uint32_t n)
{
    uint32_t G = k / TWM_GROUP;
#pragma omp parallel for schedule(static)
    for (int64_t col = 0; col < (int64_t)n; col++) {
        for (uint32_t m = 0; m < m_rows; m++) {
            double sum = 0.0;
            for (uint32_t g = 0; g < G; g++) {
                double s = (double)twmo_f16_to_f32(scales[(size_t)g * n + col]);
                const uint8_t *rec = packed + ((size_t)g * n + col) * 16;
                double gd = 0.0;
                for (int i = 0; i < 32; i++)
                    gd += (double)a[(size_t)m * k + g * 32 + i] * (double)(nibble_at(rec, i) - 8);
                sum += gd * s;
            }
            c[(size_t)m * n + col] = sum;
        }
    }
}

/* The reference's CPU semantics for one projection, composed the way the
 * reference composes them on the CPU: TW-Marlin unpack to a dense f32 [K, N]
 * matrix (gemma_moe_q4.rs:218-254 inverted; quantize.rs:1219-1238), then
 * cpu_gemm (gemm.rs:162-172).  `dense` is caller scratch of K*N floats.
 * This is what bench.py times as cpu_baseline. */
void twmo_linear_dense(const float *a, const uint8_t *packed, const uint16_t *scales,
                       float *dense, float *c, uint32_t m_rows, uint32_t k, uint32_t n)
{
    twmo_dequant_f32(packed, scales, k, n, dense);
    twmo_cpu_gemm(a, dense, c, m_rows, n, k);
}

/* All-host-cores variant of the same arithmetic: columns split over OpenMP
 * threads, each thread runs the reference kernel's per-column loop.  Returns
 * the number of threads used. */
int twmo_gemv_ref_order_mt(const float *a, const uint8_t *packed, const uint16_t *scales,
                           float *c, uint32_t m_rows, uint32_t k, uint32_t n)
{
    uint32_t G = k / TWM_GROUP;
    int used = 1;
#ifdef _OPENMP
    used = omp_get_max_threads();
#endif
#pragma omp parallel for schedule(static)
    for (int64_t col = 0; col < (int64_t)n; col++) {
        for (uint32_t m = 0; m < m_rows; m++) {
            const float *arow = a + (size_t)m * k;
            float dot = 0.0f;
            for (uint32_t g = 0; g < G; g++) {
                float s = twmo_f16_to_f32(scales[(size_t)g * n + col]);
                const uint8_t *rec = packed + ((size_t)g * n + col) * 16;
                float gdot = 0.0f;
                for (int i = 0; i < 32; i++)
                    gdot = fmaf(arow[g * 32 + i], (float)(nibble_at(rec, i) - 8), gdot);
                dot = fmaf(gdot, s, dot);
            }
            c[(size_t)m * n + col] = dot;
        }
    }
    return used;
}

/* ------------------------------------------------------------------ */
/* Split-K heuristic                                                   */
/* ------------------------------------------------------------------ */

/* quantize.rs:1314-1325 (repeated at 1446-1453, 1501-1508, 1746-1750), all in
 * u32 arithmetic. */
void twmo_pick_splits(uint32_t k, uint32_t n, uint32_t *n_blocks_out,
                      uint32_t *splits_out, uint32_t *kbps_out)
{
    uint32_t G = k / TWM_GROUP;
    uint32_t threads = 256u;
    uint32_t n_blocks = (n + threads - 1) / threads;
    uint32_t splits;
    if (k < 2048u || n_blocks >= 128u) {
        splits = 1;
    } else {
        uint32_t target = 256u;
        uint32_t max_splits = G / 8u; if (max_splits < 1u) max_splits = 1u;
        splits = (target + n_blocks - 1) / n_blocks;
        if (splits < 1u) splits = 1u;
        if (splits > max_splits) splits = max_splits;
    }
    *n_blocks_out = n_blocks;
    *splits_out = splits;
    *kbps_out = (G + splits - 1) / splits;
}

/* ------------------------------------------------------------------ */
/* Deterministic synthetic inputs shared by tests and bench            */
/* ------------------------------------------------------------------ */

static inline uint64_t splitmix64(uint64_t *s)
{
    uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* bytes i.i.d. uniform 0..255 (= nibbles uniform 0..15) */
void twmo_fill_packed(uint8_t *dst, size_t bytes, uint64_t seed)
{
    uint64_t s = seed;
    size_t i = 0;
    for (; i + 8 <= bytes; i += 8) { uint64_t r = splitmix64(&s); memcpy(dst + i, &r, 8); }
    if (i < bytes) { uint64_t r = splitmix64(&s); memcpy(dst + i, &r, bytes - i); }
}

static inline double u01(uint64_t *s) { return ((double)(splitmix64(s) >> 11) + 0.5) * (1.0 / 9007199254740992.0); }

/* standard normal by Box-Muller, f32 */
void twmo_fill_normal_f32(float *dst, size_t count, uint64_t seed)
{
    uint64_t s = seed;
    for (size_t i = 0; i < count; i += 2) {
        double u1 = u01(&s), u2 = u01(&s);
        double r = sqrt(-2.0 * log(u1));
        dst[i] = (float)(r * cos(6.283185307179586 * u2));
        if (i + 1 < count) dst[i + 1] = (float)(r * sin(6.283185307179586 * u2));
    }
}

/* f16(N(0,1)) activations */
void twmo_fill_act_f16(uint16_t *dst, size_t count, uint64_t seed)
{
    uint64_t s = seed;
    for (size_t i = 0; i < count; i += 2) {
        double u1 = u01(&s), u2 = u01(&s);
        double r = sqrt(-2.0 * log(u1));
        dst[i] = twmo_f32_to_f16((float)(r * cos(6.283185307179586 * u2)));
        if (i + 1 < count) dst[i + 1] = twmo_f32_to_f16((float)(r * sin(6.283185307179586 * u2)));
    }
}

/* f16(|N(0,1)| * 0.02) scales */
void twmo_fill_scales_f16(uint16_t *dst, size_t count, uint64_t seed)
{
    uint64_t s = seed;
    for (size_t i = 0; i < count; i += 2) {
        double u1 = u01(&s), u2 = u01(&s);
        double r = sqrt(-2.0 * log(u1));
        dst[i] = twmo_f32_to_f16((float)(fabs(r * cos(6.283185307179586 * u2)) * 0.02));
        if (i + 1 < count) dst[i + 1] = twmo_f32_to_f16((float)(fabs(r * sin(6.283185307179586 * u2)) * 0.02));
    }
}

void twmo_f16_to_f32_array(const uint16_t *src, float *dst, size_t count)
{
    for (size_t i = 0; i < count; i++) dst[i] = twmo_f16_to_f32(src[i]);
}

void twmo_f32_to_f16_array(const float *src, uint16_t *dst, size_t count)
{
    for (size_t i = 0; i < count; i++) dst[i] = twmo_f32_to_f16(src[i]);
}

int twmo_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

// Internal declarations shared by the kernel file and the C-ABI host file.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace twm {

// ---- repacked ("wave tile") weight layout ---------------------------------------
// n-tile  = 16 output columns, k-chunk = 4 groups = 128 input features.
//   qw : uint4 [k_chunks][n_tiles][64]   lane l = (kb = l/16, c = l%16); component i of the
//        uint4 is word kb (k = 8*kb .. 8*kb+7) of group 4*kc+i, column 16*nt+c, with its eight
//        nibbles reordered so that bit position 4*p holds k-offset {0,2,4,6,1,3,5,7}[p].
//   sc : uint2 [k_chunks][n_tiles][16]   four f16 scales (groups 4*kc .. 4*kc+3) of column c.
// The k-chunk index is the slow one: waves working on neighbouring n-tiles advance through k
// together, so at any moment the whole GPU reads one contiguous band of the array (DRAM pages
// stay open) instead of thousands of far-apart streams.
// Columns >= N and groups >= G are padded with nibble 8 / scale 0 (weight exactly 0).
constexpr int kTileN = 16;
constexpr int kChunkGroups = 4;
constexpr int kNPadTo = 64;      // N is padded to a multiple of this, so 1, 2 or 4 tiles per block divide
constexpr int kMaxSegs = 4;
constexpr int kMaxStreamM = 32;     // rows per launch of the batched-decode streaming kernel
constexpr uint32_t kColBlockBytes = 4608;  // column-lane copy: 4 x 1024 B of nibbles + 512 B of scales per (tile, chunk)

// Column order of a "paired" gate_up weight: 32 gate columns, then the 32 up columns of the same
// features, and so on, so that every 64-column tile a kernel owns holds both halves of its features.
// Column j of gate sits at paired_col(j), column j of up kPairWidth further.
constexpr uint32_t kPairWidth = 32;
__host__ __device__ __forceinline__ uint32_t paired_col(uint32_t j) { return (j >> 5) * 64u + (j & 31u); }

struct OutSeg {
    float *ptr;
    uint32_t start;  // first fused column of this segment
    uint32_t width;  // number of columns = row stride of ptr
    const float *bias;  // optional [width] f32 added to every row in the store (nullptr: none)
};
struct OutSpec {
    OutSeg seg[kMaxSegs];
    uint32_t count;
    // Paired gate/up weight only: when set, the store writes silu(gate) * up of every feature to
    // swiglu[row][n / 2] instead of the n columns to the segments.
    float *swiglu;
    uint32_t gate_act;  // 1 = gelu_tanh(gate) * up (GEGLU), otherwise silu(gate) * up
    // f32 activations at M >= 5: row r of the activations was scaled by a power of two to sit inside the f16 range
    // (launch_f32_rows_to_f16), and every sum of row r is multiplied by row_scale[r] before bias, gate and store
    // (exact; 1 for a row that needed nothing).  Null: no scaling.
    const float *row_scale;
};

// feature index of internal column `col` of a paired weight (col % 64 < 32: the gate column; + 32: its up column)
__host__ __device__ __forceinline__ uint32_t paired_feature(uint32_t col) { return (col >> 6) * kPairWidth + (col & 31u); }

struct WeightView {
    const void *qw;
    const void *sc;
    const void *cq;  // column-lane copy (see twm_gemv4.hip): 4608-byte blocks [tiles64][k_chunks]
    uint32_t k, n, groups, n_tiles, k_chunks;
};

// Expert bank: `experts` matrices of the same (K, N) in the column-lane order, expert e at cq + e * expert_bytes
struct BankView {
    const void *cq;
    size_t expert_bytes;
    uint32_t experts, k, n, n_pad, k_chunks;
};
// The reference's own expert slabs (nothing repacked): packed u8 [G][N][16] and scales f16 [G][N] per expert, expert x at
// packed + x * packed_stride / scales + x * scales_stride, or -- offset tables set -- the one expert `index` at
// packed + packed_offs[index] (bytes) / scales + scales_offs[index] (f16 elements), the tables read on the device.
struct RawView {
    const uint8_t *packed;
    const uint16_t *scales;
    uint32_t packed_stride, scales_stride;
    const uint32_t *packed_offs, *scales_offs;
    int index;
    uint32_t k, n;
};
constexpr int kMaxBankSlots = 16;   // top-k of the fused down + axpy launch (one wave or more per slot)

struct DecodePlan {
    uint32_t nt;      // tiles per workgroup (1, 2, 4)
    uint32_t waves;   // waves per workgroup (4, 8, 16); they split the workgroup's k-range
    uint32_t splits;  // cross-workgroup split-K factor
    uint32_t lane_col;  // 1: M <= 4 kernel, one lane per column (nt = 64-column tiles per workgroup)
};

// ---- host-side helpers shared by the files that hold C-ABI entry points ---------------
// records the message for twm_last_error() on the calling thread and returns `code`
int api_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// the DeviceError variant of the failure just recorded by api_fail (TWM_KIND_*), where the code alone does not tell
void set_error_kind(int kind);
// K % 32 == 0 and K x N within the ABI's limit, else TWM_SHAPE_ERROR with the message set
int check_kn(const char *who, uint32_t k, uint32_t n);
// What the dispatch of the GEMV on the reference's arrays needs from its caller: the stream, the knobs, and the
// split-K scratch (f32 partial sums and one arrival counter per column tile, zero between launches).
struct M1Env {
    hipStream_t stream;
    int exact, splits, force_sub, force_waves;
    float *ws;
    size_t ws_bytes;
    unsigned *counters;
    uint32_t n_counters;
    bool clear_counters;  // zero the counters a split launch uses first (a scratch shared with unknown earlier calls)
};
int m1_dispatch(const M1Env &env, const char *who, const float *a_dev, const uint8_t *packed_dev,
                const uint16_t *scales_dev, float *c_dev, uint32_t n, uint32_t k);

// twm_noalloc.hip: device address of the no-allocation entry point's static scratch on the current device (looked
// up once per device; twm_ctx_create calls it so that the lookup has happened before any capture); nullptr on failure
void *noalloc_scratch_for_current_device(const char *who);

// Profiling aid (twm_debug_trace): while ptr is set, every launch of the M <= 4 sub-tile kernel with at most
// `capacity` workgroups has each workgroup record four 32-bit words (start, loaded, end on the 100 MHz clock, hardware id).
struct TraceBuf {
    uint32_t *ptr;
    uint32_t capacity;
};

// ---- launchers (all asynchronous on `s`, return the launch status) ---------------
hipError_t launch_fill_zero(hipStream_t s, void *ptr, size_t bytes);
hipError_t launch_quantize_q4_0(hipStream_t s, const float *w_kn, uint32_t k, uint32_t n, uint8_t *q4);
hipError_t launch_reorder(hipStream_t s, const uint8_t *q4, uint32_t k, uint32_t n, uint8_t *packed, uint16_t *scales);
hipError_t launch_quantize_twm(hipStream_t s, const float *w, int w_is_nk, uint32_t k, uint32_t n,
                               uint8_t *packed, uint16_t *scales);
hipError_t launch_fuse_one(hipStream_t s, const uint8_t *packed_in, const uint16_t *scales_in, uint32_t groups,
                           uint32_t ni, uint32_t total_n, uint32_t col_off, uint8_t *packed_out, uint16_t *scales_out);
hipError_t launch_dequant(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                          void *out, bool f16_out);
hipError_t launch_cast(hipStream_t s, const void *src, void *dst, size_t count, bool to_f16);
hipError_t launch_split_qkv(hipStream_t s, const float *qkv, float *q, float *kk, float *v, uint32_t h,
                            uint32_t kv, uint32_t batch);
hipError_t launch_split_gate_up(hipStream_t s, const float *gu, float *g, float *u, uint32_t ffn, uint32_t batch);
hipError_t launch_silu_mul(hipStream_t s, const float *gate, const float *up, float *out, size_t count);
hipError_t launch_swiglu_rows(hipStream_t s, const float *gu, float *out, uint32_t ffn, uint32_t batch, bool paired);
hipError_t launch_pair_gate_up(hipStream_t s, const uint8_t *gate_packed, const uint16_t *gate_scales,
                               const uint8_t *up_packed, const uint16_t *up_scales, uint32_t groups, uint32_t ffn,
                               uint8_t *packed_out, uint16_t *scales_out);
hipError_t launch_argmax(hipStream_t s, const float *in, uint32_t rows, uint32_t cols, int *out, void *scratch,
                         size_t scratch_bytes);
hipError_t launch_ref_gemv(hipStream_t s, const float *a, const uint8_t *packed, const uint16_t *scales, float *c,
                           uint32_t n, uint32_t k, uint32_t splits, uint32_t groups_per_split);
hipError_t launch_repack(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                         void *qw, void *sc, uint32_t n_tiles, uint32_t k_chunks);
hipError_t launch_weight_dequant_f16(hipStream_t s, const WeightView &w, uint16_t *out_kn);
// pair_ffn != 0: the source columns are [gate | up] halves of width pair_ffn and the copy is written in the
// paired order (32 gate, 32 up, ...)
// one repacked copy from the other (n_tiles is a multiple of 4)
hipError_t launch_col_to_tile(hipStream_t s, const void *cq, uint32_t n_tiles, uint32_t k_chunks, void *qw, void *sc);
hipError_t launch_tile_to_col(hipStream_t s, const void *qw, const void *sc, uint32_t n_tiles, uint32_t k_chunks, void *cq);
hipError_t launch_repack_col(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                             void *cq, uint32_t n_pad, uint32_t k_chunks, uint32_t pair_ffn = 0);
hipError_t launch_weight_dequant_f16_col(hipStream_t s, const WeightView &w, uint16_t *out_kn);
// swiglu_out != nullptr (the weight in the paired gate_up column order, N = 2*ffn a multiple of 64): instead
// of the N columns, write silu(gate) * up of every feature to swiglu_out[m][ffn]; `out` is ignored.
hipError_t launch_gemv4s(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                         float *ws, unsigned *counters, uint32_t sub, uint32_t waves, uint32_t splits, TraceBuf trace = TraceBuf{nullptr, 0});
hipError_t launch_gemv4s_ref(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                             const float *a, float *c, float *ws, unsigned *counters, uint32_t sub, uint32_t waves,
                             uint32_t splits);
hipError_t launch_gemv4(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                        float *ws, unsigned *counters, uint32_t nt, uint32_t waves, uint32_t splits,
                        float *swiglu_out = nullptr);
hipError_t launch_gemv4_ref(hipStream_t s, const uint8_t *packed, const uint16_t *scales, uint32_t k, uint32_t n,
                            const float *a, float *c, float *ws, unsigned *counters, uint32_t waves, uint32_t splits);
hipError_t init_prefill();
hipError_t launch_prefill(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                          uint32_t block_rows, uint32_t splits, void *scratch, size_t scratch_bytes);
// out[row][col] = sum over splits (in order) of partials[split][row][col], partials rows n_ld floats wide
hipError_t launch_splitk_reduce(hipStream_t s, const float *partials, const OutSpec &out, uint32_t m, uint32_t n,
                                uint32_t n_ld, uint32_t splits);
hipError_t launch_stream(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                         uint32_t splits, uint32_t waves, float *partials, size_t partial_bytes);
// f32 -> two f16 arrays: hi = f16(a), lo = f16(a - hi)
// f32 activation rows -> f16: hi = f16(a * 2^-s), lo = f16(a * 2^-s - hi) (lo null: the one rounded term only), with a
// power of two per row that brings the row's largest magnitude to [2^13, 2^14) when it lies outside [2^-2, 2^14], and
// row_scale[row] = 2^s for the stores (1 otherwise; a row of zeros, infinities or NaNs is left as it is).
hipError_t launch_f32_rows_to_f16(hipStream_t s, const float *a, _Float16 *hi, _Float16 *lo, float *row_scale, uint32_t rows,
                                  uint32_t k);
// batched decode with the activations shared through LDS (M <= 32); tiles_per_wave 1 or 2, k_slices 1, 2 or 4
hipError_t launch_batch(hipStream_t s, const WeightView &w, const void *a, bool a_f32, uint32_t m, const OutSpec &out,
                        uint32_t splits, uint32_t tiles_per_wave, uint32_t k_slices, uint32_t quads_per_group,
                        bool rounded, float *scratch, size_t scratch_bytes);
// the block form (64, 128, or 192 = 128 rows x 192 columns) and K-split launch_prefill takes for `rows` rows of f16 activations with that much scratch
void prefill_plan_of(uint32_t rows, uint32_t block_rows, uint32_t splits, uint32_t n_tiles, uint32_t k_chunks, size_t ws_bytes,
                     bool gated, uint32_t *block_rows_out, uint32_t *splits_out);
hipError_t launch_geglu_rows(hipStream_t s, const float *gu, float *out, uint32_t dim, uint32_t batch, bool paired);
// act: 0 out[slot][n]; 1 gelu_tanh(gate) * up, 2 silu(gate) * up into out[slot][n/2] (paired bank)
hipError_t launch_bank_gemv(hipStream_t s, const BankView &b, const void *a, bool a_f32, uint32_t a_slot_stride,
                            const float *ids, uint32_t slots, int act, float *out, int force_sub = 0, int force_waves = 0);
hipError_t launch_bank_down_axpy(hipStream_t s, const BankView &b, const void *a_all, bool a_f32, const float *ids,
                                 const float *weights, uint32_t slots, float *accum, int force_sub = 0, int force_waves = 0);

// the same two launches on the reference's slabs, f32 activations (moe_batched_marlin.rs:153-214, quantize_indirect.rs:228-253)
hipError_t launch_raw_gemv(hipStream_t s, const RawView &v, const float *a, uint32_t a_slot_stride, const float *ids,
                           uint32_t slots, float *out, int force_sub = 0, int force_waves = 0);
hipError_t launch_raw_down_axpy(hipStream_t s, const RawView &v, const float *a_all, const float *ids, const float *weights,
                                uint32_t slots, float *accum, int force_sub = 0, int force_waves = 0);

}  // namespace twm

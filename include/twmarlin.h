/*
 * twmarlin.h - C ABI of libtwmarlin_hip.so, the MI355X (gfx950) implementation
 * of TensorWarp's TW-Marlin W4A16 quantized-linear path.
 *
 * The library stands in for vendor/cudarc + the NVRTC kernel strings of
 * crates/kernels/src/quantize.rs on this one path.  Every entry point cites the
 * reference interface it replaces (paths relative to the reference checkout).
 *
 * Conventions (taken from the reference's own C API, crates/kernels/src/c_api.rs:26-67):
 *   - opaque handles, every create paired with a destroy, NULL handles rejected;
 *   - functions return an int status whose values equal c_api.rs `WarpError`;
 *   - nothing panics or aborts across the ABI; twm_last_error() holds the text the
 *     reference would have put in DeviceError::{Init,Memory,Launch}(String)
 *     (crates/kernels/src/device.rs:278-292);
 *   - all work is asynchronous and ordered on the context's stream; the caller
 *     synchronises (device.rs:196-200).  A context must be driven by one host
 *     thread / one stream at a time: split-K scratch memory is per context.
 *   - pointers named *_dev are device pointers (from twm_malloc or any other
 *     hipMalloc-compatible allocator, e.g. a torch tensor's data_ptr()); pointers
 *     named *_host are host pointers.
 *
 * TW-Marlin format (quantize.rs:892-907, 1190-1191; gemma_moe_q4.rs:213-254), G = K/32:
 *   packed : u8  [G][N][16]   byte i of a record = q[32g+2i] | q[32g+2i+1] << 4
 *   scales : f16 [G][N]
 *   weight : w[k][n] = f32(scales[k/32][n]) * (q[k][n] - 8)
 */
#ifndef TWMARLIN_H
#define TWMARLIN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* c_api.rs:41-50 `WarpError` */
enum {
    TWM_OK = 0,
    TWM_DEVICE_ERROR = 1,
    TWM_MEMORY_ERROR = 2,
    TWM_SHAPE_ERROR = 3,
    TWM_UNSUPPORTED_OP = 4,
    TWM_INVALID_HANDLE = 5
};

/* c_api.rs:31-39 `WarpDType` */
enum {
    TWM_F32 = 0,
    TWM_F16 = 1,
    TWM_I32 = 2,
    TWM_I8 = 3,
    TWM_U8 = 4
};

typedef struct twm_ctx twm_ctx;       /* WarpDevice + KernelCache (device.rs, cache.rs) */
typedef struct twm_weight twm_weight; /* one projection's (packed, scales) pair, repacked for gfx950 */
typedef struct twm_graph twm_graph;   /* GraphCapture (cuda_graph.rs:72-118) */

/* ---- library / device ------------------------------------------------------ */

/* c_api.rs:107-112 warp_version */
const char *twm_version(void);
/* c_api.rs:101-105 warp_device_count */
int twm_device_count(void);
/* Text of the last failure on the calling thread ("" if none). */
const char *twm_last_error(void);
/* Which DeviceError variant of the reference (device.rs:278-292: Init, PtxLoad, FuncNotFound, Sync, Memory, Launch) the
 * last failure on the calling thread corresponds to, for a wrapper that maps codes back to that enum: a failed
 * context creation is Init (a device that is not gfx950, for which the library holds no code object, is PtxLoad),
 * a failed synchronise Sync, a failed allocation or copy Memory, everything else that reached the device Launch;
 * argument errors (shape, handle, unsupported) never reached the device and are TWM_KIND_NONE. */
enum {
    TWM_KIND_NONE = 0,
    TWM_KIND_INIT = 1,
    TWM_KIND_CODE_OBJECT = 2,    /* DeviceError::PtxLoad */
    TWM_KIND_FUNC_NOT_FOUND = 3, /* (never raised: kernels are linked into the library) */
    TWM_KIND_SYNC = 4,
    TWM_KIND_MEMORY = 5,
    TWM_KIND_LAUNCH = 6
};
int twm_last_error_kind(void);

/* c_api.rs:52-59 warp_device_create / WarpDevice::new (device.rs) + KernelCache::new.
 * All kernels are precompiled gfx950 code inside the library, so there is no
 * JIT step.  Creates the context's own stream and its split-K scratch.
 * Returns NULL on failure. */
twm_ctx *twm_ctx_create(int ordinal);
/* c_api.rs:61-67 warp_device_destroy */
void twm_ctx_destroy(twm_ctx *ctx);
/* c_api.rs:90-99 warp_device_sync / WarpDevice::synchronize (device.rs:196-200) */
int twm_ctx_sync(twm_ctx *ctx);
/* WarpDevice::with_stream (device.rs:230-265): run subsequent work on a caller-owned
 * hipStream_t (e.g. the stream a framework already uses).  NULL restores the
 * context's own stream. */
int twm_ctx_set_stream(twm_ctx *ctx, void *hip_stream);
/* The hipStream_t work is currently issued on. */
void *twm_ctx_stream(twm_ctx *ctx);
/* Stream objects for a caller that has none of its own (the reference creates its streams through the driver crate,
 * device.rs:230-265): a non-blocking hipStream_t at the default priority on the context's device, to be handed to
 * twm_ctx_set_stream; destroy it only after the context has been pointed elsewhere.  twm_stream_sync blocks until the
 * stream's work is done (a failure reports TWM_KIND_SYNC). */
void *twm_stream_create(twm_ctx *ctx);
int twm_stream_destroy(twm_ctx *ctx, void *hip_stream);
int twm_stream_sync(twm_ctx *ctx, void *hip_stream);
/* c_api.rs:69-80 warp_device_info: fills buf with "<name> | <CUs> CUs | <GiB> GiB". */
int twm_ctx_info(twm_ctx *ctx, char *buf, size_t buf_len);
/* Tuning knobs for per-shape sweeps (the role AutoTuner::tune_gemm plays in
 * crates/kernels/src/autotune.rs:254-396); 0 = library's choice unless noted:
 *   "nt"            column tiles per workgroup of the decode kernels (1, 2, 4)
 *   "waves"         waves per workgroup of the decode kernels (1, 2, 4, 8, 16; streaming kernel 4 or 8)
 *   "sub"           M <= 4 and expert-bank kernels: 1 = whole 64-column tiles per workgroup, 16 or 32 = sub-tiles
 *                   of that many columns (with "waves" waves, default 8), 0 = the planner's choice per shape
 *   "kernel"        decode kernel: 2 = one-lane-per-column kernel on whole 64-column tiles
 *                   (M <= 4 only), 3 = batched-decode streaming kernel (32-row blocks), 4 = batched-decode kernel
 *                   with the activations shared through LDS (32-row blocks; "nt" 1 / 2 = tiles per wave, 4 / 3 =
 *                   two / three column quads per workgroup, "waves" 8 / 16 = two / four k-slices per workgroup)
 *   "dequant_src"   which repacked copy twm_weight_dequant_f16 unpacks: 0 = 16-column tiles, 1 = column lanes
 *   "tune_on_upload" new weight handles (twm_weight_upload, twm_weight_from_device, twm_weight_fuse_n; not the paired
 *                   gate/up handles) get measured plans at once, as if twm_weight_tune had been called on them: 1 = for
 *                   the decode row counts 1, 4, 8, 16, 32; 2 = also for the prefill row counts 128, 512, 2048; 0 (default)
 *                   = no.  Costs about half a second per row count and handle; a handle whose tuning fails is not returned.
 *                   The tuner measures kernels of both repacked orders, so a tuned handle holds both copies whatever
 *                   "weight_copies" says (twm_weight_drop frees one afterwards).
 *   "weight_copies" the repacked orders a new weight handle is given: 0 or 3 = both, 1 = 16-column tiles only,
 *                   2 = column lanes only (twm_weight_ensure)
 *   "sub_waves"     waves per workgroup of the sub-tile kernels when "sub" forces their width (1 .. 16)
 *   "prefill_min_m" smallest M that runs the prefill GEMM (default 33; below it the decode kernels run)
 *   "prefill_bm"    prefill block form: 64 = 64 rows x 256 columns, 128 = 128 x 256, 192 = 128 rows x 192 columns
 *   "m1_exact"      twm_gemm_tw_marlin_m1: 1 = f32 activations and f32 FMAs in the reference kernel's order with
 *                   the reference's split-K rule and float atomics (bit-equal to the reference order when that
 *                   rule yields one split); 0 (default) = the MFMA kernel
 *   "m1_splits"     twm_gemm_tw_marlin_m1: split-K factor of the MFMA kernel (0 .. 64)
 *   "m1_align16"    twm_gemm_tw_marlin_m1: 1 = a call whose activations or packed weights are not 16-byte aligned (a slab
 *                   offset that is only 4-byte aligned, the reference kernel's own limit) returns TWM_SHAPE_ERROR instead
 *                   of silently taking the plain f32 kernel, which is about 3.6 times slower; 0 (default) = take it
 *   "batch_rounded" twm_gemm at M = 17 .. 32: 1 = weights rounded to f16 and summed over K by the MFMAs, the arithmetic
 *                   of the prefill GEMM; 0 (default) = exact weights with f32 group scales as for M <= 16
 * Values outside these sets return TWM_SHAPE_ERROR, unknown keys TWM_UNSUPPORTED_OP. */
int twm_ctx_set_option(twm_ctx *ctx, const char *key, int value);

/* Profiling aid, no counterpart in the reference: while trace_dev is set on a context, every launch of the M = 1
 * sub-tile GEMV kernel (f16 activations) that this context issues with at most capacity_workgroups workgroups runs a
 * traced twin of the kernel (other contexts are not affected),
 * in which workgroup b writes four 32-bit words at trace_dev[4 b]: the GPU's 100 MHz clock at its start, after its
 * first wave has unpacked its weights, and at its end, and the hardware id of the CU it ran on (bits 0-15 HW_ID, bits
 * 16-19 the XCD).  NULL or 0 switches it off; the product kernels carry no trace code. */
int twm_debug_trace(twm_ctx *ctx, uint32_t *trace_dev, uint32_t capacity_workgroups);
/* Profiling aid, no counterpart in the reference: the FP16 matrix throughput (TFLOP/s, into *tflops) that this GPU
 * delivers under the instruction mixes of a W4A16 prefill block, measured on constant data by a kernel of its own, one
 * or two workgroups per CU, `steps` 32-deep steps (a multiple of 16).  form 0: one wave issues the 32 MFMAs of a step
 * and, between them, the parts selected by bits of `parts`: 1 the Q4 unpack of four B operands, 2 eight ds_read_b128,
 * 4 four global_load_dwordx4, 8 four ds_write_b128 (parts 0, 1, 3, 5, 7, 15).  form 1: eight waves per workgroup, four
 * that only read operands from LDS (2: the A operands, 16: the B operands too) and issue MFMAs, four that load, unpack
 * (1) and write the B operands to LDS (parts 0, 2, 18, 19).  Synchronises; uses the context's scratch. */
int twm_debug_mfma_mix(twm_ctx *ctx, int form, int parts, int workgroups_per_cu, int steps, float *tflops);

/* ---- device memory (GpuTensor::{zeros,from_host,to_host}, tensor.rs:9-104) ------ */

void *twm_malloc(twm_ctx *ctx, size_t bytes);
int twm_free(twm_ctx *ctx, void *ptr_dev);
int twm_memcpy_h2d(twm_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes); /* synchronous */
int twm_memcpy_d2h(twm_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes); /* synchronous */
int twm_memcpy_d2d(twm_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes);  /* stream ordered */
/* stream.memset_zeros (quantize.rs:1349); done by a fill kernel so that it may be graph captured */
int twm_memset_zero(twm_ctx *ctx, void *ptr_dev, size_t bytes);

/* ---- timing on the context's stream --------------------------------------------- */

void *twm_event_create(twm_ctx *ctx);
int twm_event_destroy(twm_ctx *ctx, void *event);
int twm_event_record(twm_ctx *ctx, void *event);
/* waits for `stop`, then returns the time between the two records in milliseconds */
int twm_event_elapsed_ms(twm_ctx *ctx, void *start, void *stop, float *ms_out);

/* ---- TW-Marlin format operations on device arrays in the reference layout -------- */

/* quantize_weights_q4_0 (quantize.rs:414-474): w_kn_dev f32 row-major [K,N] ->
 * Q4_0 20-byte blocks, column-major placement (col*G + g)*20 as documented at
 * quantize.rs:410-413 and read by every consumer. */
int twm_quantize_weights_q4_0(twm_ctx *ctx, const float *w_kn_dev, uint32_t k, uint32_t n,
                              uint8_t *q4_dev);
/* reorder_to_tw_marlin (quantize.rs:912-956): Q4_0 column-major -> (packed, scales f16). */
int twm_reorder_to_tw_marlin(twm_ctx *ctx, const uint8_t *q4_dev, uint32_t k, uint32_t n,
                             uint8_t *packed_dev, uint16_t *scales_dev);
/* quantize_f32_to_tw_marlin (quantize.rs:1171-1180) in one pass; also equals
 * cpu_quantize_tw_marlin (gemma_moe_q4.rs:218-254) when w_is_nk != 0 and the
 * input is row-major [N,K]. */
int twm_quantize_f32_to_tw_marlin(twm_ctx *ctx, const float *w_dev, int w_is_nk, uint32_t k,
                                  uint32_t n, uint8_t *packed_dev, uint16_t *scales_dev);
/* fuse_tw_marlin_n (quantize.rs:1018-1063): concatenate `count` matrices along N.
 * packed_devs / scales_devs / ns are host arrays of `count` entries. */
int twm_fuse_tw_marlin_n(twm_ctx *ctx, const uint8_t *const *packed_devs,
                         const uint16_t *const *scales_devs, uint32_t k, const uint32_t *ns,
                         uint32_t count, uint8_t *packed_out_dev, uint16_t *scales_out_dev);
/* warp_dequant_q4_to_f16 / dequant_q4_to_f16 (quantize.rs:534-618) for TW-Marlin input:
 * out[k][n] = f16_rne(f32(scale) * (q - 8)), row-major [K,N].  The "Q4 unpack". */
int twm_dequant_to_f16(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev,
                       uint32_t k, uint32_t n, uint16_t *out_kn_dev);
/* same, f32 output (exact product) */
int twm_dequant_to_f32(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev,
                       uint32_t k, uint32_t n, float *out_kn_dev);
/* fp16::cast_f32_to_f16 / cast_f16_to_f32 (crates/kernels/src/fp16.rs:133-166): elementwise, round to nearest even.
 * The GEMM entry points write f32 rows, as the reference's decode buffers are (generate.rs:1382-1404); a caller that
 * keeps f16 rows (the reference's FP16 pipeline) converts with these, and converts its f32 norm output to f16 once
 * where it wants the faster TWM_F16 input. */
int twm_cast_f32_to_f16(twm_ctx *ctx, const float *src_dev, uint16_t *dst_dev, size_t count);
int twm_cast_f16_to_f32(twm_ctx *ctx, const uint16_t *src_dev, float *dst_dev, size_t count);
/* split_qkv (ops.rs:2300-2321) and split_gate_up (ops.rs:2324-2343) */
int twm_split_qkv(twm_ctx *ctx, const float *qkv_dev, float *q_dev, float *k_dev, float *v_dev,
                  uint32_t h, uint32_t kv_dim, uint32_t batch);
int twm_split_gate_up(twm_ctx *ctx, const float *gate_up_dev, float *gate_dev, float *up_dev,
                      uint32_t ffn_dim, uint32_t batch);

/* fused_silu_mul (ops.rs:1139-1155, kernel warp_fused_silu_mul ops.rs:966-976): the SwiGLU gate,
 * out[i] = gate[i] / (1 + expf(-gate[i])) * up[i] in f32, i < count. */
int twm_silu_mul(twm_ctx *ctx, const float *gate_dev, const float *up_dev, float *out_dev, size_t count);
/* split_gate_up + fused_silu_mul in one pass (generate.rs:1086-1093, 2198-2203):
 * out[b][j] = silu(gate_up[b][gate column j]) * gate_up[b][up column j], gate_up [batch, 2*ffn_dim].
 * paired = 0: the reference's fused order, gate columns then up columns.
 * paired = 1: the order of twm_pair_gate_up (ffn_dim must be a multiple of 32). */
int twm_swiglu_rows(twm_ctx *ctx, const float *gate_up_dev, uint32_t batch, uint32_t ffn_dim, int paired,
                    float *out_dev);
/* Like fuse_tw_marlin_n of (gate, up), but with the columns interleaved in runs of 32: output column
 * 64*(j/32) + j%32 is gate column j and the up column j sits 32 further, so any kernel that owns 64
 * consecutive columns has both halves of 32 features.  ffn_dim must be a multiple of 32.  Outputs are
 * TW-Marlin arrays of shape [K/32][2*ffn_dim]; a byte permutation of the reference's fused arrays. */
int twm_pair_gate_up(twm_ctx *ctx, const uint8_t *gate_packed_dev, const uint16_t *gate_scales_dev,
                     const uint8_t *up_packed_dev, const uint16_t *up_scales_dev, uint32_t k,
                     uint32_t ffn_dim, uint8_t *packed_out_dev, uint16_t *scales_out_dev);

/* argmax (crates/kernels/src/missing_ops.rs:24-58): out[row] = first index of the row's maximum, with the
 * reference's starting value: only values > -1e30 compete, a row without any yields 0; NaNs never win.
 * input [rows, cols] f32 row-major, out [rows] i32.  Used on the LM-head logits (generate.rs:1417-1418)
 * so that greedy decoding reads back 4 bytes instead of the logits. */
int twm_argmax_f32(twm_ctx *ctx, const float *input_dev, uint32_t rows, uint32_t cols, int32_t *out_dev);

/* ---- the quantized-GEMM entry point, reference layout in, no repack ------------------ */

/* gemm_tw_marlin_m1 (quantize.rs:1301-1360): C[1,N] = A[1,K] * dequant(packed, scales),
 * f32 activations and output, arrays exactly as the reference holds them (packed at least 4-byte aligned, the
 * alignment the reference's own kernel needs; 16-byte aligned for the fast kernel).
 * Runs the M <= 4 MFMA kernel straight on those arrays: weights (q - 8) exact, every f32 activation
 * enters as two f16 terms, a first term and the residual a - first (about 21 bits; any finite f32: where a value lies
 * beyond the f16 range, the kernel first scales that stretch of the row by a power of two and the sums back, both
 * exact), f32 sum per group times f32(scale), deterministic split-K.  Option "m1_exact" selects the
 * plain f32 kernel in the reference's order instead (also taken when a_dev or packed_dev is not 16-byte aligned).
 * K % 32 != 0 returns TWM_SHAPE_ERROR where the reference asserts (quantize.rs:1311).
 * Uses the context's scratch like twm_gemm. */
int twm_gemm_tw_marlin_m1(twm_ctx *ctx, const float *a_dev, const uint8_t *packed_dev,
                          const uint16_t *scales_dev, float *c_dev, uint32_t n, uint32_t k);
/* gemm_tw_marlin_m1_from_buffer (quantize.rs:1731-1782): offsets in bytes (packed) and in
 * f16 elements (scales) into larger slabs. */
int twm_gemm_tw_marlin_m1_from_buffer(twm_ctx *ctx, const float *a_dev, const uint8_t *packed_buf_dev,
                                      size_t packed_offset, const uint16_t *scales_buf_dev,
                                      size_t scales_offset, float *c_dev, uint32_t n, uint32_t k);
/* twm_gemm_tw_marlin_m1 for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  It takes no context: work is issued on
 * hip_stream (a hipStream_t, NULL = the null stream) of the current device, with the library's default plan, and
 * the split-K scratch is a static device array inside the library (64 KiB of partial sums + 256 counters per GPU,
 * held until the process ends; the default plan cuts K over workgroups on matrices of at most 1024 columns whose K is
 * at least 16384 deep, e.g. 16384 -> 256, and those launches park their partial sums there).  The call itself allocates and frees nothing and never synchronises.  Results are
 * bit-identical to twm_gemm_tw_marlin_m1 with default options.  Limits: N <= 2^20 and K <= 2^20, beyond which
 * TWM_SHAPE_ERROR is returned; alignment rules as twm_gemm_tw_marlin_m1.  All calls on one GPU share that GPU's
 * array: two calls that overlap in time on one GPU (two streams, two threads) race; calls on one stream do not. */
int twm_gemm_tw_marlin_m1_noalloc(void *hip_stream, const float *a_dev, const uint8_t *packed_dev,
                                  const uint16_t *scales_dev, float *c_dev, uint32_t n, uint32_t k);
/* Testing aid for the entry point above (no counterpart in the reference): sets every byte of the current GPU's static
 * scratch, partial sums and arrival counters, to `value` on hip_stream.  A test poisons the scratch with it and then
 * shows that a call's result does not depend on what was there.  Not for use under graph capture. */
int twm_noalloc_scratch_fill(void *hip_stream, int value);
/* The reference's adaptive split-K rule, bit for bit (quantize.rs:1314-1325). */
void twm_pick_splits_reference(uint32_t k, uint32_t n, uint32_t *n_blocks, uint32_t *splits,
                               uint32_t *groups_per_split);

/* ---- the same path with weights repacked once at upload (the fast path) ------------- */

/* Takes exactly the reference's TW-Marlin arrays (host) and repacks them on the GPU into
 * the wavefront tile order the gfx950 kernels stream.  Replaces the from_host uploads at
 * quantize.rs:950-953 / 1057-1060. */
twm_weight *twm_weight_upload(twm_ctx *ctx, const uint8_t *packed_host, const uint16_t *scales_host,
                              uint32_t k, uint32_t n);
/* Same from device arrays (e.g. the output of twm_fuse_tw_marlin_n). The inputs are not retained. */
twm_weight *twm_weight_from_device(twm_ctx *ctx, const uint8_t *packed_dev, const uint16_t *scales_dev,
                                   uint32_t k, uint32_t n);
/* fuse_tw_marlin_n on handles (crates/kernels/src/quantize.rs:1018-1063: QKV = [h | kv | kv], gate+up = [ffn | ffn]):
 * a new handle whose columns are those of parts[0], parts[1], ... in turn; the parts stay valid and unchanged.  Works on
 * the repacked copies (block copies, no unpacking), so every part but the last must be a multiple of 64 columns wide --
 * which the reference's head and ffn dimensions are; otherwise fuse the arrays (twm_fuse_tw_marlin_n) and upload.
 * Results are bit-identical to a handle made from the fused arrays.  All parts share K and the context. */
twm_weight *twm_weight_fuse_n(twm_ctx *ctx, const twm_weight *const *parts, uint32_t count);
void twm_weight_destroy(twm_weight *w);
int twm_weight_dims(const twm_weight *w, uint32_t *k, uint32_t *n);
/* device bytes held by the repacked weight */
size_t twm_weight_bytes(const twm_weight *w);
/* The handle holds the weight in up to two orders: the 16-column tile order (copy 1: the kernels for M >= 5 and the
 * prefill GEMM) and the column-lane order (copy 2: M <= 4, and M = 5 .. 16 on narrow matrices), 4.5 bits per weight
 * each.  Option "weight_copies" says which ones a new handle gets (0 or 3 = both, the default; 1; 2); a call that needs
 * a copy the handle does not hold builds it from the other one on the spot -- which allocates, so inside a graph
 * capture such a call fails with TWM_UNSUPPORTED_OP: ask for the copy beforehand with twm_weight_ensure.
 * twm_weight_drop frees one of two copies (synchronises the stream); twm_weight_copies returns the mask held.
 * No counterpart in the reference, whose kernels read the one TW-Marlin order. */
/* Measured plans, the role of AutoTuner::tune_gemm and its per-shape table (crates/kernels/src/autotune.rs:254-396):
 * for each of the `count` row counts in ms[], times this weight's GEMM in the launch forms that the option knobs can
 * ask for (sub-tile widths and waves, whole tiles with K-splits, streaming and LDS-shared batched-decode forms, prefill
 * block heights and K-splits) on synthetic f16 activations -- as captured graphs replayed over copies of the weight that
 * together exceed the 256 MB cache -- and keeps the fastest for that bucket of row counts (1, 2, 3-4, 5-8, ...
 * 513-1024, above) when it beats the planners' own choice by more than 2 %.  Later calls with f16
 * activations, splits = 0 and no knob set run the kept form; the table travels with twm_weight_export / _import.
 * Allocates trial buffers and synchronises: a load-time call, not for a graph capture.
 * twm_weight_tuned_plan returns the bucket's entry as eight ints: valid, kernel, nt, waves, sub, sub_waves, splits,
 * prefill_bm (valid = 0: the planners' choice runs). */
int twm_weight_tune(twm_ctx *ctx, twm_weight *w, const uint32_t *ms, uint32_t count);
int twm_weight_tuned_plan(const twm_weight *w, uint32_t m, int *knobs8);
int twm_weight_ensure(twm_ctx *ctx, twm_weight *w, int copies);
int twm_weight_drop(twm_ctx *ctx, twm_weight *w, int copies);
int twm_weight_copies(const twm_weight *w);
/* The repacked weight as a self-describing byte blob, for an on-disk cache of the internal order
 * beside the reference's pre-quantized `.warp` cache (crates/loader/src/warp_cache.rs:1-21: store
 * it there as one U8 tensor per projection).  Import skips quantize / reorder / fuse / repack: it
 * is one host-to-device copy.  The blob carries a layout number; a library whose repacked order
 * differs refuses it (TWM_UNSUPPORTED_OP) and the caller repacks from the TW-Marlin arrays.
 * A checksum catches truncated or corrupt blobs (TWM_SHAPE_ERROR).  Both calls synchronise. */
size_t twm_weight_blob_bytes(const twm_weight *w);
int twm_weight_export(twm_ctx *ctx, const twm_weight *w, void *blob_host, size_t blob_bytes);
twm_weight *twm_weight_import(twm_ctx *ctx, const void *blob_host, size_t blob_bytes);
/* "Q4 unpack" straight from the repacked form: out[k][n] f16 row-major [K,N]; must be
 * bit-identical to twm_dequant_to_f16 of the arrays the weight was made from. */
int twm_weight_dequant_f16(twm_ctx *ctx, const twm_weight *w, uint16_t *out_kn_dev);

/* C[M,N] (f32, row-major) = A[M,K] (f16 or f32, row-major) * dequant(W), f32 accumulation.
 * M = 1 is gemm_tw_marlin_m1 (quantize.rs:1301); M > 1 has the semantics of gemm_q4_0
 * (quantize.rs:1825-1858).  splits = 0 lets the library choose (twm_pick_splits).
 * M <= 32: decode kernels (M <= 4 one lane per column, above that 16-column tiles), weights exact,
 *          each group's f32 sum scaled by f32(scale): a row's result does not depend on the batch it is in
 *          beyond f32 summation order.  (Option "batch_rounded": M = 17 .. 32 on the FP16 Q4 unpack.)
 * Up to M = 32 f32 activations enter as two f16 terms, a first term and the residual, about 21 bits.  Any finite f32
 * row is taken, as by the reference's kernels, which multiply in f32 (quantize.rs:1188, 186-246): values beyond the f16
 * range, and rows too small for it, are scaled by a power of two first and the sums back, both exact -- per stretch of
 * a row inside the kernels at M <= 4, per row by a conversion kernel ahead of the GEMM from M = 5 on.
 * M  > 32: prefill GEMM on the FP16 Q4 unpack (the arithmetic of the reference's FP16 route, DequantizedF16Weights +
 *          HGEMM, quantize.rs:620-670).  f32 activations are scaled per row in the same way and then rounded to ONE f16
 *          term: a deviation from gemm_q4_0 (quantize.rs:1825-1858), which multiplies f32 A by f32 weights -- about
 *          11 bits per activation, inside the 1e-2 bar on the sum but not the reference's f32 product; a caller that
 *          needs the f32 product of many rows calls in blocks of 32 rows ("prefill_min_m").
 * Uses the context's scratch: one context must not run two calls at the same time. */
int twm_gemm(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m,
             float *c_dev, uint32_t splits);
/* Fused projection with the split folded into the store: column ranges of the fused
 * weight go straight to separate buffers, replacing gemm_tw_marlin_m1 + split_qkv /
 * split_gate_up (generate.rs:2152-2155, 2195-2198).  outs_dev / ns are host arrays;
 * sum(ns) must equal the weight's N; out i is row-major [M, ns[i]] f32. */
int twm_gemm_split(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m,
                   float *const *outs_dev, const uint32_t *ns, uint32_t count, uint32_t splits);
/* twm_gemm with f16 result rows: c_dev_f16[M][N] = f16_rne(the f32 result of twm_gemm).  The reference's decode buffers
 * are f32 (generate.rs:1382-1404) and its FP16 pipeline keeps f16 rows (crates/kernels/src/fp16.rs:133-166 casts between
 * them); this entry point serves the second kind of caller without a buffer of its own: the kernels store f32 rows into
 * the back half of the context's scratch and the cast kernel rounds them into c_dev_f16, in row blocks when M x N x 4
 * bytes exceed that half (32 MB by default).  One more launch per block than twm_gemm, no allocation (capturable).
 * TWM_MEMORY_ERROR when a single row of f32 results does not fit: call twm_gemm and twm_cast_f32_to_f16 instead. */
int twm_gemm_f16out(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, uint16_t *c_dev_f16,
                    uint32_t splits);
/* twm_gemm_split with an f32 bias per output: out i = A x W_i + biases_dev[i][0..ns[i]) on every row
 * (one f32 add per element, GEMV result first).  biases_dev is a host array of `count` device
 * pointers, entries may be NULL; biases_dev itself may be NULL.  For the Q/K/V biases bq/bk/bv
 * (quantize.rs:1078-1080), which the reference adds in its fused bias + RoPE kernel
 * (generate.rs:2162-2178): with the sum already in q/k/v that kernel runs with has_bias = false. */
int twm_gemm_split_bias(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m,
                        float *const *outs_dev, const float *const *biases_dev, const uint32_t *ns,
                        uint32_t count, uint32_t splits);
/* Gate/up weight for twm_gemm_swiglu: twm_pair_gate_up followed by twm_weight_from_device, with the
 * handle marked as paired.  twm_gemm / twm_gemm_split on such a handle return the 2*ffn_dim columns
 * in the paired order. */
twm_weight *twm_weight_gate_up(twm_ctx *ctx, const uint8_t *gate_packed_dev, const uint16_t *gate_scales_dev,
                               const uint8_t *up_packed_dev, const uint16_t *up_scales_dev, uint32_t k,
                               uint32_t ffn_dim);
int twm_weight_is_paired(const twm_weight *w);
/* The MLP front half in one call: out[M][ffn_dim] = silu(A x W_gate) * (A x W_up), replacing
 * gemm_tw_marlin_m1 + split_gate_up + fused_silu_mul (generate.rs:2195-2203; prefill: 1086-1093).
 * w must come from twm_weight_gate_up.  The gate is applied in the GEMM's store (or, with split-K,
 * in the kernel that adds the partial sums), so the [M][2*ffn_dim] intermediate never reaches
 * memory, for every M.  The arithmetic of the projections is twm_gemm's for the same M.
 * out_dev must be 16-byte aligned. */
int twm_gemm_swiglu(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m,
                    float *out_dev, uint32_t splits);
/* The same with the GEGLU gate of the Gemma models, gelu_tanh(gate) * up (fused_gelu_mul,
 * ops.rs:1157-1190; callers gemma_generate.rs:463, 623). */
int twm_gemm_geglu(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m,
                   float *out_dev, uint32_t splits);
/* ---- expert banks: the TW-Marlin GEMVs of mixture-of-experts decode ------------------------- */

typedef struct twm_bank twm_bank;

/* Repacks num_experts matrices of the same (K, N) that lie in one pair of device buffers, expert e at
 * packed_base + e * packed_bytes_per_expert (bytes) and scales_base + e * scales_per_expert (f16
 * elements): the layout and the two strides of batched_marlin_gate_up
 * (crates/kernels/src/moe_batched_marlin.rs:20-36, 153-166).  pair_gate_up != 0: every matrix is a fused
 * [gate | up] (N = 2 * dim, a multiple of 64) and is stored in the paired column order, which lets
 * twm_bank_gemv apply the gate in its store.  The inputs are not retained. */
twm_bank *twm_bank_from_device(twm_ctx *ctx, const uint8_t *packed_base_dev, const uint16_t *scales_base_dev,
                               size_t packed_bytes_per_expert, size_t scales_per_expert, uint32_t k,
                               uint32_t n, uint32_t num_experts, int pair_gate_up);
/* The same bank from per-expert offset tables: expert e lies at packed_base + packed_offsets[e] (bytes, a multiple of
 * 4) and scales_base + scales_offsets[e] (f16 elements), both tables u32 arrays of num_experts entries in device
 * memory -- the arguments of gemm_tw_marlin_m1_indirect (crates/kernels/src/quantize_indirect.rs:228-253), whose
 * experts need not be equally spaced.  The tables are read once, here (a synchronous copy); the inputs are not retained. */
twm_bank *twm_bank_from_device_offsets(twm_ctx *ctx, const uint8_t *packed_base_dev, const uint16_t *scales_base_dev,
                                       const uint32_t *packed_offsets_dev, const uint32_t *scales_offsets_dev, uint32_t k,
                                       uint32_t n, uint32_t num_experts, int pair_gate_up);
void twm_bank_destroy(twm_bank *b);
size_t twm_bank_bytes(const twm_bank *b);
/* All top_k expert GEMVs in one launch, the expert of slot s being (int)topk_ids_dev[s], read on the
 * device (batched_marlin_gate_up, moe_batched_marlin.rs:20-74, 153-182): out[s][n] = A_s x W[id_s].
 * a_slot_stride (elements) = 0 shares one activation row [1, K] among the slots, K gives every slot
 * its own row of a [top_k, K] matrix.  With top_k = 1 and topk_ids_dev pointing at the wanted entry it
 * is the device-indexed GEMV gemm_tw_marlin_m1_indirect (quantize_indirect.rs:185-253).
 * act = 0: out is [top_k, N].  act = 1 / 2 (paired bank only): the store applies
 * gelu_tanh(gate) * up (batched_marlin_split_geglu, :137-151) or silu(gate) * up, out is [top_k, N/2]
 * and no [top_k, N] intermediate exists.  An id outside [0, num_experts) yields zeros. */
int twm_bank_gemv(twm_ctx *ctx, const twm_bank *b, const void *a_dev, int a_dtype, uint32_t a_slot_stride,
                  const float *topk_ids_dev, uint32_t top_k, int act, float *out_dev);
/* batched_marlin_down_axpy (moe_batched_marlin.rs:78-134, 184-213): acc[n] += sum over the slots of
 * topk_weights[s] * (A[s] x W[id_s]) with A [top_k, K].  The reference adds with float atomics in no
 * fixed order; here the terms are added to acc in slot order, one launch, deterministic.
 * top_k <= 16. */
int twm_bank_down_axpy(twm_ctx *ctx, const twm_bank *b, const void *a_all_dev, int a_dtype,
                       const float *topk_ids_dev, const float *topk_weights_dev, uint32_t top_k,
                       float *acc_dev);
/* batched_marlin_split_geglu (moe_batched_marlin.rs:137-151, 215-232):
 * out[b][j] = gelu_tanh(gate_up[b][gate column j]) * gate_up[b][up column j], gate_up [batch, 2*dim];
 * paired as in twm_swiglu_rows. */
int twm_geglu_rows(twm_ctx *ctx, const float *gate_up_dev, uint32_t batch, uint32_t dim, int paired,
                   float *out_dev);

/* ---- the reference's MoE launches with its own arguments: raw slabs, nothing repacked, no bank ---- */

/* batched_marlin_gate_up (crates/kernels/src/moe_batched_marlin.rs:153-182): output[s][n] = input[1, K] x W[id_s] for
 * s < top_k in one launch, id_s = (int)topk_ids_dev[s] read on the device; expert x's TW-Marlin arrays lie at
 * packed_buf_dev + x * packed_bytes_per_expert (u8 [K/32][N][16]) and scales_buf_dev + x * scales_per_expert
 * (f16 [K/32][N]).  Arguments in the reference's order.  f32 activations enter as two f16 terms (any finite value,
 * as in twm_gemm_tw_marlin_m1); an id below zero or NaN gives a row of zeros where the reference reads out of bounds.
 * Slower than a bank (twm_bank_gemv) by what the [G][N] order costs: a wave's four group rows are N * 16 bytes apart. */
int twm_batched_marlin_gate_up(twm_ctx *ctx, const float *input_dev, const uint8_t *packed_buf_dev,
                               const uint16_t *scales_buf_dev, const float *topk_ids_dev, float *output_dev,
                               uint32_t packed_bytes_per_expert, uint32_t scales_per_expert, uint32_t n, uint32_t k,
                               uint32_t top_k);
/* batched_marlin_down_axpy (moe_batched_marlin.rs:184-213): acc[n] += sum over s < top_k of topk_weights[s] *
 * (geglu_all[s][K] x W[id_s]).  The reference adds with float atomics in no fixed order; here slot by slot, in order,
 * deterministic (sixteen slots per launch, further launches for more). */
int twm_batched_marlin_down_axpy(twm_ctx *ctx, const float *geglu_all_dev, const uint8_t *packed_buf_dev,
                                 const uint16_t *scales_buf_dev, const float *topk_ids_dev, const float *topk_weights_dev,
                                 float *acc_dev, uint32_t packed_bytes_per_expert, uint32_t scales_per_expert, uint32_t n,
                                 uint32_t k, uint32_t top_k);
/* batched_marlin_split_geglu (moe_batched_marlin.rs:215-232): output[s][j] = gelu_tanh(gate_up[s][j]) *
 * gate_up[s][moe_dim + j]; = twm_geglu_rows with the plain column order. */
int twm_batched_marlin_split_geglu(twm_ctx *ctx, const float *gate_up_dev, float *output_dev, uint32_t moe_dim,
                                   uint32_t top_k);
/* gemm_tw_marlin_m1_indirect (crates/kernels/src/quantize_indirect.rs:228-253): C[1, N] = A[1, K] x W[expert_idx] with
 * the expert's arrays at packed_buf_dev + packed_offsets_dev[expert_idx] (bytes, a multiple of 4) and scales_buf_dev +
 * scales_offsets_dev[expert_idx] (f16 elements); both tables u32 arrays in device memory, read by the kernel. */
int twm_gemm_tw_marlin_m1_indirect(twm_ctx *ctx, const float *a_dev, const uint8_t *packed_buf_dev,
                                   const uint32_t *packed_offsets_dev, const uint16_t *scales_buf_dev,
                                   const uint32_t *scales_offsets_dev, int expert_idx, float *c_dev, uint32_t n, uint32_t k);

/* The library's split-K choice for MI355X (256 CUs) with f16 activations; same role as quantize.rs:1317-1325.
 * 1 where the plan needs no split (among others wherever M <= 16 runs on column sub-tiles). */
uint32_t twm_pick_splits(uint32_t k, uint32_t n, uint32_t m);

/* What twm_gemm would launch for a K x N weight, m rows of f16 / f32 activations and (gated != 0) the gated store of a
 * paired weight, as one line of text: the kernel, its workgroup shape, the K-split and the repacked copy it reads.
 * ctx = NULL: a fresh context's defaults; otherwise the context's options count.  Touches no device: usable to
 * see what the planners decide -- the counterpart of AutoTuner::heuristic_variant and ::report
 * (crates/kernels/src/autotune.rs:505-515, 648-668) -- and to test them without a GPU. */
int twm_plan_describe(const twm_ctx *ctx, uint32_t k, uint32_t n, uint32_t m, int a_dtype, int gated, char *text, size_t bytes);
/* The same for twm_gemm_tw_marlin_m1 on the reference's arrays (16-byte aligned activations and records assumed; others
 * run the reference-order kernel): which kernel reads them, with how many columns and waves per workgroup and which
 * K-split.  The reference's own choice for this call is pick_splits (quantize.rs:1317-1325), mirrored by
 * twm_pick_splits_reference. */
int twm_plan_describe_m1(const twm_ctx *ctx, uint32_t k, uint32_t n, char *text, size_t bytes);

/* ---- graph capture / replay (GraphCapture::{record_with_device, replay}, cuda_graph.rs:85-117) */

/* Starts capturing the work issued on the context's stream. */
int twm_graph_begin(twm_ctx *ctx);
/* Ends capture and instantiates; NULL on failure. */
twm_graph *twm_graph_end(twm_ctx *ctx);
/* GraphCapture::replay */
int twm_graph_launch(twm_ctx *ctx, twm_graph *g);
void twm_graph_destroy(twm_graph *g);

#ifdef __cplusplus
}
#endif
#endif /* TWMARLIN_H */

// What the files that hold the C ABI share: the handle types behind the opaque pointers of include/twmarlin.h and the
// helpers that cross file boundaries.
//   twm_api.hip          contexts, device memory, events, format operations, the GEMV on the reference's arrays, graphs
//   twm_api_weights.hip  repacked weight handles and their byte blob
//   twm_api_gemm.hip     launch planners, the dispatcher of twm_gemm and its variants, measured plans
//   twm_api_moe.hip      expert banks and the reference's MoE launches on raw slabs
#pragma once
#include "../../include/twmarlin.h"
#include "twm_internal.h"

#include <cstdio>
#include <cstring>
#include <new>
#include <vector>

#define HIP_TRY(expr, code, what)                                                      \
    do {                                                                               \
        hipError_t e__ = (expr);                                                       \
        if (e__ != hipSuccess) {                                                       \
            (void)hipGetLastError(); /* (the runtime keeps the error for the next caller of hipGetLastError otherwise) */ \
            return api_fail(code, "%s: %s", what, hipGetErrorString(e__));             \
        }                                                                              \
    } while (0)

struct twm_ctx {
    int ordinal;
    twm::TraceBuf trace;  // twm_debug_trace: where this context's M = 1 sub-tile launches record their clocks (null: off)
    hipStream_t own_stream;
    hipStream_t stream;
    float *ws;            // split-K partial tiles
    size_t ws_bytes;
    unsigned *counters;   // one arrival counter per tile group, zero between launches
    uint32_t n_counters;
    bool capturing;
    int force_nt;         // 0 = heuristic
    int force_waves;      // 0 = heuristic
    int force_sub_waves;  // sub-tile kernels with a forced width: waves per workgroup (1 .. 16), 0 = "waves" or eight
    int force_sub;        // M <= 4: 0 = heuristic, 1 = whole 64-column tiles per workgroup, 32 or 16 = the sub-tile kernel
    int force_kernel;     // 0 = heuristic, 2 = one-lane-per-column kernel on whole tiles (M <= 4), 3 = streaming kernel (M <= 32),
                          // 4 = batched-decode kernel with LDS-shared activations (M <= 32; "nt" = tiles per wave, "waves" 8 / 16 = 2 / 4 k-slices)
    int prefill_bm;       // prefill block form: 0 = choose, 64 = 64 rows x 256 columns, 128 = 128 x 256, 192 = 128 rows x 192 columns
    int prefill_min_m;    // M from which the LDS/MFMA prefill kernel runs instead of 16-row decode blocks
    int dequant_src;      // which copy twm_weight_dequant_f16 unpacks: 0 = 16-column tiles, 1 = column-lane
    int tune_on_upload;   // new plain weight handles are tuned at once: 0 = no, 1 = decode row counts, 2 = prefill row counts too
    int weight_copies;    // copies a new weight handle is given: 0 or 3 = both, 1 = 16-column tiles only, 2 = column-lane only
    int m1_align16;       // twm_gemm_tw_marlin_m1: 1 = refuse arrays that are not 16-byte aligned instead of running k_ref_gemv
    int m1_exact;         // twm_gemm_tw_marlin_m1: 1 = f32 activations and f32 FMAs in the reference's order
    int m1_splits;        // twm_gemm_tw_marlin_m1: split-K factor of the MFMA kernel, 0 = heuristic
    int batch_rounded;    // M = 17 .. 32: 1 = weights rounded to f16 (the reference's dequant-then-FP16-GEMM arithmetic), 0 = exact
    hipDeviceProp_t prop;
};

// A launch form as the option knobs name it (twm_ctx_set_option), measured to be the fastest for one weight and one
// bucket of row counts by twm_weight_tune: the role of the per-shape table of crates/kernels/src/autotune.rs:254-396.
struct TunedPlan {
    uint8_t valid, kernel, nt, waves, sub, sub_waves, splits, prefill_bm;
};
static_assert(sizeof(TunedPlan) == 8, "a tuned plan is eight bytes of the weight blob");
constexpr int kTuneBuckets = 12;
// row counts 1, 2, 3-4, 5-8, 9-16, 17-32, 33-64, 65-128, 129-256, 257-512, 513-1024, above
inline int tune_bucket(uint32_t m)
{
    if (m <= 2) return (int)m - 1;
    int b = 2;
    for (uint32_t top = 4; m > top && b < kTuneBuckets - 1; top *= 2) b++;
    return b;
}

// The two repacked copies are allocations of their own, each made when the handle is created (option
// "weight_copies") or at the first call that needs it (weight_ensure): a decode-only or prefill-only deployment holds
// one copy, 4.5 bits per weight.
enum { kCopyTile = 1, kCopyCol = 2 };
struct twm_weight {
    twm_ctx *ctx;
    void *qw;   // 16-column tile order: nibbles (qw) and scales (sc) in one allocation; nullptr while not built
    void *sc;
    void *cq;   // column-lane copy: 4608-byte blocks (nibbles + scales together); nullptr while not built
    uint32_t k, n, groups, n_tiles, k_chunks;
    size_t copy_bytes;  // one copy
    size_t bytes;       // device memory held now
    bool paired;  // gate_up weight whose columns are in the paired order (32 gate, 32 up, ...)
    TunedPlan tuned[kTuneBuckets];  // measured plans per row-count bucket (twm_weight_tune); valid = 0: the planners' choice
};

struct twm_bank {
    twm_ctx *ctx;
    void *cq;           // experts x column-lane copy
    size_t expert_bytes, bytes;
    uint32_t experts, k, n, n_pad, k_chunks;
    bool paired;
};

struct twm_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

constexpr size_t kWsBytes = 64ull << 20;    // split-K scratch of a context
constexpr uint32_t kCounters = 1u << 16;     // arrival counters of a context

// twm_api_weights.hip
twm_weight *weight_alloc(twm_ctx *ctx, uint32_t k, uint32_t n);
// device memory for the copies in `mask` that the handle does not hold yet (contents undefined)
int weight_alloc_copies(twm_weight *w, int mask, const char *who);
void weight_release(twm_weight *w);
inline int copies_of(const twm_weight *w) { return (w->qw ? kCopyTile : 0) | (w->cq ? kCopyCol : 0); }
// the handle holds the copies in `mask` afterwards, a missing one built from the other (allocates: not inside a capture)
int weight_ensure(twm_ctx *ctx, const twm_weight *w, int mask, const char *who);
twm::WeightView view_of(const twm_weight *w);
// twm_api.hip
int check_pair_args(const char *who, uint32_t k, uint32_t ffn_dim);

// C ABI, part: the quantized-GEMM dispatcher -- launch planners, the choice of a launch form, twm_gemm and its fused
// variants, measured plans (twm_weight_tune).  Host-side counterpart of crates/kernels/src/quantize.rs:1301-1360.
#include "twm_api_impl.h"

using namespace twm;

extern "C" {

/* ---- dispatcher --------------------------------------------------------------------------- */

// M <= 4 kernel (one lane per column): a workgroup of `waves` waves shares nt tiles of 64 columns
// and splits its k-chunks among the waves; workgroups split K further when 64-column tiles alone
// leave CUs idle.  Aim for about 16 waves per CU with at least two chunks per wave.
static DecodePlan plan_gemv4(uint32_t n_tiles, uint32_t k_chunks, int force_nt, int force_waves, uint32_t force_splits)
{
    DecodePlan p;
    p.lane_col = 1;
    uint32_t tiles64 = n_tiles * kTileN / 64;
    p.nt = 1;
    if (force_nt == 2 && tiles64 % 2 == 0) p.nt = 2;
    uint32_t tg = tiles64 / p.nt;
    // eight waves unless half of them would find no chunk: with a shallow K one chunk per wave puts every load
    // in flight at once (896-deep: 3.6 us with eight waves, 4.2 us with two)
    p.waves = 8;
    while (p.waves > 1 && k_chunks <= p.waves / 2) p.waves /= 2;
    // 64 .. 127 tiles with a deep K (4096 -> 4096 is the case): sixteen waves per tile put as many waves in flight
    // as a two-way split-K of eight-wave workgroups would, without its partial sums (5.9 against 6.5 us)
    if (p.waves == 8 && tg >= 64 && tg < 128 && k_chunks >= 32) p.waves = 16;
    if (force_waves) p.waves = (uint32_t)force_waves;
    uint32_t sp = 1;  // splitting across workgroups costs a synchronisation: only for matrices with few tiles
    while (tg * p.waves * sp < 1024 && k_chunks / (sp * 2) >= p.waves * 2) sp *= 2;
    if (force_splits) sp = force_splits;
    if (sp > k_chunks) sp = k_chunks ? k_chunks : 1;
    p.splits = sp;
    return p;
}

// Sub-tile variant of the M <= 4 kernel: 16 or 32 columns per workgroup, each wave one pass (4 or 2 chunks) of
// them, so that narrow matrices fill the CUs without a cross-workgroup split-K and wide ones run as many
// short-lived workgroups.  sub = 0: keep the 64-column plan.  Fitted to sweeps over the Qwen2.5-7B, Llama-7B and
// Qwen2.5-0.5B projections (M = 1, 2, 4; f16 and f32 activations); what it loses on are the activations, which
// every lane reads 64 / sub times per chunk: four distinct rows, or f32 rows cut into two terms, shift the
// balance back to wider workgroups.
struct SubPlan {
    uint32_t sub, waves;
};
static SubPlan plan_gemv4_sub(uint32_t tiles64, uint32_t k_chunks, uint32_t m, bool a_f32, bool gated)
{
    const SubPlan none = {0, 0};
    // shallow K, one row: short-lived workgroups on sub-tiles, whose waves sum by lane swaps and one LDS hop, are ahead
    // of the 64-column plan (896 -> 1152 2.64 against 3.09 us, 1536 -> 2048 2.69 / 3.90, 1536 -> 1536 2.67 / 3.86,
    // 896 -> 9728 3.34 / 3.59; f32 rows 2.72 / 3.31, 2.91 / 4.06); more rows: nothing measured, the 64-column plan stays
    if (k_chunks < 16) {
        if (m != 1) return none;
        const uint32_t p16 = (k_chunks + 3) / 4;
        return tiles64 > 128 ? SubPlan{32, 8} : SubPlan{16, p16 < 4 ? 4u : p16};
    }
    const bool two_pass = a_f32 && m > 2;
    const uint32_t passes16 = (k_chunks + 3) / 4;
    // waves per workgroup on 16 columns: one pass each while eight or sixteen cover K; deeper, the pipelined pass loop
    // on eight waves for one row and on four from two rows on (18944 -> 3584: M = 1 8.96 / 9.01 / 9.05 us on 8 / 4 / 16
    // waves, M = 2 9.5 / 9.2 / 9.7, M = 4 11.2 / 10.75 / 11.75)
    // (one row of f32 activations, which a lane takes as one shared piece: 9.3 / 9.6 us on 4 / 8 waves)
    // (one f16 row after the kernel's arguments all came preloaded: four waves ahead from 28 passes on -- 18944 -> 3584
    // 8.58 against 8.74 us on eight, 14336 -> 4096 7.48 / 7.64 -- and level or behind below: 11008 -> 4096 6.60 / 6.62,
    // 11008 -> 2048 5.75 / 5.63, 8960 -> 1536 5.01 / 4.87)
    // (one row, 17 .. 32 passes: two passes per wave with all their loads issued up front, k_gemv4s_upfront -- 11008 -> 4096
    // 6.20 against 6.44 us in the loop, f32 row 6.35 / 6.64; 14336 -> 4096 7.28 / 7.64; 8960 -> 1536 4.51 / 4.85; three
    // passes per wave, 18944 -> 3584, are level with the loop on four waves: 8.35 / 8.27)
    const SubPlan narrow16 = {16, passes16 <= 8 ? 8u : passes16 <= 16 ? 16u : (m == 1 && passes16 <= 32) ? (passes16 + 1) / 2
                                  : ((m >= 2 && !a_f32) || (m == 1 && (a_f32 || passes16 >= 28))) ? 4u : 8u};
    if (tiles64 > 128) {
        // wide matrices: only the cheapest activations (f16, up to two rows) leave the sub-tiles ahead
        // (3584 -> 37888: 15.8 against 17.0 us at M = 1, 18.3 against 17.3 at M = 4, 19.9 against 17.9 with f32 rows)
        // and only while every wave gets exactly one pass (K <= 4096): beyond that the 64-column kernel is ahead
        // again (5120 -> 15360: 9.2 against 12.5 us; 8192 -> 57344: 42.3 against 49.7)
        // and where whole tiles would leave their last round of 256 workgroups under 80 % full, which is the loss the
        // finer workgroups remove (4096 -> 22016, 344 tiles = 1.34 rounds: 10.6 against 12.1 us; 3584 -> 37888, 2.31
        // rounds: 14.8 against 15.5; but 4096 -> 28672, 1.75 rounds: 13.2 against 12.7, and 3584 -> 152064, 9.3
        // rounds: 49.3 against 47.8)
        const uint32_t rounds = (tiles64 + 255) / 256;
        const bool poor_fill = tiles64 * 5 < rounds * 256 * 4;
        // One row, plain store: since the waves sum by lane swaps and the first wave alone finishes, 16 columns are ahead
        // on every wide shape measured, whatever the fill and the depth -- f16 row on eight waves (one pass each up to
        // K = 4096, two or three up front, the pass loop beyond): 4096 -> 28672 12.1 against 12.7 us on whole tiles,
        // 3584 -> 152064 45.5 / 47.6, 4096 -> 128256 44.4 / 45.8, 8192 -> 28672 21.3 / 23.2, 8192 -> 10240 9.8 / 11.6,
        // 11008 -> 16384 17.5 / 18.4, 5120 -> 15360 level; f32 row on four waves up to K = 4096 (4096 -> 28672 13.0 / 14.3,
        // 4096 -> 14336 8.1 / 8.9, 3584 -> 152064 level), eight up to K = 8192 (8192 -> 28672 22.5 / 24.8, 5120 -> 15360
        // 10.0 / 10.4), four beyond (11008 -> 16384 19.2 / 19.3).  Two rows stay with the rules below (3584 -> 152064 at
        // M = 2: 48.7 against 47.8), and so does the gated store, which takes 32 columns.
        if (m == 1 && !gated) {
            if (a_f32) return SubPlan{16, passes16 <= 8 || passes16 > 64 ? 4u : 8u};
            return SubPlan{16, passes16 <= 4 ? 4u : passes16 <= 8 ? ((passes16 + 1u) & ~1u) : 8u};
        }
        // (an even number of waves, so that the workgroups of a CU lie evenly on its four SIMDs and four of them fit:
        // 3584 -> 37888 at M = 1 13.4 us on eight waves, the eighth idle, against 14.2 on seven)
        if (!a_f32 && m <= 2 && passes16 <= 8 && poor_fill) return SubPlan{16, (passes16 + 1u) & ~1u};
        // (three and four rows: only where the last round is under 70 % full -- 4096 -> 22016, 67 %: 11.6 / 12.4 against
        // 12.8 / 12.9 us on whole tiles; 3584 -> 37888, 77 %: 16.3 / 17.5 against 16.0 / 16.1)
        if (!a_f32 && m <= 4 && passes16 <= 8 && tiles64 * 10 < rounds * 256 * 7) return SubPlan{16, passes16};
        // one row of f32 activations: the shared-piece form in the pipelined loop on four waves (3584 -> 37888: 15.75 us
        // against 17.0 with one pass per wave and 16.8 on whole tiles)
        if (a_f32 && m == 1 && passes16 <= 8 && poor_fill) return SubPlan{16, 4};
        if (a_f32 && m <= 2 && tiles64 < 256 && k_chunks <= 32) return SubPlan{32, 16};
        return none;
    }
    if (two_pass && passes16 > 16) return k_chunks <= 100 ? SubPlan{32, 8} : none;  // (the looping 16-column variant spills)
    // very deep K, three or four rows: with f32 rows the 64-column split-K plan is level or ahead; with f16 rows the
    // pipelined pass loop is (18944 -> 3584 at M = 3 / 4: 9.96 / 10.75 against 11.75 / 11.84 us)
    if (m > 2 && passes16 > 32 && a_f32) return none;
    // 65 .. 128 tiles: 16 columns would leave a second, part-full round of workgroups, and 32 columns on sixteen waves are
    // ahead -- except for one row on a deep K, where eight waves in the pipelined pass loop on 16 columns win (13824 ->
    // 5120: 10.6 against 11.2 us with f16, 11.5 against 12.4 with f32 activations; 14336 -> 6144 11.2 / 11.9; 18944 -> 4608
    // 13.2 / 13.8; 13824 -> 7168 11.4 / 12.6; two rows level, four rows 32 columns again: 14.6 against 12.2)
    if (tiles64 > 64 && m == 1 && passes16 > 16) return SubPlan{16, 8};
    if (tiles64 > 64) return SubPlan{32, 16};
    return narrow16;
}

// M = 5 .. 16 (f16 rows): the same kernel repeats its MFMA chain per group of four rows on the unpacked weights.
// It pays where the streaming kernel's 64-column workgroups leave most CUs idle, i.e. on narrow matrices, and
// only in the one-pass form (the looping form runs out of registers): 3584 -> 3584 at M = 8 / 16: 4.8 / 6.5 us
// against 6.9 / 8.2; 3584 -> 4608: 5.5 / 7.4 against 6.9 / 8.2; 3584 -> 37888: 21.7 / 35 against 19.5 / 23.2.
static SubPlan plan_gemv4_sub_rows(uint32_t tiles64, uint32_t k_chunks)
{
    const SubPlan none = {0, 0};
    if (k_chunks < 16 || tiles64 > 128) return none;
    const uint32_t passes16 = (k_chunks + 3) / 4, passes32 = (k_chunks + 1) / 2;
    if (tiles64 <= 64 && passes16 <= 16) return SubPlan{16, passes16 <= 8 ? 8u : 16u};
    if (passes32 <= 16) return SubPlan{32, 16};
    return none;
}

// Batched-decode streaming kernel (M = 5 .. 32): one workgroup of eight waves per 64 columns and k-range.  K is
// cut when the column quads alone leave CUs idle, up to about one workgroup per CU, keeping two chunks per
// wave (one for the 32-row variant, whose chunks cost twice the arithmetic); the partial sums cost a second
// kernel.  Fitted to the per-shape sweep (bench.py --sweep-splits).
static uint32_t plan_stream(uint32_t n_tiles, uint32_t k_chunks, uint32_t m)
{
    uint32_t quads = n_tiles / 4;
    if (quads == 0 || quads >= 256) return 1;
    uint32_t sp = 256 / quads;
    uint32_t cap = k_chunks / (m > 16 ? 7 : 16);  // (3584 -> 3584 at M = 32: four splits of seven chunks 9.2 us, three 10.6)
    if (sp > cap) sp = cap;
    return sp < 2 ? 1 : sp;
}

// Waves per workgroup of the streaming kernel: eight, except that the 32-row variant (158 registers) fits
// only one eight-wave workgroup per CU, so with many column quads four-wave workgroups fill the CUs better.
static uint32_t stream_waves(uint32_t n_tiles, uint32_t m, int force_waves)
{
    if (force_waves == 4 || force_waves == 8) return (uint32_t)force_waves;
    return (m > 16 && n_tiles / 4 >= 256) ? 4 : 8;
}

// Batched-decode kernel with LDS-shared activations: split-K factor over workgroups, k-slices inside a workgroup and
// the columns that share one activation tile (one, two or three 64-column quads per workgroup with one tile per
// wave, or two quads with two tiles per wave) by a small cost model fitted to forced sweeps on fifteen projection
// shapes of 1.5B .. 70B models (microseconds).  A CU works through quad steps (one 128-deep chunk of one 64-column
// quad) at up to 3.5 per us with two row blocks (4.9 with one) when it holds enough waves.  The activation tile
// comes from L2 once per workgroup and chunk, and those requests compete with the weight stream for the CU's memory
// requests in flight: with two or three quads per workgroup the rate is 4.3 (5.2), with two tiles per wave 3.95
// (5.1).  A single slice alone advances at 1.9 (2.5) steps per us, 1.8 (2.4) with eight or twelve waves, 1.7 (2.2)
// with two tiles per wave: the latency of its barrier-and-load chain.  The busiest CU holds ceil(workgroups / 256)
// workgroups of `slices` slices, each with chunks / (splits * slices) steps (the time is the larger of the two
// bounds plus 15 % of the smaller: 8192 -> 10240 at M = 16 on 160 workgroups of two slices, both bounds 13, read 17.5 us
// with the launch, with four slices 15.4); a K-split over workgroups costs the
// second kernel (2.5) and, per split, 0.2 plus the partial sums written and read back at 2.7 TB/s
// (18944 -> 3584 at M = 32 read 19.0 us on nine splits against 17.2 on four).  A more elaborate plan has to win by
// 3 %; a slice keeps two chunks or more (eight with two tiles per wave).
// (3584 -> 37888, 592 quads x 28 chunks, M = 32: one quad per workgroup 26.1 us, two 26.0 -- 296 workgroups put four
// quads on some CUs instead of three --, three 22.4, two k-slices 27.3, two K-splits 30.3; 4096 -> 22016, 344 x 32:
// one quad 20.5, two quads x two slices 16.8; 8192 -> 57344, 896 x 64: one quad 72.4, two 63.2, two tiles per wave
// 61.9; 18944 -> 3584, 56 x 148: 4 splits x 2 slices 17.1, 4 x 1 20.7; 8192 -> 10240, 160 x 64: 3 splits, two quads x
// two slices 17.0, one quad 18.5.)
struct BatchPlan {
    uint32_t splits, slices, tiles_per_wave, quads_per_group;
};
static BatchPlan plan_batch(uint32_t n_tiles, uint32_t k_chunks, uint32_t m, bool rows_f32, uint32_t force_splits = 0)
{
    const uint32_t quads = n_tiles / 4;
    const bool two_blocks = m > 16;
    const double partial_us = (double)m * n_tiles * 16.0 * 4.0 * 2.0 / 4.0e6;  // one split's partial sums, written and read
    BatchPlan best = {force_splits ? (force_splits < k_chunks ? force_splits : k_chunks) : 1u, 1u, 1u, 1u};
    double best_us = 1e30;
    static const struct { uint32_t tpw, qpg, max_slices; double full2, full1, lone2, lone1; } kForms[] = {
        {1, 1, 4, 3.5, 4.9, 1.9, 2.5}, {1, 2, 2, 4.3, 5.2, 1.8, 2.4}, {1, 3, 1, 4.3, 5.2, 1.8, 2.4}, {2, 1, 2, 3.95, 5.1, 1.7, 2.2}};
    for (const auto &f : kForms) {
        const double full_rate = two_blocks ? f.full2 : f.full1, lone_rate = two_blocks ? f.lone2 : f.lone1;
        const uint32_t share = f.tpw * f.qpg;  // quads per workgroup
        const uint64_t groups = (quads + share - 1) / share;
        // (the 32-row two-term variant has LDS for one slice of eight waves, two of four)
        const uint32_t max_slices = two_blocks && rows_f32 ? (f.qpg == 2 ? 1u : f.max_slices < 2 ? f.max_slices : 2u) : f.max_slices;
        for (uint32_t sp = 1; sp <= 16 && sp <= k_chunks; sp++) {
            if (force_splits && sp != best.splits) continue;
            const uint32_t cps = (k_chunks + sp - 1) / sp;
            if (!force_splits && (k_chunks + cps - 1) / cps != sp) continue;  // same work as a smaller factor
            const double wgs_on_cu = (double)((groups * sp + 255) / 256);
            for (uint32_t ks = 1; ks <= max_slices; ks *= 2) {
                if (ks > 1 && cps < (f.tpw == 1 ? 2 : 8) * ks) continue;
                const double steps = (double)((cps + ks - 1) / ks);
                const double busy = wgs_on_cu * share * ks * steps / full_rate, chain = steps / lone_rate;
                double t = busy > chain ? busy + 0.15 * chain : chain + 0.15 * busy;  // (neither hides the other entirely)
                if (ks > 1) t += 0.3 * ks;  // the slices' sums through LDS, the wider barriers
                if (sp > 1) t += 2.5 + sp * (0.2 + 1.5 * partial_us);
                if (t < best_us * 0.97) {
                    best_us = t;
                    best.splits = sp;
                    best.slices = ks;
                    best.tiles_per_wave = f.tpw;
                    best.quads_per_group = f.qpg;
                }
            }
        }
    }
    return best;
}

// ---- the launch form of a GEMM: chosen in one place, launched in another ---------------------------------
// What twm_gemm will run for a weight's shape, a row count and the context's knobs.  Nothing here touches the device.
enum FormKind { kFormPrefill = 0, kFormSubTile = 1, kFormWholeTile = 2, kFormBatch = 3, kFormStream = 4, kFormNone = 5 };
struct LaunchForm {
    int kind;
    int copy;                 // the repacked order it reads (kCopyTile / kCopyCol)
    uint32_t sub, waves;      // sub-tile kernel: columns per workgroup, waves; whole tiles / streaming: waves
    uint32_t nt;              // whole tiles: 64-column tiles per workgroup
    uint32_t splits;          // K-splits over workgroups (prefill: the forced factor, 0 = plan_prefill's choice)
    bool batch_auto;          // LDS-shared batched decode: plan_batch per 32-row block, else `batch` as forced
    bool rounded;             //   ... on f16-rounded weights (option "batch_rounded")
    BatchPlan batch;
};
struct FormEnv {              // the knobs and limits of a context
    int kernel, nt, waves, sub, sub_waves, prefill_min_m, batch_rounded;
    size_t ws_bytes;          // split-K scratch
    uint32_t n_counters;      // arrival counters
};
static FormEnv form_env(const twm_ctx *c)
{
    return FormEnv{c->force_kernel, c->force_nt, c->force_waves, c->force_sub, c->force_sub_waves, c->prefill_min_m,
                   c->batch_rounded, c->ws_bytes, c->n_counters};
}

// n_tiles: 16-column tiles of the padded weight; gated: the gated store of a paired weight
static LaunchForm choose_form(const FormEnv &e, uint32_t n_tiles, uint32_t k_chunks, uint32_t m, bool a_f32, uint32_t splits, bool gated)
{
    LaunchForm f = {};
    const uint32_t n_ld = n_tiles * kTileN, tiles64 = n_ld / 64;
    f.splits = splits;
    if (m >= (uint32_t)e.prefill_min_m) {
        f.kind = kFormPrefill;
        f.copy = kCopyTile;
        return f;
    }
    // the sub-tile kernel's K-split fits the scratch and the counters
    auto fit_sub_splits = [&](uint32_t sub) {
        uint32_t ssp = splits ? splits : 1;
        if (ssp > k_chunks) ssp = k_chunks;
        while (ssp > 1 && (size_t)ssp * m * n_ld * 4 > e.ws_bytes) ssp--;
        if (n_ld / sub > e.n_counters) ssp = 1;
        return ssp;
    };
    auto fit_whole_splits = [&](DecodePlan &plan) {
        while (plan.splits > 1 && (size_t)plan.splits * m * n_ld * 4 > e.ws_bytes) plan.splits--;
        if (n_tiles / plan.nt > e.n_counters) plan.splits = 1;
    };
    if (e.kernel == 0 && m > 4 && m <= 16 && !a_f32 && e.sub != 1) {
        // M = 5 .. 16 on narrow matrices: the lane-per-column sub-tile kernel with two to four row groups
        SubPlan sub = {0, 0};
        if (e.sub >= 16) sub = SubPlan{(uint32_t)e.sub, e.sub_waves ? (uint32_t)e.sub_waves : e.waves ? (uint32_t)e.waves : 8};
        else if (!e.nt && !e.waves && !splits) sub = plan_gemv4_sub_rows(tiles64, k_chunks);
        if (sub.sub) {
            f.kind = kFormSubTile;
            f.copy = kCopyCol;
            f.sub = sub.sub;
            f.waves = sub.waves;
            f.splits = fit_sub_splits(sub.sub);
            return f;
        }
        if (m <= 8 && tiles64 > 128 && !e.nt && !splits) {
            // M = 5 .. 8 on wide matrices: the 64-column lane-per-column kernel with two row groups, which unpacks with
            // fewer vector instructions than the streaming kernel (3584 -> 37888 at M = 8: 18.0 against 19.2 us,
            // 3584 -> 152064: 54.8 against 60.0; with four row groups, M = 9 .. 16, it needs 127 registers and loses;
            // on 128 tiles or fewer the streaming kernel's split-K is ahead: 14336 -> 4096 11.4 against 19.8 us)
            DecodePlan plan = plan_gemv4(n_tiles, k_chunks, 1, e.waves, 0);
            fit_whole_splits(plan);
            f.kind = kFormWholeTile;
            f.copy = kCopyCol;
            f.nt = 1;
            f.waves = plan.waves;
            f.splits = plan.splits;
            return f;
        }
    }
    const bool batch_auto = e.kernel == 0 && !e.nt && !e.waves &&
                            (m > 16 || (!splits && ((m > 8 && (tiles64 > 128 || a_f32)) || (a_f32 && m > 4 && k_chunks <= 64))));
    if (e.kernel == 4 || batch_auto) {
        // batched decode with the activations shared through LDS, in 32-row blocks: from 17 rows on (the same exact
        // arithmetic as below 17 rows; option "batch_rounded" runs the f16-rounded weights of the prefill kernel
        // there), and from 9 rows on wide
        // matrices (3584 -> 37888: M = 16 19.8 against 22.8 us of the streaming kernel, M = 32 26.7 against
        // 33.3; 18944 -> 3584 at M = 32 17.3 against 21.8; at M = 9 .. 16 on narrow matrices the two are within 3 %
        // with f16 rows).  f32 rows, which the streaming kernel holds twice in registers: from 9 rows on everywhere
        // (3584 -> 4608 at M = 16 10.9 against 15.1 us, 18944 -> 3584 20.6 against 23.3), from 5 rows on up to 64
        // chunks deep (3584 -> 4608 at M = 8 10.5 against 11.4; 13824 -> 5120 would lose 18.6 against 18.5)
        f.kind = kFormBatch;
        f.copy = kCopyTile;
        f.batch_auto = batch_auto;
        f.rounded = e.batch_rounded && m > 16;
        // forced: "nt" 2 = two tiles per wave, 4 = two quads per workgroup, 3 = three; "waves" 8 / 16 = 2 / 4 k-slices
        f.batch = BatchPlan{splits ? splits : 1, e.waves == 8 ? 2u : e.waves == 16 ? 4u : 1u, e.nt == 2 ? 2u : 1u,
                            e.nt == 4 ? 2u : e.nt == 3 ? 3u : 1u};
        return f;
    }
    if (e.kernel == 3 || (e.kernel == 0 && m > 4)) {
        f.kind = kFormStream;   // batched decode: 32-row blocks of the streaming kernel
        f.copy = kCopyTile;
        return f;
    }
    // M <= 4: one lane per column (whole 64-column tiles, or the sub-tile kernel where the planner takes it)
    if (m > 4) {
        f.kind = kFormNone;
        return f;
    }
    f.copy = kCopyCol;
    SubPlan sub = {0, 0};
    if (e.sub >= 16) {
        sub.sub = (uint32_t)e.sub;
        sub.waves = e.sub_waves ? (uint32_t)e.sub_waves : e.waves ? (uint32_t)e.waves : 8;
    } else if (e.sub == 0 && !e.nt && !e.waves && !splits) {
        // (an explicit nt, waves or split factor asks for the 64-column kernel's plan)
        sub = plan_gemv4_sub(tiles64, k_chunks, m, a_f32, gated);
        // the gated store splits a sub-tile into a gate and an up half: 16 columns would read 128-byte runs
        // (3584 -> 2 x 18944 at M = 1: 17.0 us on 16 columns, 16.3 on 32, 17.1 on whole tiles)
        // (up to two rows and K = 4096 sixteen waves of one pass each: 3584 -> 2 x 18944 15.0 against 15.8 us on eight
        // waves in the pass loop, 4096 -> 2 x 11008 10.5 / 11.4, at M = 2 15.3 / 15.7 and 10.8 / 11.7; four rows 13.1 / 12.6)
        if (gated && sub.sub == 16) sub = SubPlan{32, (m <= 2 && k_chunks > 16 && k_chunks <= 32) ? 16u : 8u};
    }
    if (sub.sub) {
        f.kind = kFormSubTile;
        f.sub = sub.sub;
        f.waves = sub.waves;
        f.splits = fit_sub_splits(sub.sub);
        return f;
    }
    DecodePlan plan = plan_gemv4(n_tiles, k_chunks, e.nt, e.waves, splits);
    fit_whole_splits(plan);  // the scratch must hold splits x m x n_ld partials and one counter per tile group
    f.kind = kFormWholeTile;
    f.nt = plan.nt;
    f.waves = plan.waves;
    f.splits = plan.splits;
    return f;
}

static void tiles_of(uint32_t k, uint32_t n, uint32_t &n_tiles, uint32_t &k_chunks)
{
    n_tiles = ((n + kNPadTo - 1) / kNPadTo) * kNPadTo / kTileN;
    k_chunks = (k / 32 + kChunkGroups - 1) / kChunkGroups;
}
static FormEnv default_env()
{
    return FormEnv{0, 0, 0, 0, 0, 33, 0, kWsBytes, kCounters};
}

uint32_t twm_pick_splits(uint32_t k, uint32_t n, uint32_t m)
{
    uint32_t n_tiles, k_chunks;
    tiles_of(k, n, n_tiles, k_chunks);
    if (m == 0 || n_tiles == 0 || k_chunks == 0) return 1;
    // (f16 activations, nothing forced, the default scratch)
    const LaunchForm f = choose_form(default_env(), n_tiles, k_chunks, m, false, 0, false);
    switch (f.kind) {
    case kFormSubTile:
    case kFormWholeTile: return f.splits;
    case kFormBatch: return plan_batch(n_tiles, k_chunks, m < 32 ? m : 32, false).splits;
    case kFormStream: return plan_stream(n_tiles, k_chunks, m < 32 ? m : 32);
    default: return 1;  // prefill: see twm_plan_describe
    }
}

int twm_plan_describe(const twm_ctx *ctx, uint32_t k, uint32_t n, uint32_t m, int a_dtype, int gated, char *text, size_t bytes)
{
    if (!text || bytes == 0) return api_fail(TWM_INVALID_HANDLE, "twm_plan_describe: null buffer");
    if (a_dtype != TWM_F16 && a_dtype != TWM_F32) return api_fail(TWM_UNSUPPORTED_OP, "twm_plan_describe: activations must be f16 or f32");
    if (int rc = check_kn("twm_plan_describe", k, n)) return rc;
    uint32_t n_tiles, k_chunks;
    tiles_of(k, n, n_tiles, k_chunks);
    if (m == 0 || n == 0 || k == 0) {
        snprintf(text, bytes, "nothing to launch");
        return TWM_OK;
    }
    const bool a_f32 = a_dtype == TWM_F32;
    const FormEnv e = ctx ? form_env(ctx) : default_env();
    const LaunchForm f = choose_form(e, n_tiles, k_chunks, m, a_f32, 0, gated != 0);
    const uint32_t mb = m < (uint32_t)kMaxStreamM ? m : (uint32_t)kMaxStreamM;
    switch (f.kind) {
    case kFormPrefill: {
        uint32_t bm = 0, sp = 0;
        prefill_plan_of(m, 0, 0, n_tiles, k_chunks, e.ws_bytes, gated != 0, &bm, &sp);
        snprintf(text, bytes, "k_prefill: %u-row x %u-column blocks, %u K-split%s%s; 16-column tile copy", bm == 64 ? 64u : 128u,
                 bm == 192 ? 192u : 256u, sp, sp == 1 ? "" : "s", sp > 1 ? " + k_splitk_reduce" : "");
        break;
    }
    case kFormSubTile:
        snprintf(text, bytes, "k_gemv4s: %u-column sub-tiles, %u waves, %u K-split%s; column-lane copy", f.sub, f.waves, f.splits,
                 f.splits == 1 ? "" : "s");
        break;
    case kFormWholeTile:
        snprintf(text, bytes, "k_gemv4: %u x 64-column tiles per workgroup, %u waves, %u K-split%s; column-lane copy", f.nt, f.waves,
                 f.splits, f.splits == 1 ? "" : "s");
        break;
    case kFormBatch: {
        const BatchPlan bp = f.batch_auto ? plan_batch(n_tiles, k_chunks, f.rounded ? 32 : mb, a_f32, 0) : f.batch;
        snprintf(text, bytes, "k_batch: %u quad%s per workgroup, %u tile%s per wave, %u k-slice%s, %u K-split%s%s; 16-column tile copy",
                 bp.quads_per_group, bp.quads_per_group == 1 ? "" : "s", bp.tiles_per_wave, bp.tiles_per_wave == 1 ? "" : "s", bp.slices,
                 bp.slices == 1 ? "" : "s", bp.splits, bp.splits == 1 ? "" : "s", bp.splits > 1 ? " + k_splitk_reduce" : "");
        break;
    }
    case kFormStream: {
        const uint32_t sp = plan_stream(n_tiles, k_chunks, mb);
        snprintf(text, bytes, "k_stream: %u waves, %u K-split%s%s; 16-column tile copy", stream_waves(n_tiles, mb, e.waves), sp,
                 sp == 1 ? "" : "s", sp > 1 ? " + k_splitk_reduce" : "");
        break;
    }
    default: snprintf(text, bytes, "no kernel takes this case with the knobs set"); break;
    }
    return TWM_OK;
}

// swiglu_out (paired weight): the launch writes silu(gate) * up to swiglu_out[m][n/2] instead of the columns
// to `out`.
static int gemm_dispatch(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, const OutSpec &out,
                         uint32_t splits, const char *who, float *swiglu_out = nullptr, uint32_t gate_act = 2)
{
    if (a_dtype != TWM_F16 && a_dtype != TWM_F32) return api_fail(TWM_UNSUPPORTED_OP, "%s: activations must be f16 or f32", who);
    if (m == 0 || w->n == 0) return TWM_OK;
    if (w->k == 0) {
        for (uint32_t s = 0; s < out.count; s++) {
            if (!out.seg[s].bias) {
                if (int rc = twm_memset_zero(ctx, out.seg[s].ptr, (size_t)m * out.seg[s].width * 4)) return rc;
                continue;
            }
            for (uint32_t r = 0; r < m; r++)  // an empty sum plus the bias
                if (int rc = twm_memcpy_d2d(ctx, out.seg[s].ptr + (size_t)r * out.seg[s].width, out.seg[s].bias,
                                            (size_t)out.seg[s].width * 4))
                    return rc;
        }
        return TWM_OK;
    }
    if (!a_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null activations", who);
    if (((uintptr_t)a_dev & 15) != 0) return api_fail(TWM_SHAPE_ERROR, "%s: activations must be 16-byte aligned", who);
    const bool a_f32 = a_dtype == TWM_F32;
    const size_t a_row_bytes = (size_t)w->k * (a_f32 ? 4 : 2);
    OutSpec gated = out;
    gated.swiglu = swiglu_out;
    gated.gate_act = gate_act;
    const LaunchForm f = choose_form(form_env(ctx), w->n_tiles, w->k_chunks, m, a_f32, splits, swiglu_out != nullptr);
    if (f.kind == kFormNone) return api_fail(TWM_UNSUPPORTED_OP, "%s: the one-lane-per-column kernel takes M <= 4", who);
    // the copy the launch reads is built here if the handle does not hold it yet
    if (int rc = weight_ensure(ctx, w, f.copy, who)) return rc;
    const WeightView v = view_of(w);
    // rows beyond 32: blocks of 32 rows, each a launch of its own
    auto row_blocks = [&](auto &&launch_block) -> int {
        for (uint32_t m0 = 0; m0 < m; m0 += kMaxStreamM) {
            const uint32_t mb = m - m0 < (uint32_t)kMaxStreamM ? m - m0 : (uint32_t)kMaxStreamM;
            OutSpec o = gated;
            for (uint32_t s = 0; s < o.count; s++) o.seg[s].ptr += (size_t)m0 * o.seg[s].width;
            if (o.swiglu) o.swiglu += (size_t)m0 * (w->n / 2);
            if (int rc = launch_block((const char *)a_dev + (size_t)m0 * a_row_bytes, mb, o)) return rc;
        }
        return TWM_OK;
    };
    switch (f.kind) {
    case kFormPrefill: {
        HIP_TRY(launch_prefill(ctx->stream, v, a_dev, a_f32, m, gated, (uint32_t)ctx->prefill_bm, splits, ctx->ws, ctx->ws_bytes),
                TWM_DEVICE_ERROR, "prefill launch");
        return TWM_OK;
    }
    case kFormSubTile:
        HIP_TRY(launch_gemv4s(ctx->stream, v, a_dev, a_f32, m, gated, ctx->ws, ctx->counters, f.sub, f.waves, f.splits, ctx->trace), TWM_DEVICE_ERROR,
                "sub-tile gemv launch");
        return TWM_OK;
    case kFormWholeTile:
        HIP_TRY(launch_gemv4(ctx->stream, v, a_dev, a_f32, m, gated, ctx->ws, ctx->counters, f.nt, f.waves, f.splits, swiglu_out),
                TWM_DEVICE_ERROR, "gemv launch");
        return TWM_OK;
    case kFormBatch:
        return row_blocks([&](const char *a_blk, uint32_t mb, const OutSpec &o) -> int {
            const BatchPlan bp = f.batch_auto ? plan_batch(w->n_tiles, w->k_chunks, f.rounded ? 32 : mb, a_f32, splits) : f.batch;
            HIP_TRY(launch_batch(ctx->stream, v, a_blk, a_f32, mb, o, bp.splits, bp.tiles_per_wave, bp.slices, bp.quads_per_group, f.rounded,
                                 ctx->ws, ctx->ws_bytes),
                    TWM_DEVICE_ERROR, "batched decode launch");
            return TWM_OK;
        });
    default:  // kFormStream
        return row_blocks([&](const char *a_blk, uint32_t mb, const OutSpec &o) -> int {
            HIP_TRY(launch_stream(ctx->stream, v, a_blk, a_f32, mb, o, splits ? splits : plan_stream(w->n_tiles, w->k_chunks, mb),
                                  stream_waves(w->n_tiles, mb, ctx->force_waves), ctx->ws, ctx->ws_bytes),
                    TWM_DEVICE_ERROR, "batched decode launch");
            return TWM_OK;
        });
    }
}

// The knobs of a launch form, saved and set as one
struct Knobs {
    int kernel, nt, waves, sub, sub_waves, prefill_bm;
};
static Knobs knobs_of(const twm_ctx *c) { return Knobs{c->force_kernel, c->force_nt, c->force_waves, c->force_sub, c->force_sub_waves, c->prefill_bm}; }
static void set_knobs(twm_ctx *c, const Knobs &k)
{
    c->force_kernel = k.kernel;
    c->force_nt = k.nt;
    c->force_waves = k.waves;
    c->force_sub = k.sub;
    c->force_sub_waves = k.sub_waves;
    c->prefill_bm = k.prefill_bm;
}

// With nothing forced by the caller, a plan that twm_weight_tune measured for this weight and row count is what runs.
static int gemm_common(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, const OutSpec &out,
                       uint32_t splits, const char *who, float *swiglu_out = nullptr, uint32_t gate_act = 2)
{
    const Knobs user = knobs_of(ctx);
    const bool free_choice = !splits && !user.kernel && !user.nt && !user.waves && !user.sub && !user.sub_waves && !user.prefill_bm;
    const TunedPlan *tp = (m >= 1 && free_choice && !swiglu_out && a_dtype == TWM_F16) ? &w->tuned[tune_bucket(m)] : nullptr;
    if (!tp || !tp->valid) return gemm_dispatch(ctx, w, a_dev, a_dtype, m, out, splits, who, swiglu_out, gate_act);
    set_knobs(ctx, Knobs{tp->kernel, tp->nt, tp->waves, tp->sub, tp->sub_waves, tp->prefill_bm});
    const int rc = gemm_dispatch(ctx, w, a_dev, a_dtype, m, out, tp->splits, who, swiglu_out, gate_act);
    set_knobs(ctx, user);
    return rc;
}

// Candidate launch forms for `m` rows: what the option knobs can ask for.  The first entry is the planners' own choice.
static void tune_candidates(uint32_t m, uint32_t k_chunks, std::vector<TunedPlan> &out)
{
    auto add = [&](int kernel, int nt, int waves, int sub, int sub_waves, int splits, int bm) {
        out.push_back(TunedPlan{1, (uint8_t)kernel, (uint8_t)nt, (uint8_t)waves, (uint8_t)sub, (uint8_t)sub_waves, (uint8_t)splits, (uint8_t)bm});
    };
    add(0, 0, 0, 0, 0, 0, 0);
    const uint32_t passes16 = (k_chunks + 3) / 4, passes32 = (k_chunks + 1) / 2;
    if (m <= 16) {
        // sub-tile kernel: one pass per wave where sixteen waves cover K, else the pass loop on 4, 8 or 16 waves
        for (int sub : {16, 32}) {
            const uint32_t passes = sub == 16 ? passes16 : passes32;
            if (passes <= 16) add(0, 0, 0, sub, (int)passes, 0, 0);
            for (int wv : {4, 8, 16})
                if ((uint32_t)wv < passes || (passes <= 16 && (uint32_t)wv != passes)) add(0, 0, 0, sub, wv, 0, 0);
        }
    }
    if (m <= 4) {
        for (int wv : {8, 16})
            for (int sp : {1, 2, 4, 8}) add(2, 1, wv, 0, 0, sp, 0);   // whole 64-column tiles, K split over workgroups
        add(2, 2, 8, 0, 0, 1, 0);
    } else if (m <= 32) {
        for (int sp : {1, 2, 3, 4, 6, 8}) add(3, 0, 0, 0, 0, sp, 0);  // streaming kernel
        for (int nt : {1, 2, 3, 4})                                     // LDS-shared kernel: tiles per wave / quads per workgroup
            for (int wv : {0, 8, 16})                                   // k-slices
                for (int sp : {1, 2, 3, 4, 6})
                    if (!(wv == 16 && nt != 1) && !(wv == 8 && nt == 3)) add(4, nt, wv, 0, 0, sp, 0);
    } else {
        for (int bm : {64, 128, 192})
            for (int sp : {1, 2, 3, 4, 6, 8}) add(0, 0, 0, 0, 0, sp, bm);
    }
}

int twm_weight_tune(twm_ctx *ctx, twm_weight *w, const uint32_t *ms, uint32_t count)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_weight_tune: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_weight_tune: weight belongs to another context");
    if (ctx->capturing) return api_fail(TWM_UNSUPPORTED_OP, "twm_weight_tune: not allowed inside a graph capture");
    if (count != 0 && !ms) return api_fail(TWM_INVALID_HANDLE, "twm_weight_tune: null row counts");
    if (w->copy_bytes == 0 || w->k == 0 || w->n == 0) return TWM_OK;
    uint32_t m_max = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (ms[i] == 0 || ms[i] > 65536u) return api_fail(TWM_SHAPE_ERROR, "twm_weight_tune: row counts are 1 .. 65536");
        if (ms[i] > m_max) m_max = ms[i];
    }
    if (m_max == 0) return TWM_OK;
    // synthetic f16 activations (a fixed pattern of small values) and an output, both released at the end
    void *a_dev = nullptr, *c_dev = nullptr;
    const size_t a_bytes = (size_t)m_max * w->k * 2, c_bytes = (size_t)m_max * w->n * 4;
    if (hipMalloc(&a_dev, a_bytes) != hipSuccess || hipMalloc(&c_dev, c_bytes) != hipSuccess) {
        if (a_dev) (void)hipFree(a_dev);
        return api_fail(TWM_MEMORY_ERROR, "twm_weight_tune: hipMalloc of the trial buffers");
    }
    int rc = TWM_OK;
    {
        std::vector<uint16_t> host(a_bytes / 2);
        uint32_t x = 2463534242u;
        for (auto &h : host) {
            x ^= x << 13; x ^= x >> 17; x ^= x << 5;
            h = (uint16_t)(0x3000u + (x & 0x0FFFu)) | (uint16_t)((x >> 16) & 0x8000u);  // +-[0.125, 0.5)
        }
        rc = twm_memcpy_h2d(ctx, a_dev, host.data(), a_bytes);
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (rc == TWM_OK && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess))
        rc = api_fail(TWM_DEVICE_ERROR, "twm_weight_tune: hipEventCreate");
    // The trials rotate over copies of the weight that together exceed the 256 MB cache in front of HBM, as the layers
    // of a model do: timed on one resident copy, the forms that are best from the caches would win.
    if (rc == TWM_OK) rc = weight_ensure(ctx, w, kCopyTile | kCopyCol, "twm_weight_tune");
    std::vector<twm_weight> clones;
    if (rc == TWM_OK) {
        size_t want = ((size_t)320 << 20) / (2 * w->copy_bytes) + 1;
        if (want > 32) want = 32;
        for (size_t c = 0; c + 1 < want && rc == TWM_OK; c++) {
            twm_weight cl = *w;
            cl.qw = cl.sc = cl.cq = nullptr;
            if (hipMalloc(&cl.qw, w->copy_bytes) != hipSuccess || hipMalloc(&cl.cq, w->copy_bytes) != hipSuccess) {
                if (cl.qw) (void)hipFree(cl.qw);
                (void)hipGetLastError();
                break;   // (fewer copies: the trials are warmer than a model's layers would be, but still fair among themselves)
            }
            cl.sc = (char *)cl.qw + (size_t)w->n_tiles * w->k_chunks * 1024;
            if (hipMemcpyAsync(cl.qw, w->qw, w->copy_bytes, hipMemcpyDeviceToDevice, ctx->stream) != hipSuccess ||
                hipMemcpyAsync(cl.cq, w->cq, w->copy_bytes, hipMemcpyDeviceToDevice, ctx->stream) != hipSuccess)
                rc = api_fail(TWM_DEVICE_ERROR, "twm_weight_tune: copying the weight");
            clones.push_back(cl);
        }
    }
    uint32_t turn = 0;
    auto next_weight = [&]() -> const twm_weight * {
        const size_t n = clones.size() + 1;
        const size_t at = turn++ % n;
        return at == 0 ? w : &clones[at - 1];
    };
    const Knobs user = knobs_of(ctx);
    OutSpec out;
    memset(&out, 0, sizeof out);
    out.count = 1;
    out.seg[0].ptr = (float *)c_dev;
    out.seg[0].width = w->n;
    for (uint32_t i = 0; i < count && rc == TWM_OK; i++) {
        const uint32_t m = ms[i];
        std::vector<TunedPlan> cands;
        tune_candidates(m, w->k_chunks, cands);
        const int reps = m <= 32 ? 24 : 6;
        float best_ms = 0.f, own_ms = 0.f;
        TunedPlan best = cands[0];
        for (size_t c = 0; c < cands.size(); c++) {
            const TunedPlan &p = cands[c];
            set_knobs(ctx, Knobs{p.kernel, p.nt, p.waves, p.sub, p.sub_waves, p.prefill_bm});
            bool ok = true;
            for (int r = 0; r < 2 && ok; r++) ok = gemm_dispatch(ctx, next_weight(), a_dev, TWM_F16, m, out, p.splits, "twm_weight_tune") == TWM_OK;
            float ms_taken = 0.f;
            // timed as the decode loop runs it: a captured graph of `reps` launches over the rotating copies, replayed
            hipGraph_t graph = nullptr;
            hipGraphExec_t exec = nullptr;
            if (ok) {
                ok = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed) == hipSuccess;
                bool launched = ok;
                for (int r = 0; r < reps && launched; r++)
                    launched = gemm_dispatch(ctx, next_weight(), a_dev, TWM_F16, m, out, p.splits, "twm_weight_tune") == TWM_OK;
                if (ok) ok = hipStreamEndCapture(ctx->stream, &graph) == hipSuccess && launched;
                ok = ok && graph && hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess;
            }
            for (int run = 0; run < 3 && ok; run++) {   // one untimed replay, then the faster of two timed ones
                float t = 0.f;
                (void)hipEventRecord(e0, ctx->stream);
                ok = hipGraphLaunch(exec, ctx->stream) == hipSuccess;
                (void)hipEventRecord(e1, ctx->stream);
                ok = ok && hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&t, e0, e1) == hipSuccess;
                if (run == 1 || (run == 2 && t < ms_taken)) ms_taken = t;
            }
            if (exec) (void)hipGraphExecDestroy(exec);
            if (graph) (void)hipGraphDestroy(graph);
            if (!ok) {   // a form this shape does not take: skipped
                (void)hipGetLastError();
                continue;
            }
            if (c == 0) own_ms = ms_taken;
            if (best_ms == 0.f || ms_taken < best_ms) {
                best_ms = ms_taken;
                best = p;
            }
        }
        // the planners' choice stays unless a forced form beats it by more than 2 % (timing noise)
        TunedPlan &slot = w->tuned[tune_bucket(m)];
        if (own_ms > 0.f && best_ms < 0.98f * own_ms && (best.kernel || best.nt || best.waves || best.sub || best.sub_waves || best.splits || best.prefill_bm))
            slot = best;
        else
            memset(&slot, 0, sizeof slot);
    }
    set_knobs(ctx, user);
    (void)hipStreamSynchronize(ctx->stream);
    for (twm_weight &cl : clones) {
        (void)hipFree(cl.qw);
        (void)hipFree(cl.cq);
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(a_dev);
    (void)hipFree(c_dev);
    return rc;
}

int twm_weight_tuned_plan(const twm_weight *w, uint32_t m, int *knobs8)
{
    if (!w || !knobs8 || m == 0) return api_fail(TWM_INVALID_HANDLE, "twm_weight_tuned_plan: null argument");
    const TunedPlan &p = w->tuned[tune_bucket(m)];
    const int v[8] = {p.valid, p.kernel, p.nt, p.waves, p.sub, p.sub_waves, p.splits, p.prefill_bm};
    for (int i = 0; i < 8; i++) knobs8[i] = v[i];
    return TWM_OK;
}

int twm_gemm(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *c_dev, uint32_t splits)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_gemm: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_gemm: weight belongs to another context");
    if (m != 0 && w->n != 0 && !c_dev) return api_fail(TWM_INVALID_HANDLE, "twm_gemm: null output");
    OutSpec out;
    memset(&out, 0, sizeof out);
    out.count = 1;
    out.seg[0].ptr = c_dev;
    out.seg[0].start = 0;
    out.seg[0].width = w->n;
    return gemm_common(ctx, w, a_dev, a_dtype, m, out, splits, "twm_gemm");
}

// twm_gemm with f16 result rows: the kernels store f32 (what the reference's buffers hold), so the rows are computed in
// blocks into the back half of the context's scratch and rounded from there by the cast kernel -- no allocation, one
// more launch per block; the front half stays the launch's own scratch (split-K sums, f32 activation terms).
int twm_gemm_f16out(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, uint16_t *c_dev_f16,
                    uint32_t splits)
{
    const char *who = "twm_gemm_f16out";
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "%s: null handle", who);
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "%s: weight belongs to another context", who);
    if (m != 0 && w->n != 0 && !c_dev_f16) return api_fail(TWM_INVALID_HANDLE, "%s: null output", who);
    if (a_dtype != TWM_F16 && a_dtype != TWM_F32) return api_fail(TWM_UNSUPPORTED_OP, "%s: activations must be f16 or f32", who);
    if (m == 0 || w->n == 0) return TWM_OK;
    const size_t row_bytes = (size_t)w->n * 4, half = (ctx->ws_bytes / 2) & ~(size_t)255;
    if (!ctx->ws || row_bytes > half)
        return api_fail(TWM_MEMORY_ERROR, "%s: one row of f32 results (%zu bytes) does not fit half of the context's scratch; "
                        "use twm_gemm and twm_cast_f32_to_f16", who, row_bytes);
    uint32_t block = half / row_bytes < m ? (uint32_t)(half / row_bytes) : m;
    if (block >= 128) block -= block % 128;   // (whole prefill row blocks)
    float *stage = (float *)((char *)ctx->ws + ctx->ws_bytes - half);
    const size_t a_row_bytes = (size_t)w->k * (a_dtype == TWM_F32 ? 4 : 2), saved = ctx->ws_bytes;
    int rc = TWM_OK;
    ctx->ws_bytes = saved - half;
    for (uint32_t m0 = 0; m0 < m && rc == TWM_OK; m0 += block) {
        const uint32_t rows = m - m0 < block ? m - m0 : block;
        rc = twm_gemm(ctx, w, (const char *)a_dev + (size_t)m0 * a_row_bytes, a_dtype, rows, stage, splits);
        if (rc == TWM_OK && launch_cast(ctx->stream, stage, c_dev_f16 + (size_t)m0 * w->n, (size_t)rows * w->n, true) != hipSuccess)
            rc = api_fail(TWM_DEVICE_ERROR, "%s: cast kernel launch: %s", who, hipGetErrorString(hipGetLastError()));
    }
    ctx->ws_bytes = saved;
    return rc;
}

int twm_gemm_split_bias(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m,
                        float *const *outs_dev, const float *const *biases_dev, const uint32_t *ns, uint32_t count,
                        uint32_t splits)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_split_bias: null handle");
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_split_bias: weight belongs to another context");
    if (!outs_dev || !ns) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_split_bias: null array");
    if (count == 0 || count > (uint32_t)kMaxSegs)
        return api_fail(TWM_SHAPE_ERROR, "twm_gemm_split_bias: between 1 and %d outputs are supported", kMaxSegs);
    OutSpec out;
    memset(&out, 0, sizeof out);
    uint64_t total = 0;
    uint32_t used = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (ns[i] == 0) continue;
        if (m != 0 && !outs_dev[i]) return api_fail(TWM_INVALID_HANDLE, "twm_gemm_split_bias: null output %u", i);
        out.seg[used].ptr = outs_dev[i];
        out.seg[used].start = (uint32_t)total;
        out.seg[used].width = ns[i];
        out.seg[used].bias = biases_dev ? biases_dev[i] : nullptr;
        used++;
        total += ns[i];
    }
    out.count = used;
    if (total != w->n) return api_fail(TWM_SHAPE_ERROR, "twm_gemm_split_bias: outputs cover %llu columns, weight has %u",
                                   (unsigned long long)total, w->n);
    return gemm_common(ctx, w, a_dev, a_dtype, m, out, splits, "twm_gemm_split_bias");
}

int twm_gemm_split(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *const *outs_dev,
                   const uint32_t *ns, uint32_t count, uint32_t splits)
{
    return twm_gemm_split_bias(ctx, w, a_dev, a_dtype, m, outs_dev, nullptr, ns, count, splits);
}

static int gemm_gated(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *out_dev,
                      uint32_t splits, uint32_t act, const char *who)
{
    if (!ctx || !w) return api_fail(TWM_INVALID_HANDLE, "%s: null handle", who);
    if (w->ctx != ctx) return api_fail(TWM_INVALID_HANDLE, "%s: weight belongs to another context", who);
    if (!w->paired) return api_fail(TWM_UNSUPPORTED_OP, "%s: the weight was not built by twm_weight_gate_up", who);
    uint32_t ffn = w->n / 2;
    if (m == 0 || ffn == 0) return TWM_OK;
    if (!out_dev) return api_fail(TWM_INVALID_HANDLE, "%s: null output", who);
    if (((uintptr_t)out_dev & 15) != 0) return api_fail(TWM_SHAPE_ERROR, "%s: the output must be 16-byte aligned", who);
    if (w->k == 0) return twm_memset_zero(ctx, out_dev, (size_t)m * ffn * 4);  // gate(0) * 0
    OutSpec out;
    memset(&out, 0, sizeof out);
    return gemm_common(ctx, w, a_dev, a_dtype, m, out, splits, who, out_dev, act);
}

int twm_gemm_swiglu(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *out_dev,
                    uint32_t splits)
{
    return gemm_gated(ctx, w, a_dev, a_dtype, m, out_dev, splits, 2, "twm_gemm_swiglu");
}

int twm_gemm_geglu(twm_ctx *ctx, const twm_weight *w, const void *a_dev, int a_dtype, uint32_t m, float *out_dev,
                   uint32_t splits)
{
    return gemm_gated(ctx, w, a_dev, a_dtype, m, out_dev, splits, 1, "twm_gemm_geglu");
}

}  // extern "C"

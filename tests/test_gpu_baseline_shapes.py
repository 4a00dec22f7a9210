"""GPU parity at the exact benchmark shapes, under the library's automatic plan, through the C ABI:
the LLaMA-7B MLP prefill GEMMs (M = 512 and 2048), every Qwen-7B projection at M = 4, 8, 16, 32, the LM head
3584 -> 152064 with the argmax of its output, and the Qwen-7B-shaped layer replayed as one graph.

Truth is the oracle's f64 dequant-then-matmul: on the exact weights f32(scale) * (q - 8) for the decode kernels
(M <= 32), on the FP16 Q4 unpack f16(scale * (q - 8)) for the prefill GEMM (the reference's prefill route,
quantize.rs:534-571 then an FP16 GEMM, :1825-1858).  The large prefill products are compared on samples that touch
every row block and every column block: all columns of a few rows per 64-row block, and all rows of a few columns
per 64-column block.
"""
import numpy as np
import pytest

import tensorwarp_amd as T
from oracle import twm_oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-2       # the stated tolerance
TIGHT = 2e-4     # what f32 accumulation on exact weights delivers
PREFILL = 1e-3   # one f32 accumulator over all of K on f16-rounded weights

SHAPES_7B = {"qkv": (3584, 4608), "o": (3584, 3584), "gate_up": (3584, 37888), "down": (18944, 3584)}


@pytest.fixture(scope="module")
def dev():
    d = T.WarpDevice(0)
    yield d
    d.close()


def f16_as_f32(bits):
    return bits.view(np.float16).astype(np.float32)


def rel_err(c, truth, scale=None):
    truth = np.asarray(truth, np.float64)
    top = np.abs(truth).max() if scale is None else scale
    denom = np.maximum(np.abs(truth), 1e-3 * top + 1e-30)
    return float((np.abs(np.asarray(c, np.float64) - truth) / denom).max())


def synth(k, n, m, seed):
    return O.synth_packed(k, n, seed * 3 + 1), O.synth_scales(k, n, seed * 3 + 2), O.synth_act_f16(m, k, seed * 3 + 3)


def run_gemm(dev, w, a16, m, n, splits=0, a_f32=False):
    a_dev = T.GpuTensor.from_host(dev, f16_as_f32(a16)) if a_f32 else T.GpuTensor.from_host(dev, a16, "f16")
    c = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))   # NaN canary: every output must be written
    T.gemm(dev, w, a_dev, m, c, splits)
    out = c.to_host().reshape(m, n)
    a_dev.free()
    c.free()
    return out


def sample_indices(count, block, rng):
    """First, last and one random index of every block of `block`, plus the very last index."""
    idx = set()
    for b0 in range(0, count, block):
        b1 = min(b0 + block, count)
        idx.update((b0, b1 - 1, int(rng.integers(b0, b1))))
    idx.add(count - 1)
    return np.array(sorted(idx))


def check_prefill_sampled(got, a16, packed, scales, m, k, n, rng, tag):
    w16 = O.dequant_f16(packed, scales, k, n).view(np.float16).reshape(k, n)
    a = f16_as_f32(a16).reshape(m, k).astype(np.float64)
    assert not np.isnan(got).any(), tag
    rows = sample_indices(m, 64, rng)
    cols = sample_indices(n, 64, rng)
    t_rows = a[rows] @ w16.astype(np.float64)              # [rows, all columns]
    t_cols = a @ w16[:, cols].astype(np.float64)           # [all rows, cols]
    top = max(np.abs(t_rows).max(), np.abs(t_cols).max())
    e1, e2 = rel_err(got[rows], t_rows, top), rel_err(got[:, cols], t_cols, top)
    print("%s: %d rows x all, all x %d columns, rel err %.2e / %.2e" % (tag, len(rows), len(cols), e1, e2), flush=True)
    assert max(e1, e2) < PREFILL and max(e1, e2) < TOL, tag
    # the other reading (exact f32 weights): agreement relative to the largest output
    exact_rows = O.gemm_f64(f16_as_f32(a16).reshape(m, k)[rows[:8]], packed, scales, 8, k, n) if len(rows) >= 8 else None
    if exact_rows is not None:
        assert np.abs(got[rows[:8]] - exact_rows).max() / np.abs(exact_rows).max() < 1e-3, tag


# ---------------------------------------------------------------- LLaMA-7B MLP prefill (M = 512, 2048)

@pytest.mark.parametrize("k,n", [(4096, 11008), (11008, 4096)])
@pytest.mark.parametrize("m", [512, 2048])
def test_prefill_llama7b_mlp_shapes(dev, m, k, n):
    rng = np.random.default_rng(m + k)
    packed, scales, a16 = synth(k, n, m, 7000 + m + k % 97)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    got = run_gemm(dev, w, a16, m, n)
    check_prefill_sampled(got, a16, packed, scales, m, k, n, rng, "M=%d %d->%d f16 rows" % (m, k, n))
    again = run_gemm(dev, w, a16, m, n)
    assert np.array_equal(got, again)                      # no atomics anywhere: run-to-run identical
    if m == 512:
        got32 = run_gemm(dev, w, a16, m, n, a_f32=True)    # f32 rows are rounded to f16 first: same values here
        assert np.array_equal(got32, got)
    w.free()


@pytest.mark.parametrize("bm,m,n", [(128, 680, 5848), (64, 680, 5848), (128, 1024, 8192), (192, 680, 5848), (192, 1024, 11008)])
def test_prefill_xcd_tile_order_with_ragged_bands(dev, bm, m, n):
    # The tile order that keeps an XCD's workgroups on a patch of the output is taken from 128 tiles on.  680 rows x
    # 5848 columns: 6 x 23 = 138 tiles of 128 x 256 (not a multiple of 8, last band two row blocks high, last row and
    # column blocks ragged) and 11 x 23 = 253 tiles of 64 x 256 (bands of eight, the last three high); 1024 x 8192
    # is the even case; 192-column blocks make 6 x 31 (ragged last block) and 8 x 58 tiles.  Every output is compared (K is shallow), and a NaN canary catches a tile nobody wrote.
    k = 256
    packed, scales, a16 = synth(k, n, m, 7100 + bm + n)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    w16 = O.dequant_f16(packed, scales, k, n).view(np.float16).astype(np.float64).reshape(k, n)
    exact = f16_as_f32(a16).reshape(m, k).astype(np.float64) @ w16
    try:
        dev.set_option("prefill_bm", bm)
        got = run_gemm(dev, w, a16, m, n, splits=1)
        assert not np.isnan(got).any()
        assert rel_err(got, exact) < PREFILL
    finally:
        dev.set_option("prefill_bm", 0)
    w.free()


# ---------------------------------------------------------------- batched decode, Qwen-7B projections

@pytest.mark.parametrize("name", list(SHAPES_7B))
@pytest.mark.parametrize("m", [4, 8, 16, 32])
def test_batched_decode_qwen7b_all_projections(dev, m, name):
    k, n = SHAPES_7B[name]
    packed, scales, a16 = synth(k, n, m, 7200 + m + k % 89 + n % 83)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    truth = O.gemm_f64(f16_as_f32(a16).reshape(m, k), packed, scales, m, k, n)
    got = run_gemm(dev, w, a16, m, n)
    err = rel_err(got, truth)
    print("M=%d %s %d->%d splits=%d rel err %.2e" % (m, name, k, n, T.pick_splits(k, n, m), err), flush=True)
    assert err < TIGHT and err < TOL
    # a row's result does not depend on the batch it is in, beyond f32 summation order
    alone = run_gemm(dev, w, a16[m - 1:m], 1, n)
    assert rel_err(alone[0], got[m - 1]) < TIGHT
    # f32 rows (what the reference's decode loop holds) on the same plan family
    got32 = run_gemm(dev, w, a16, m, n, a_f32=True)
    assert rel_err(got32, truth) < TIGHT
    w.free()


@pytest.mark.parametrize("name", list(SHAPES_7B))
def test_f32_rows_qwen7b_all_projections(dev, name):
    # The reference's decode loop holds f32 activations (generate.rs:2153): one and two rows of f32 values that are not
    # f16 values, on the repacked handle (each lane splits one shared piece of the row; deep K in the pipelined pass
    # loop) and, for one row, on the reference's arrays as they are.
    k, n = SHAPES_7B[name]
    packed, scales, _ = synth(k, n, 1, 7400 + k % 89 + n % 83)
    a_raw = (O.synth_normal_f32(2 * k, 7450 + n % 71) * np.float32(1.37)).reshape(2, k)
    truth = O.gemm_f64(a_raw, packed, scales, 2, k, n)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    for m in (1, 2):
        c = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))
        T.gemm(dev, w, T.GpuTensor.from_host(dev, np.ascontiguousarray(a_raw[:m])), m, c)
        err = rel_err(c.to_host().reshape(m, n), truth[:m])
        print("f32 rows M=%d %s rel err %.2e" % (m, name, err), flush=True)
        assert err < TIGHT
    pd, sd = T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales, "f16")
    c1 = T.GpuTensor.from_host(dev, np.full((n,), np.nan, np.float32))
    T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, np.ascontiguousarray(a_raw[0])), pd, sd, c1, n, k)
    assert rel_err(c1.to_host(), truth[0]) < TIGHT
    w.free()


# ---------------------------------------------------------------- planner branches away from the benchmark shapes

@pytest.mark.parametrize("k,n,ms,want", [
    # 65 .. 128 column tiles on a deep K: one row runs 16-column sub-tiles in the pipelined pass loop (f16 and f32 rows)
    (13824, 5120, (1,), "k_gemv4s: 16-column sub-tiles, 8 waves"),
    # a wide matrix whose last round of whole tiles is under 70 % full: the sub-tiles up to four f16 rows
    (4096, 22016, (3, 4), "k_gemv4s: 16-column sub-tiles, 8 waves"),
])
def test_planner_branches_on_other_model_shapes(dev, k, n, ms, want):
    packed, scales, a16 = synth(k, n, max(ms), 7700 + k % 97 + n % 89)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    for m in ms:
        assert dev.plan(k, n, m).startswith(want), dev.plan(k, n, m)
        truth = O.gemm_f64(f16_as_f32(a16[:m]).reshape(m, k), packed, scales, m, k, n)
        assert rel_err(run_gemm(dev, w, a16[:m], m, n), truth) < TIGHT, m
        if m == 1:
            assert dev.plan(k, n, m, dtype="f32").startswith(want)
            assert rel_err(run_gemm(dev, w, a16[:m], m, n, a_f32=True), truth) < TIGHT
    w.free()


# ---------------------------------------------------------------- LM head 3584 -> 152064 + argmax

def test_lm_head_gemv_and_argmax_at_vocabulary_width(dev):
    k, n = 3584, 152064
    packed, scales, a16 = synth(k, n, 8, 7300)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    for m in (1, 8):
        a = f16_as_f32(a16[:m]).reshape(m, k)
        truth = O.gemm_f64(a, packed, scales, m, k, n)
        a_dev = T.GpuTensor.from_host(dev, a16[:m], "f16")
        c = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))
        T.gemm(dev, w, a_dev, m, c)
        ids = T.GpuTensor.from_host(dev, np.full(m, -7, np.int32))
        T.argmax(dev, c, ids, m, n)
        got = c.to_host().reshape(m, n)
        err = rel_err(got, truth)
        print("LM head M=%d rel err %.2e" % (m, err), flush=True)
        assert err < TIGHT
        # the token id: bit-exact against the oracle's scan of the same logits, and the f64 truth's maximum is
        # either the same column or within the error bar of it
        assert np.array_equal(ids.to_host(), O.argmax(got, m, n))
        for r in range(m):
            best = int(np.argmax(truth[r]))
            assert ids.to_host()[r] == best or abs(truth[r, best] - truth[r, ids.to_host()[r]]) <= TIGHT * np.abs(truth[r]).max()
        for t in (a_dev, c, ids):
            t.free()
    w.free()


# ---------------------------------------------------------------- the Qwen-7B-shaped layer as one graph

def test_qwen7b_layer_graph_replays_match_eager(dev):
    ws, acts, outs, eager = {}, {}, {}, {}
    for i, (nm, (k, n)) in enumerate(SHAPES_7B.items()):
        p, s, a16 = synth(k, n, 1, 7400 + i)
        ws[nm] = T.MarlinWeight.upload(dev, p, s, k, n)
        acts[nm] = T.GpuTensor.from_host(dev, a16, "f16")
        outs[nm] = T.GpuTensor.zeros(dev, (n,), "f32")
        T.gemm(dev, ws[nm], acts[nm], 1, outs[nm])
        eager[nm] = outs[nm].to_host()
        assert rel_err(eager[nm], O.gemm_f64(f16_as_f32(a16).reshape(1, k), p, s, 1, k, n)[0]) < TIGHT, nm

    def body():
        for nm in SHAPES_7B:
            T.gemm(dev, ws[nm], acts[nm], 1, outs[nm])

    graph = T.GraphCapture.record_with_device(dev, body)
    for rep in range(4):
        for nm, (k, n) in SHAPES_7B.items():
            outs[nm].copy_from_host(np.full(n, np.nan, np.float32))
        graph.replay()
        dev.synchronize()
        for nm in SHAPES_7B:
            assert np.array_equal(outs[nm].to_host(), eager[nm]), (rep, nm)
        T.gemm(dev, ws["down"], acts["down"], 1, outs["down"], 5)      # eager work between replays
        dev.synchronize()
    graph.destroy()
    for nm in SHAPES_7B:
        ws[nm].free()

"""Pins the CPU oracle (oracle/twm_oracle.c) before anything is checked against it.

Every check here is independent of the oracle's own formulas: numpy's IEEE
binary16, the committed fixtures (made by tests/golden/make_fixtures.py from a
numpy restatement), closed forms, brute force, and the known answers the
reference's own tests hold (gemm.rs:185-190; generators quantize.rs:3009,
3054-3059, 3618-3620).
"""
import os

import numpy as np
import pytest

from oracle import twm_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")
CASES = ["lcg_k64_n8_m1", "lcg_k128_n64_m4", "synth_k128_n64_m1", "synth_k256_n80_m5",
         "synth_k160_n33_m17"]


def load(name):
    return np.load(os.path.join(GOLD, name + ".npz"))


# ---------- binary16 conversions ----------

def test_f16_to_f32_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    got = O.f16_to_f32(h)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_f32_to_f16_corners_fixture():
    d = load("f16_corners")
    assert np.array_equal(O.f32_to_f16(d["vals"]), d["bits"])


def test_f32_to_f16_random_and_ties():
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    f = f[np.isfinite(f)]
    # exact ties between neighbouring halves, normal and subnormal
    h = np.arange(0, 0x7BFF, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    ties = ((lo + hi) / 2).astype(np.float32)
    f = np.concatenate([f, ties, -ties, np.nextafter(ties, np.float32(np.inf)),
                        np.nextafter(ties, np.float32(-np.inf))])
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.f32_to_f16(f), want)


def test_f32_to_f16_nan_stays_nan():
    out = O.f32_to_f16(np.array([np.nan, -np.nan], np.float32))
    assert np.all((out & 0x7C00) == 0x7C00) and np.all((out & 0x3FF) != 0)


# ---------- quantizers ----------

@pytest.mark.parametrize("name", ["lcg_k64_n8_m1", "lcg_k128_n64_m4"])
def test_quantize_tw_marlin_matches_fixture(name):
    d = load(name)
    k, n = int(d["k"]), int(d["n"])
    packed, scales = O.quantize_tw_marlin_nk(np.ascontiguousarray(d["w_kn"].T), k, n)
    assert np.array_equal(packed, d["packed"])
    assert np.array_equal(scales, d["scales"])


def test_quantizer_round_half_away_and_clamp():
    # one group whose amax is 7 so that inv == 1 and v*inv hits exact .5 ties
    v = np.zeros((1, 32), np.float32)
    v[0, :8] = [7.0, -7.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5]
    packed, scales = O.quantize_tw_marlin_nk(v, 32, 1)
    q = np.empty(32, np.int32)
    q[0::2] = packed & 0xF
    q[1::2] = packed >> 4
    # half away from zero: 0.5->1, -0.5->-1, 1.5->2, -1.5->-2, 2.5->3, -2.5->-3 (half-to-even would give 0,0,2,-2,2,-2)
    assert list(q[:8] - 8) == [7, -7, 1, -1, 2, -2, 3, -3]
    assert np.all(q[8:] == 8)
    assert scales[0] == np.float16(1.0).view(np.uint16)


def test_quantizer_zero_group_and_nearest_grid_point():
    rng = np.random.default_rng(5)
    k, n = 96, 7
    w = rng.standard_normal((n, k)).astype(np.float32)
    w[3, 32:64] = 0.0                                   # all-zero group -> scale 0, q = 8
    packed, scales = O.quantize_tw_marlin_nk(w, k, n)
    pk = packed.reshape(k // 32, n, 16)
    assert np.all(pk[1, 3] == 0x88) and scales.reshape(k // 32, n)[1, 3] == 0
    # brute force: with the f32 scale amax/7, the chosen q is the nearest of the 16 grid points
    q = np.empty((k // 32, n, 32), np.int32)
    q[:, :, 0::2] = pk & 0xF
    q[:, :, 1::2] = pk >> 4
    v = w.reshape(n, k // 32, 32).transpose(1, 0, 2)
    amax = np.abs(v).max(axis=2, keepdims=True)
    scale = amax / np.float32(7.0)
    grid = (np.arange(16) - 8).astype(np.float32)
    err_all = np.abs(v[..., None] - scale[..., None] * grid)       # [G,N,32,16]
    chosen = np.take_along_axis(err_all, q[..., None], axis=3)[..., 0]
    assert np.all(chosen <= err_all.min(axis=3) + 1e-6 * amax)
    assert q.min() >= 1 and q.max() <= 15                          # this quantizer never emits q=0


def test_q4_0_roundtrip_reference_generator():
    # reference test q4_0_roundtrip_correctness (quantize.rs:3001-3042): x[i]=((7i+3)%200)*0.01-1
    i = np.arange(1024)
    x = (((i * 7 + 3) % 200).astype(np.float32) * np.float32(0.01) - np.float32(1.0))
    y = O.q4_0_roundtrip(x)
    amax = np.abs(x.reshape(-1, 32)).max(axis=1)
    # property the reference prints: quantization error <= scale/2 (+ulp)
    assert np.all(np.abs(x - y).reshape(-1, 32) <= (amax / 7 / 2 * 1.0001)[:, None])
    # dequantized values are integer multiples of the block scale in [-7, 7]
    ratio = y.reshape(-1, 32) / (amax / np.float32(7.0))[:, None]
    assert np.allclose(ratio, np.round(ratio), atol=1e-4) and np.abs(ratio).max() <= 7.0001


def test_q4_col_major_and_kn_quantizers_agree():
    rng = np.random.default_rng(9)
    k, n = 64, 5
    w_kn = rng.standard_normal((k, n)).astype(np.float32)
    a = O.quantize_weights_q4_0_kn(w_kn, k, n)
    b = O.quantize_q4_col_major_nk(np.ascontiguousarray(w_kn.T), k, n)
    assert np.array_equal(a, b)
    # block-major placement (what quantize.rs:435 writes) is the same blocks transposed
    bm = O.quantize_weights_q4_0_kn(w_kn, k, n, block_major=True).reshape(k // 32, n, 20)
    assert np.array_equal(bm.transpose(1, 0, 2).reshape(-1), a)


# ---------- transforms ----------

def test_reorder_equals_direct_quantize():
    # invariant: reorder(quant_q4_colmajor(W)) == cpu_quantize_tw_marlin(W^T)
    rng = np.random.default_rng(11)
    k, n = 128, 19
    w_nk = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    q4 = O.quantize_q4_col_major_nk(w_nk, k, n)
    p1, s1 = O.reorder_to_tw_marlin(q4, k, n)
    p2, s2 = O.quantize_tw_marlin_nk(w_nk, k, n)
    assert np.array_equal(p1, p2) and np.array_equal(s1, s2)
    # reorder is a pure permutation of the 16-byte records
    blocks = q4.reshape(n, k // 32, 20)
    assert np.array_equal(p1.reshape(k // 32, n, 16), blocks[:, :, 4:].transpose(1, 0, 2))


def test_fuse_is_concat_along_n():
    rng = np.random.default_rng(13)
    k = 96
    ns = [5, 3, 8]
    mats = []
    for ni in ns:
        mats.append((rng.integers(0, 256, (k // 32) * ni * 16, dtype=np.uint8),
                     rng.integers(0, 0x3C00, (k // 32) * ni, dtype=np.uint16)))
    fp, fs = O.fuse_tw_marlin_n(mats, k, ns)
    want_p = np.concatenate([m[0].reshape(k // 32, ni, 16) for m, ni in zip(mats, ns)], axis=1)
    want_s = np.concatenate([m[1].reshape(k // 32, ni) for m, ni in zip(mats, ns)], axis=1)
    assert np.array_equal(fp, want_p.reshape(-1)) and np.array_equal(fs, want_s.reshape(-1))
    # dequant(fuse) == hstack(dequant)
    d = O.dequant_f32(fp, fs, k, sum(ns))
    parts = [O.dequant_f32(m[0], m[1], k, ni) for m, ni in zip(mats, ns)]
    assert np.array_equal(d, np.hstack(parts))


def test_split_qkv_and_gate_up():
    rng = np.random.default_rng(17)
    h, kv, batch = 12, 4, 3
    x = rng.standard_normal((batch, h + 2 * kv)).astype(np.float32)
    q, kk, v = O.split_qkv(x, h, kv, batch)
    assert np.array_equal(q.reshape(batch, h), x[:, :h])
    assert np.array_equal(kk.reshape(batch, kv), x[:, h:h + kv])
    assert np.array_equal(v.reshape(batch, kv), x[:, h + kv:])
    y = rng.standard_normal((batch, 10)).astype(np.float32)
    g, u = O.split_gate_up(y, 5, batch)
    assert np.array_equal(g.reshape(batch, 5), y[:, :5]) and np.array_equal(u.reshape(batch, 5), y[:, 5:])


# ---------- dequant ----------

@pytest.mark.parametrize("name", CASES)
def test_dequant_matches_fixture(name):
    d = load(name)
    k, n = int(d["k"]), int(d["n"])
    assert np.array_equal(O.dequant_f32(d["packed"], d["scales"], k, n), d["dequant_f32"])
    assert np.array_equal(O.dequant_f16(d["packed"], d["scales"], k, n), d["dequant_f16"])


def test_dequant_f16_exhaustive_scale_times_nibble():
    # all 65536 scale bit patterns x 16 nibbles, against numpy float32*int -> float16 (RNE)
    s_bits = np.arange(65536, dtype=np.uint16)
    n = 65536
    packed = np.zeros((1, n, 16), np.uint8)
    for i in range(16):
        packed[0, :, i // 2] |= np.uint8(i << (4 * (i & 1)))       # nibble value i at k=i
    got = O.dequant_f16(packed.reshape(-1), s_bits, 32, n)[:16]    # [16, n]
    s32 = s_bits.view(np.float16).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = (s32[None, :] * (np.arange(16, dtype=np.float32)[:, None] - 8)).astype(np.float16)
    wb = want.view(np.uint16)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan], wb[~nan])
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x3FF) != 0)


def test_dequant_q4_0_reference_generator():
    # reference test dequant_q4_to_f16_correctness (quantize.rs:3607-3668): K=128, N=64,
    # w[i] = ((17i+3)%101)*0.02-1; FP16 output within 1e-2 of scale*q and of the f32 weights' grid
    d = load("lcg_k128_n64_m4")
    k, n = 128, 64
    q4 = O.quantize_weights_q4_0_kn(d["w_kn"], k, n)
    out = O.dequant_q4_0_to_f16(q4, k, n).view(np.float16).astype(np.float32)
    blocks = q4.reshape(n, k // 32, 20)
    scale = blocks[:, :, :4].copy().view(np.float32)[:, :, 0]       # [N, G]
    nib = blocks[:, :, 4:]
    q = np.empty((n, k // 32, 32), np.int32)
    q[:, :, 0::2] = nib & 0xF
    q[:, :, 1::2] = nib >> 4
    want = (scale[:, :, None] * (q - 8)).reshape(n, k).T
    assert np.abs(out - want).max() < 0.01                          # the reference's tolerance
    assert np.array_equal(out, want.astype(np.float16).astype(np.float32))   # and in fact RNE-exact


# ---------- GEMV / GEMM ----------

def test_cpu_gemm_known_answer():
    # gemm.rs:185-190
    a = np.array([1, 2, 3, 4, 5, 6, 7, 8], np.float32)
    b = np.array([1, 2, 3, 4, 5, 6], np.float32)
    c = O.cpu_gemm(a, b, 4, 3, 2)
    assert c.reshape(-1).tolist() == [9, 12, 15, 19, 26, 33, 29, 40, 51, 39, 54, 69]


@pytest.mark.parametrize("name", CASES)
def test_gemv_matches_fixture_f64(name):
    d = load(name)
    k, n, m = int(d["k"]), int(d["n"]), int(d["m"])
    a = d["a_f16"].view(np.float16).astype(np.float32)
    c64 = d["c_f64"]
    denom = np.maximum(np.abs(c64), 1e-3 * np.abs(c64).max())
    assert np.abs(O.gemm_f64(a, d["packed"], d["scales"], m, k, n) - c64).max() < 1e-9 * np.abs(c64).max()
    for c in (O.gemv_ref_order(a, d["packed"], d["scales"], m, k, n, 1),
              O.gemv_ref_order(a, d["packed"], d["scales"], m, k, n, 3),
              O.gemm_tile_order(a, d["packed"], d["scales"], m, k, n),
              O.linear_dense(a, d["packed"], d["scales"], m, k, n),
              O.gemv_ref_order_mt(a, d["packed"], d["scales"], m, k, n)[0]):
        assert (np.abs(c - c64) / denom).max() < 1e-4


def test_gemv_closed_forms():
    rng = np.random.default_rng(23)
    k, n = 128, 24
    scales = (np.abs(rng.standard_normal((k // 32) * n)) * 0.02).astype(np.float16).view(np.uint16)
    a = rng.standard_normal((1, k)).astype(np.float16).astype(np.float32)
    # all nibbles 8 -> every weight is exactly 0 -> C == 0
    c = O.gemv_ref_order(a, np.full((k // 32) * n * 16, 0x88, np.uint8), scales, 1, k, n)
    assert np.all(c == 0)
    # scale 1, nibble 9 -> every weight is exactly 1 -> C[n] = sum(A), in the kernel's order
    one = np.full((k // 32) * n, np.float16(1.0).view(np.uint16), np.uint16)
    c = O.gemv_ref_order(a, np.full((k // 32) * n * 16, 0x99, np.uint8), one, 1, k, n)
    assert np.allclose(c, a.astype(np.float64).sum(), rtol=0, atol=1e-4)
    # one-hot A picks out one dequantized row exactly
    packed = rng.integers(0, 256, (k // 32) * n * 16, dtype=np.uint8)
    deq = O.dequant_f32(packed, scales, k, n)
    for kk in (0, 1, 31, 32, 77, 127):
        e = np.zeros((1, k), np.float32)
        e[0, kk] = 1.0
        assert np.array_equal(O.gemv_ref_order(e, packed, scales, 1, k, n)[0], deq[kk])
        assert np.array_equal(O.gemm_tile_order(e, packed, scales, 1, k, n)[0], deq[kk])


def test_fused_gemv_equals_concat_of_gemvs_bitwise():
    rng = np.random.default_rng(29)
    k, ns = 96, [16, 8, 8]
    mats = [(rng.integers(0, 256, (k // 32) * ni * 16, dtype=np.uint8),
             (np.abs(rng.standard_normal((k // 32) * ni)) * 0.02).astype(np.float16).view(np.uint16))
            for ni in ns]
    a = rng.standard_normal((1, k)).astype(np.float32)
    fp, fs = O.fuse_tw_marlin_n(mats, k, ns)
    fused = O.gemv_ref_order(a, fp, fs, 1, k, sum(ns))
    parts = np.hstack([O.gemv_ref_order(a, m[0], m[1], 1, k, ni) for m, ni in zip(mats, ns)])
    assert np.array_equal(fused, parts)


# ---------- split-K heuristic ----------

KNOWN_SPLITS = [  # (K, N) -> (n_blocks, splits, groups per split); quantize.rs:1317-1325 worked by hand
    ((4096, 4096), (16, 16, 8)),
    ((896, 1152), (5, 1, 28)), ((896, 896), (4, 1, 28)), ((896, 9728), (38, 1, 28)),
    ((4864, 896), (4, 19, 8)),
    ((3584, 4608), (18, 14, 8)), ((3584, 3584), (14, 14, 8)), ((3584, 37888), (148, 1, 112)),
    ((18944, 3584), (14, 19, 32)),
    ((4096, 11008), (43, 6, 22)), ((11008, 4096), (16, 16, 22)),
]


@pytest.mark.parametrize("shape,want", KNOWN_SPLITS)
def test_pick_splits_known_answers(shape, want):
    assert O.pick_splits(*shape) == want


def test_synthetic_generators_are_deterministic_and_shaped():
    p = O.synth_packed(128, 64, 7)
    assert np.array_equal(p, O.synth_packed(128, 64, 7)) and not np.array_equal(p, O.synth_packed(128, 64, 8))
    nib = np.concatenate([p & 0xF, p >> 4])
    assert nib.min() == 0 and nib.max() == 15
    s = O.synth_scales(4096, 64, 3).view(np.float16).astype(np.float32)
    assert s.min() >= 0 and abs(s.mean() - 0.02 * np.sqrt(2 / np.pi)) < 1e-3
    a = O.synth_act_f16(4, 4096, 5).view(np.float16).astype(np.float32)
    assert abs(a.mean()) < 0.03 and abs(a.std() - 1) < 0.03


def test_argmax_follows_the_reference_scan():
    # warp_argmax (missing_ops.rs:24-39): first index of the maximum; only values > -1e30 compete; NaN never wins.
    # Pinned against numpy where the two definitions coincide and by hand where they do not.
    rng = np.random.default_rng(5)
    x = rng.standard_normal((7, 1000)).astype(np.float32)
    assert np.array_equal(O.argmax(x, 7, 1000), np.argmax(x, axis=1).astype(np.int32))
    ties = np.zeros((1, 9), np.float32)
    ties[0, [3, 5, 8]] = 2.5
    assert O.argmax(ties, 1, 9)[0] == 3                                   # first of equal maxima
    low = np.full((1, 5), -2e30, np.float32)
    assert O.argmax(low, 1, 5)[0] == 0                                    # nothing above the starting value
    low[0, 4] = -1e30
    assert O.argmax(low, 1, 5)[0] == 0                                    # equal to it does not count either
    low[0, 2] = np.float32(-9.9e29)
    assert O.argmax(low, 1, 5)[0] == 2
    nan = np.array([[np.nan, 1.0, np.nan, 3.0, np.nan]], np.float32)
    assert O.argmax(nan, 1, 5)[0] == 3                                    # comparisons with NaN are false
    assert O.argmax(np.full((1, 4), np.nan, np.float32), 1, 4)[0] == 0
    assert O.argmax(np.zeros((2, 0), np.float32), 2, 0).tolist() == [0, 0]  # empty rows
    inf = np.array([[1.0, np.inf, np.inf, -np.inf]], np.float32)
    assert O.argmax(inf, 1, 4)[0] == 1


def test_silu_mul_against_f64_and_its_invariants():
    # warp_fused_silu_mul (ops.rs:966-976): g / (1 + expf(-g)) * up.  Checked against the same expression in
    # f64 (a few f32 ulps), the identity silu(g) - silu(-g) = g, and the limits at 0 and at both tails.
    g = (O.synth_normal_f32(5000, 910) * np.float32(4.0)).astype(np.float32)
    u = O.synth_normal_f32(5000, 911)
    out = O.silu_mul(g, u)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    truth = g64 / (1.0 + np.exp(-g64)) * u64
    assert np.max(np.abs(out - truth) / np.maximum(np.abs(truth), 1e-30)) < 1e-6
    ones = np.ones_like(g)
    assert np.allclose(O.silu_mul(g, ones).astype(np.float64) - O.silu_mul(-g, ones), g64, rtol=0, atol=2e-6)
    edge = np.array([0.0, -0.0, 100.0, -100.0, 1e4, -1e4, 1.0], np.float32)
    r = O.silu_mul(edge, np.full(7, 2.0, np.float32))
    assert r[0] == 0.0 and r[1] == 0.0
    assert r[2] == 200.0 and r[4] == 2e4                 # exp(-g) vanishes: silu(g) = g
    assert abs(r[3]) < 1e-40 and r[5] == 0.0             # exp(-g) overflows to inf: g / inf = -0
    assert abs(r[6] - 2.0 / (1.0 + np.exp(-1.0))) < 1e-6
    assert O.silu_mul(np.zeros(0, np.float32), np.zeros(0, np.float32)).size == 0


def test_pair_gate_up_is_the_32_column_interleave():
    # independent restatement with reshapes: [G][ffn/32][32] blocks of gate and up stacked side by side
    k, ffn = 96, 160
    gp, gs = O.synth_packed(k, ffn, 920), O.synth_scales(k, ffn, 921)
    up, us = O.synth_packed(k, ffn, 922), O.synth_scales(k, ffn, 923)
    pp, ps = O.pair_gate_up(gp, gs, up, us, k, ffn)
    G = k // 32
    want_p = np.stack([gp.reshape(G, ffn // 32, 32, 16), up.reshape(G, ffn // 32, 32, 16)], axis=2).reshape(-1)
    want_s = np.stack([gs.reshape(G, ffn // 32, 32), us.reshape(G, ffn // 32, 32)], axis=2).reshape(-1)
    assert np.array_equal(pp, want_p) and np.array_equal(ps, want_s)
    # the weights are those of fuse_tw_marlin_n([gate, up]) with the columns permuted
    fp, fs = O.fuse_tw_marlin_n([(gp, gs), (up, us)], k, [ffn, ffn])
    wf = O.dequant_f32(fp, fs, k, 2 * ffn)
    wp = O.dequant_f32(pp, ps, k, 2 * ffn)
    j = np.arange(ffn)
    col = (j // 32) * 64 + j % 32
    assert np.array_equal(wp[:, col], wf[:, :ffn]) and np.array_equal(wp[:, col + 32], wf[:, ffn:])


def test_gelu_mul_against_f64_and_its_limits():
    # batched_marlin_split_geglu / warp_fused_gelu_mul: 0.5 g (1 + tanh(0.7978845608 (g + 0.044715 g^3))) * up.
    # Against the same expression in f64 (the 1 + tanh cancellation for negative g turns one ulp of tanhf into
    # an absolute error of about 2^-24 |g u|), the identity gelu(g) - gelu(-g) = g, and both tails.
    g = (O.synth_normal_f32(5000, 1010) * np.float32(3.0)).astype(np.float32)
    u = O.synth_normal_f32(5000, 1011)
    out = O.gelu_mul(g, u)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    truth = 0.5 * g64 * (1.0 + np.tanh(np.float64(np.float32(0.7978845608)) * (g64 + np.float64(np.float32(0.044715)) * g64 ** 3))) * u64
    assert np.all(np.abs(out - truth) <= 4e-7 * np.abs(g64 * u64) + 1e-30)
    ones = np.ones_like(g)
    assert np.allclose(O.gelu_mul(g, ones).astype(np.float64) - O.gelu_mul(-g, ones), g64, rtol=0, atol=2e-6)
    edge = np.array([0.0, 10.0, -10.0, 1.0], np.float32)
    r = O.gelu_mul(edge, np.full(4, 3.0, np.float32))
    assert r[0] == 0.0 and r[1] == 30.0 and r[2] == 0.0
    assert abs(r[3] - 3.0 * 0.8411919906082768) < 1e-6      # gelu_tanh(1) = 0.84119199...

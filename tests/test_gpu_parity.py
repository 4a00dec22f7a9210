"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle and
the committed golden fixtures.

Bars: bit-exact for byte/integer work (quantizer output, reorder, fuse, repack, Q4 unpack
to FP16, splits); max relative error <= 1e-2 for GEMV/GEMM outputs (f32 accumulation), where
    rel = max_i |c_i - t_i| / max(|t_i|, 1e-3 * max_j |t_j|)
and t is the oracle's f64 dequant-then-matmul.  The floor keeps near-cancelling outputs from
turning an absolute error of a few ulps into a huge ratio.  Observed errors are ~1e-6, so the
tests also assert a much tighter 2e-4.
"""
import os

import numpy as np
import pytest

import tensorwarp_amd as T
from oracle import twm_oracle as O

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
TOL = 1e-2         # the stated tolerance
TIGHT = 2e-4       # what f32 accumulation actually delivers


@pytest.fixture(scope="module")
def dev():
    d = T.WarpDevice(0)
    print("device:", d.summary(), flush=True)
    yield d
    d.close()


def rel_err(c, truth):
    truth = np.asarray(truth, np.float64)
    denom = np.maximum(np.abs(truth), 1e-3 * np.abs(truth).max() + 1e-30)
    return float((np.abs(np.asarray(c, np.float64) - truth) / denom).max())


def synth(k, n, m, seed):
    packed = O.synth_packed(k, n, seed * 3 + 1)
    scales = O.synth_scales(k, n, seed * 3 + 2)
    a16 = O.synth_act_f16(m, k, seed * 3 + 3)
    return packed, scales, a16


def f16_as_f32(bits):
    return bits.view(np.float16).astype(np.float32)


EXACT_MAX_M = 32   # the decode kernels (M <= 32) use exact weights; the prefill GEMM above that the FP16 Q4 unpack


def gemm_truth(a16, packed, scales, m, k, n, rounded=False):
    """f64 dequant-then-matmul the library's default path is held to: exact weights f32(scale)*(q-8) up to
    M = 32 (every decode kernel); above that, or with rounded=True, the FP16 Q4 unpack f16(scale*(q-8)) of the
    prefill GEMM, which is the reference's dequant-then-FP16-GEMM route (quantize.rs:534-571)."""
    a = f16_as_f32(a16).reshape(m, k)
    if m <= EXACT_MAX_M and not rounded:
        return O.gemm_f64(a, packed, scales, m, k, n)
    w16 = O.dequant_f16(packed, scales, k, n).view(np.float16).astype(np.float64).reshape(k, n)
    return a.astype(np.float64) @ w16


# ---------------------------------------------------------------- format operations

def test_quantize_reorder_fuse_bit_exact(dev):
    k, n = 256, 200
    w_kn = O.synth_normal_f32(k * n, 41).reshape(k, n) * np.float32(0.05)
    w_kn[32:64, 7] = 0.0                       # an all-zero group
    w_kn[0, 3] = 0.35                          # make some exact .5 ties likely irrelevant but harmless
    wd = T.GpuTensor.from_host(dev, w_kn)
    q4 = T.quantize_weights_q4_0(dev, wd, k, n)
    assert np.array_equal(q4.to_host(), O.quantize_weights_q4_0_kn(w_kn, k, n))
    packed, scales = T.reorder_to_tw_marlin(dev, q4, k, n)
    op, os_ = O.reorder_to_tw_marlin(O.quantize_weights_q4_0_kn(w_kn, k, n), k, n)
    assert np.array_equal(packed.to_host(), op) and np.array_equal(scales.to_host(), os_)
    # one-pass quantizer from [K,N] and from [N,K]
    p2, s2 = T.quantize_f32_to_tw_marlin(dev, wd, k, n)
    assert np.array_equal(p2.to_host(), op) and np.array_equal(s2.to_host(), os_)
    wnk = T.GpuTensor.from_host(dev, np.ascontiguousarray(w_kn.T))
    p3, s3 = T.quantize_f32_to_tw_marlin(dev, wnk, k, n, weights_are_nk=True)
    rp, rs = O.quantize_tw_marlin_nk(np.ascontiguousarray(w_kn.T), k, n)
    assert np.array_equal(p3.to_host(), rp) and np.array_equal(s3.to_host(), rs)


def test_quantizer_ties_round_half_away(dev):
    v = np.zeros((1, 32), np.float32)
    v[0, :8] = [7.0, -7.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5]
    p, s = T.quantize_f32_to_tw_marlin(dev, T.GpuTensor.from_host(dev, v), 32, 1, weights_are_nk=True)
    rp, rs = O.quantize_tw_marlin_nk(v, 32, 1)
    assert np.array_equal(p.to_host(), rp) and np.array_equal(s.to_host(), rs)


def test_lcg_fixture_quantizes_to_golden_bytes(dev):
    d = np.load(os.path.join(GOLD, "lcg_k128_n64_m4.npz"))
    k, n = 128, 64
    p, s = T.quantize_f32_to_tw_marlin(dev, T.GpuTensor.from_host(dev, d["w_kn"]), k, n)
    assert np.array_equal(p.to_host(), d["packed"]) and np.array_equal(s.to_host(), d["scales"])


def test_fuse_matches_oracle(dev):
    k, ns = 96, [48, 16, 16]
    mats_h = [(O.synth_packed(k, ni, 50 + i), O.synth_scales(k, ni, 60 + i)) for i, ni in enumerate(ns)]
    mats_d = [(T.GpuTensor.from_host(dev, p), T.GpuTensor.from_host(dev, s, "f16")) for p, s in mats_h]
    fp, fs = T.fuse_tw_marlin_n(dev, mats_d, k, ns)
    op, os_ = O.fuse_tw_marlin_n(mats_h, k, ns)
    assert np.array_equal(fp.to_host(), op) and np.array_equal(fs.to_host(), os_)


def test_split_kernels(dev):
    h, kv, batch = 96, 32, 3
    x = O.synth_normal_f32(batch * (h + 2 * kv), 70)
    q, kk, v = (T.GpuTensor.zeros(dev, (batch * h,), "f32"), T.GpuTensor.zeros(dev, (batch * kv,), "f32"),
                T.GpuTensor.zeros(dev, (batch * kv,), "f32"))
    T.split_qkv(dev, T.GpuTensor.from_host(dev, x), q, kk, v, h, kv, batch)
    oq, ok_, ov = O.split_qkv(x, h, kv, batch)
    assert np.array_equal(q.to_host(), oq) and np.array_equal(kk.to_host(), ok_) and np.array_equal(v.to_host(), ov)
    ffn = 80
    y = O.synth_normal_f32(batch * 2 * ffn, 71)
    g, u = T.GpuTensor.zeros(dev, (batch * ffn,), "f32"), T.GpuTensor.zeros(dev, (batch * ffn,), "f32")
    T.split_gate_up(dev, T.GpuTensor.from_host(dev, y), g, u, ffn, batch)
    og, ou = O.split_gate_up(y, ffn, batch)
    assert np.array_equal(g.to_host(), og) and np.array_equal(u.to_host(), ou)


def silu_close(got, want):
    """f32 results of g / (1 + expf(-g)) * u from two correctly working libm's differ by a few ulps at most."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return bool(np.all(np.abs(got - want) <= 2e-6 * np.abs(want) + 1e-37))


def test_silu_mul_and_swiglu_rows(dev):
    batch, ffn = 3, 160
    gu = (O.synth_normal_f32(batch * 2 * ffn, 930) * np.float32(3.0)).reshape(batch, 2 * ffn)
    gu[0, :6] = [0.0, -0.0, 90.0, -90.0, 1e4, -1e4]
    g, u = np.ascontiguousarray(gu[:, :ffn]), np.ascontiguousarray(gu[:, ffn:])
    want = O.silu_mul(g, u)
    gd, ud = T.GpuTensor.from_host(dev, g), T.GpuTensor.from_host(dev, u)
    out = T.GpuTensor.zeros(dev, (batch, ffn), "f32")
    T.fused_silu_mul(dev, gd, ud, out)
    assert silu_close(out.to_host(), want)
    first = out.to_host().copy()
    # split + gate in one pass, on the reference's [gate | up] order: the same bits as the two-step route
    out2 = T.GpuTensor.zeros(dev, (batch, ffn), "f32")
    T.swiglu_rows(dev, T.GpuTensor.from_host(dev, gu), out2, ffn, batch)
    assert np.array_equal(out2.to_host(), first)
    # and on the paired order
    j = np.arange(ffn)
    col = (j // 32) * 64 + j % 32
    paired = np.zeros_like(gu)
    paired[:, col] = g
    paired[:, col + 32] = u
    out3 = T.GpuTensor.zeros(dev, (batch, ffn), "f32")
    T.swiglu_rows(dev, T.GpuTensor.from_host(dev, paired), out3, ffn, batch, paired=True)
    assert np.array_equal(out3.to_host(), first)
    with pytest.raises(T.DeviceError):
        T.swiglu_rows(dev, T.GpuTensor.from_host(dev, paired), out3, 40, 1, paired=True)


def test_pair_gate_up_bit_exact(dev):
    k, ffn = 128, 224
    gp, gs = O.synth_packed(k, ffn, 940), O.synth_scales(k, ffn, 941)
    up, us = O.synth_packed(k, ffn, 942), O.synth_scales(k, ffn, 943)
    gd = (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16"))
    ud = (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16"))
    pp, ps = T.pair_gate_up(dev, gd, ud, k, ffn)
    op, os_ = O.pair_gate_up(gp, gs, up, us, k, ffn)
    assert np.array_equal(pp.to_host(), op) and np.array_equal(ps.to_host(), os_)
    with pytest.raises(T.DeviceError):
        T.pair_gate_up(dev, gd, ud, k, 48)   # not a multiple of 32


@pytest.mark.parametrize("h,ffn,m,splits", [(896, 4864, 1, 0), (896, 4864, 3, 0), (3584, 18944, 1, 0),
                                            (3584, 18944, 4, 0), (2048, 96, 1, 0), (2048, 96, 2, 4),
                                            (256, 32, 1, 1), (1184, 160, 4, 3)])
def test_gemm_swiglu_fused_epilogue(dev, h, ffn, m, splits):
    # gemm_tw_marlin_m1 + split_gate_up + fused_silu_mul (generate.rs:2195-2203) against the single launch
    gp, gs = O.synth_packed(h, ffn, 950), O.synth_scales(h, ffn, 951)
    up, us = O.synth_packed(h, ffn, 952), O.synth_scales(h, ffn, 953)
    gd = (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16"))
    ud = (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16"))
    a16 = O.synth_act_f16(m, h, 954)
    ad = T.GpuTensor.from_host(dev, a16, "f16")
    # the reference's sequence on the [gate | up] weight
    fp, fs = T.fuse_tw_marlin_n(dev, [gd, ud], h, [ffn, ffn])
    plain = T.MarlinWeight.from_device(dev, fp, fs, h, 2 * ffn)
    gate_up = T.GpuTensor.zeros(dev, (m, 2 * ffn), "f32")
    T.gemm(dev, plain, ad, m, gate_up, splits)
    g, u = T.GpuTensor.zeros(dev, (m, ffn), "f32"), T.GpuTensor.zeros(dev, (m, ffn), "f32")
    T.split_gate_up(dev, gate_up, g, u, ffn, m)
    seq = T.GpuTensor.zeros(dev, (m, ffn), "f32")
    T.fused_silu_mul(dev, g, u, seq)
    # one launch on the paired weight
    w = T.MarlinWeight.gate_up(dev, gd, ud, h, ffn)
    assert w.paired and not plain.paired
    out = T.GpuTensor.from_host(dev, np.full((m, ffn), np.nan, np.float32))
    T.gemm_swiglu(dev, w, ad, m, out, splits)
    # the same columns, unfused, on the paired handle and on the [gate | up] handle
    tmp = T.GpuTensor.zeros(dev, (m, 2 * ffn), "f32")
    T.gemm(dev, w, ad, m, tmp, splits)
    seq_p = T.GpuTensor.zeros(dev, (m, ffn), "f32")
    T.swiglu_rows(dev, tmp, seq_p, ffn, m, paired=True)
    # (bit for bit under one plan, see test_sub_tile_gated_store; the planner may give the gated launch wider
    # sub-tiles than the plain one, which changes the order of the f32 sum)
    assert rel_err(out.to_host(), seq_p.to_host()) < 1e-4
    assert rel_err(out.to_host(), seq.to_host()) < 1e-4
    # against the oracle: f64 projections, then the reference's gate in f32 (its input differs from the
    # GPU's by the GEMV's rounding, so the bar is the GEMV's)
    a = f16_as_f32(a16).reshape(m, h)
    tg, tu = O.gemm_f64(a, gp, gs, m, h, ffn), O.gemm_f64(a, up, us, m, h, ffn)
    truth = tg / (1.0 + np.exp(-tg)) * tu
    assert rel_err(out.to_host(), truth) < TIGHT
    # f32 activations take the same path
    a32 = T.GpuTensor.from_host(dev, a)
    out32 = T.GpuTensor.zeros(dev, (m, ffn), "f32")
    T.gemm_swiglu(dev, w, a32, m, out32, splits)
    # (the plan depends on the activation type, and with it the order of the sum)
    assert rel_err(out32.to_host(), out.to_host()) < 1e-4
    with pytest.raises(T.DeviceError):
        T.gemm_swiglu(dev, plain, ad, m, out)        # not a paired weight
    w.free()
    plain.free()


@pytest.mark.parametrize("m,splits", [(8, 0), (8, 3), (24, 0), (32, 2), (40, 0), (40, 2), (150, 0)])
def test_gemm_swiglu_batched_and_prefill_rows(dev, m, splits):
    # the gated store of the batched-decode kernels (M = 5..32), of the prefill GEMM, and of the split-K sum
    h, ffn = 640, 224
    gp, gs = O.synth_packed(h, ffn, 960), O.synth_scales(h, ffn, 961)
    up, us = O.synth_packed(h, ffn, 962), O.synth_scales(h, ffn, 963)
    gd = (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16"))
    ud = (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16"))
    a16 = O.synth_act_f16(m, h, 964)
    ad = T.GpuTensor.from_host(dev, a16, "f16")
    w = T.MarlinWeight.gate_up(dev, gd, ud, h, ffn)
    out = T.GpuTensor.from_host(dev, np.full((m, ffn), np.nan, np.float32))
    T.gemm_swiglu(dev, w, ad, m, out, splits)
    # the plain GEMM on a paired handle returns the columns in the paired order; gating them afterwards gives the
    # same bits as the fused store
    tmp = T.GpuTensor.zeros(dev, (m, 2 * ffn), "f32")
    T.gemm(dev, w, ad, m, tmp, splits)
    seq = T.GpuTensor.zeros(dev, (m, ffn), "f32")
    T.swiglu_rows(dev, tmp, seq, ffn, m, paired=True)
    assert np.array_equal(out.to_host(), seq.to_host())
    fp, fs = O.fuse_tw_marlin_n([(gp, gs), (up, us)], h, [ffn, ffn])
    t = gemm_truth(a16, fp, fs, m, h, 2 * ffn)
    tg, tu = t[:, :ffn], t[:, ffn:]
    truth = tg / (1.0 + np.exp(-tg)) * tu
    bar = TIGHT if m <= EXACT_MAX_M else 1e-3
    assert rel_err(out.to_host(), truth) < bar
    j = np.arange(ffn)
    col = (j // 32) * 64 + j % 32
    got = tmp.to_host().reshape(m, 2 * ffn)
    assert rel_err(got[:, col], tg) < bar and rel_err(got[:, col + 32], tu) < bar
    w.free()


@pytest.mark.parametrize("m,splits", [(1, 0), (2, 3), (4, 0), (12, 2), (40, 0), (40, 2)])
def test_gemm_geglu_gate(dev, m, splits):
    # Gemma's gate (fused_gelu_mul, ops.rs:1157-1190) in the same stores
    h, ffn = 640, 224
    gp, gs = O.synth_packed(h, ffn, 1200), O.synth_scales(h, ffn, 1201)
    up, us = O.synth_packed(h, ffn, 1202), O.synth_scales(h, ffn, 1203)
    gd = (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16"))
    ud = (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16"))
    a16 = O.synth_act_f16(m, h, 1204)
    ad = T.GpuTensor.from_host(dev, a16, "f16")
    w = T.MarlinWeight.gate_up(dev, gd, ud, h, ffn)
    out = T.GpuTensor.from_host(dev, np.full((m, ffn), np.nan, np.float32))
    # (one row: the planner gives the gated launch 32-column sub-tiles and the plain one 16; bit equality is a property
    # of one plan, so both run the gated launch's here)
    if m == 1:
        dev.set_option("sub", 32)
    T.gemm_geglu(dev, w, ad, m, out, splits)
    tmp = T.GpuTensor.zeros(dev, (m, 2 * ffn), "f32")
    T.gemm(dev, w, ad, m, tmp, splits)
    dev.set_option("sub", 0)
    seq = T.GpuTensor.zeros(dev, (m, ffn), "f32")
    T.batched_marlin_split_geglu(dev, tmp, seq, ffn, m, paired=True)
    assert np.array_equal(out.to_host(), seq.to_host())
    fp, fs = O.fuse_tw_marlin_n([(gp, gs), (up, us)], h, [ffn, ffn])
    t = gemm_truth(a16, fp, fs, m, h, 2 * ffn)
    tg, tu = t[:, :ffn], t[:, ffn:]
    truth = 0.5 * tg * (1.0 + np.tanh(0.7978845608 * (tg + 0.044715 * tg ** 3))) * tu
    assert rel_err(out.to_host(), truth) < (TIGHT if m <= EXACT_MAX_M else 1e-3)
    w.free()


def test_stream_objects_casts_and_error_kinds(dev):
    # stream objects (device.rs:230-265), the f32 <-> f16 casts (fp16.rs:133-166) bit-exact against numpy's IEEE
    # conversion, and the DeviceError variant of a failure (device.rs:278-292)
    lib = T._lib.load()
    s = lib.twm_stream_create(dev.handle)
    assert s
    own = lib.twm_ctx_stream(dev.handle)
    assert lib.twm_ctx_set_stream(dev.handle, s) == T._lib.OK
    assert lib.twm_stream_destroy(dev.handle, s) == T._lib.UNSUPPORTED_OP      # still in use by the context
    x = (O.synth_normal_f32(70001, 77) * np.float32(300.0)).astype(np.float32)
    x[:6] = [0.0, -0.0, 65504.0, 65520.0, 1e-8, -6.0e-8]                      # edge of the range, ties, subnormals
    xd = T.GpuTensor.from_host(dev, x)
    hd = T.GpuTensor.zeros(dev, (x.size,), "f16")
    assert lib.twm_cast_f32_to_f16(dev.handle, xd.ptr, hd.ptr, x.size) == T._lib.OK
    assert lib.twm_stream_sync(dev.handle, s) == T._lib.OK
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    assert np.array_equal(hd.to_host().view(np.uint16), want.view(np.uint16))
    back = T.GpuTensor.zeros(dev, (x.size,), "f32")
    assert lib.twm_cast_f16_to_f32(dev.handle, hd.ptr, back.ptr, x.size) == T._lib.OK
    assert lib.twm_stream_sync(dev.handle, s) == T._lib.OK
    assert np.array_equal(back.to_host().view(np.uint32), want.astype(np.float32).view(np.uint32))
    assert lib.twm_ctx_set_stream(dev.handle, None) == T._lib.OK
    assert lib.twm_ctx_stream(dev.handle) == own
    assert lib.twm_stream_destroy(dev.handle, own) == T._lib.INVALID_HANDLE    # the context's own stream
    assert lib.twm_stream_destroy(dev.handle, s) == T._lib.OK
    # a shape error is no DeviceError variant; an allocation the device cannot serve is Memory
    assert lib.twm_gemm_tw_marlin_m1(dev.handle, xd.ptr, xd.ptr, xd.ptr, xd.ptr, 64, 100) == T._lib.SHAPE_ERROR
    assert lib.twm_last_error_kind() == 0
    assert lib.twm_malloc(dev.handle, 1 << 60) is None and lib.twm_last_error_kind() == 5
    for t in (xd, hd, back):
        t.free()


def test_debug_trace_belongs_to_its_context(dev):
    # a trace buffer set on one context does not reroute another context's launches
    lib = T._lib.load()
    k, n = 3584, 640
    packed, scales, a16 = synth(k, n, 1, 4242)
    with T.WarpDevice(0) as other:
        w_a = T.MarlinWeight.upload(dev, packed, scales, k, n)
        w_b = T.MarlinWeight.upload(other, packed, scales, k, n)
        trace = T.GpuTensor.zeros(dev, (4 * 4096,), "i32")
        assert lib.twm_debug_trace(dev.handle, trace.ptr, 4096) == T._lib.OK
        try:
            cb = T.GpuTensor.zeros(other, (n,), "f32")
            T.gemm(other, w_b, T.GpuTensor.from_host(other, a16, "f16"), 1, cb)
            other.synchronize()
            dev.synchronize()
            assert not trace.to_host().any()                   # the other context's launch left no trace
            ca = T.GpuTensor.zeros(dev, (n,), "f32")
            T.gemm(dev, w_a, T.GpuTensor.from_host(dev, a16, "f16"), 1, ca)
            dev.synchronize()
            assert trace.to_host().any()
            assert np.array_equal(ca.to_host(), cb.to_host())   # the traced twin computes the same bits
        finally:
            assert lib.twm_debug_trace(dev.handle, None, 0) == T._lib.OK
        w_a.free()
        w_b.free()


def test_argmax_bit_exact(dev):
    # index output: bit exact against the oracle's sequential scan, including ties (first wins), values at or
    # below the -1e30 starting value, NaN, infinities, a vocabulary-sized row and an empty one
    rng = np.random.default_rng(11)
    cases = [rng.standard_normal((5, 3000)).astype(np.float32),
             rng.standard_normal((1, 152064)).astype(np.float32),
             np.round(rng.standard_normal((8, 5000)) * 2).astype(np.float32),          # many ties
             np.full((2, 2048), -2e30, np.float32),
             np.array([[np.nan, 1.0, np.nan, 3.0, 3.0, np.nan]], np.float32),
             np.array([[1.0, np.inf, np.inf, -np.inf]], np.float32),
             np.full((1, 1500), np.nan, np.float32),
             np.round(rng.standard_normal((3, 70000)) * 3).astype(np.float32),         # two-phase form with ties across spans
             np.full((2, 40000), -2e30, np.float32),
             np.full((1, 33000), np.nan, np.float32)]
    cases[3][1, 1999] = np.float32(-9.9e29)
    cases[8][1, 39999] = np.float32(-9.9e29)
    for x in cases:
        rows, cols = x.shape
        out = T.GpuTensor.from_host(dev, np.full(rows, -7, np.int32))
        T.argmax(dev, T.GpuTensor.from_host(dev, x), out, rows, cols)
        assert np.array_equal(out.to_host(), O.argmax(x, rows, cols)), x.shape
    out = T.GpuTensor.from_host(dev, np.full(3, -7, np.int32))
    T.argmax(dev, T.GpuTensor.zeros(dev, (1,), "f32"), out, 3, 0)        # cols == 0: every row yields 0
    assert out.to_host().tolist() == [0, 0, 0]


# ---------------------------------------------------------------- Q4 unpack, bit exact

@pytest.mark.parametrize("name", ["lcg_k64_n8_m1", "lcg_k128_n64_m4", "synth_k128_n64_m1",
                                  "synth_k256_n80_m5", "synth_k160_n33_m17"])
def test_dequant_matches_golden_bits(dev, name):
    d = np.load(os.path.join(GOLD, name + ".npz"))
    k, n = int(d["k"]), int(d["n"])
    p = T.GpuTensor.from_host(dev, d["packed"])
    s = T.GpuTensor.from_host(dev, d["scales"], "f16")
    assert np.array_equal(T.dequant_to_f16(dev, p, s, k, n).to_host(), d["dequant_f16"])
    assert np.array_equal(T.dequant_to_f32(dev, p, s, k, n).to_host(), d["dequant_f32"])
    w = T.MarlinWeight.from_device(dev, p, s, k, n)            # and straight from both repacked copies
    try:
        for src in (0, 1):                                      # 0 = 16-column tile order, 1 = column-lane order
            dev.set_option("dequant_src", src)
            assert np.array_equal(w.dequant_f16().to_host(), d["dequant_f16"]), src
    finally:
        dev.set_option("dequant_src", 0)
    w.free()


def test_dequant_f16_exhaustive_scales_times_nibbles(dev):
    # all 65536 scale bit patterns x 16 nibble values; NaN payloads compare as NaN
    n = 65536
    s_bits = np.arange(n, dtype=np.uint16)
    packed = np.zeros((1, n, 16), np.uint8)
    for i in range(16):
        packed[0, :, i // 2] |= np.uint8(i << (4 * (i & 1)))
    want = O.dequant_f16(packed.reshape(-1), s_bits, 32, n)
    p = T.GpuTensor.from_host(dev, packed.reshape(-1))
    s = T.GpuTensor.from_host(dev, s_bits, "f16")
    for got in (T.dequant_to_f16(dev, p, s, 32, n).to_host(),
                T.MarlinWeight.from_device(dev, p, s, 32, n).dequant_f16().to_host()):
        wn = np.isnan(want.view(np.float16))
        assert np.array_equal(got[~wn], want[~wn])
        assert np.all(np.isnan(got.view(np.float16)[wn]))


def test_repack_is_lossless_at_7b_shape(dev):
    k, n = 3584, 4608
    packed, scales, _ = synth(k, n, 1, 5)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    want = O.dequant_f16(packed, scales, k, n)
    try:
        for src in (0, 1):
            dev.set_option("dequant_src", src)
            assert np.array_equal(w.dequant_f16().to_host(), want), src
    finally:
        dev.set_option("dequant_src", 0)
    w.free()


# ---------------------------------------------------------------- GEMV on the reference layout

# (the last two: 65 .. 255 column tiles on a K past one pass per wave -- 32-column sub-tiles with sixteen, then eight
# waves looping over their passes)
@pytest.mark.parametrize("k,n", [(64, 8), (128, 64), (896, 1152), (4096, 4096), (4864, 896), (3584, 300), (4608, 4200),
                                 (6144, 8300)])
def test_gemm_tw_marlin_m1_reference_layout(dev, k, n):
    packed, scales, a16 = synth(k, n, 1, k + n)
    a = f16_as_f32(a16)
    c = T.GpuTensor.zeros(dev, (n,), "f32")
    pd, sd = T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales, "f16")
    truth = O.gemm_f64(a, packed, scales, 1, k, n)[0]
    # default: the MFMA kernel on the reference's arrays as they are
    T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, a), pd, sd, c, n, k)
    assert rel_err(c.to_host(), truth) < TIGHT
    # activations that are not f16 numbers
    a_raw = (O.synth_normal_f32(k, k + n + 1) * np.float32(1.37)).astype(np.float32)
    T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, a_raw), pd, sd, c, n, k)
    t_raw = O.gemm_f64(a_raw.reshape(1, k), packed, scales, 1, k, n)[0]
    # two f16 terms per activation, about 22 bits (one term, plain rounding to f16, is off by up to 9e-2 on the
    # near-cancelling outputs of the larger shapes)
    assert rel_err(c.to_host(), t_raw) < TIGHT
    # "m1_exact": f32 activations, f32 FMAs in the reference kernel's order and its split-K rule
    try:
        dev.set_option("m1_exact", 1)
        c.copy_from_host(np.full(n, np.nan, np.float32))
        T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, a), pd, sd, c, n, k)
        got = c.to_host()
        assert rel_err(got, truth) < TIGHT
        _, splits, _ = T.pick_splits_reference(k, n)
        if splits == 1:                                      # same order as the reference kernel: bitwise
            assert np.array_equal(got, O.gemv_ref_order(a, packed, scales, 1, k, n, 1)[0])
        T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, a_raw), pd, sd, c, n, k)
        assert rel_err(c.to_host(), t_raw) < TIGHT
    finally:
        dev.set_option("m1_exact", 0)


@pytest.mark.parametrize("k,n", [(3584, 608), (896, 1152), (18944, 192), (1184, 200)])
def test_f32_activations_beyond_the_f16_range(dev, k, n):
    # The reference's GEMV takes any f32 row (quantize.rs:1188, 1219-1238).  Here the activations reach the MFMA as f16
    # terms; a wave whose chunk holds a value past the f16 range scales the chunk by a power of two first.  Rows whose
    # entries reach 1e6, a single huge entry among ordinary ones, and the largest finite f32 magnitudes that keep the
    # f32 result finite: the drop-in entry on both its kernels (K up to 4096 and beyond) and twm_gemm at M <= 4.
    packed, scales, _ = synth(k, n, 1, 8800 + k)
    pd, sd = T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales, "f16")
    base = O.synth_normal_f32(4 * k, 8900 + k).reshape(4, k)
    rows = base.copy()
    rows[0] *= np.float32(2.5e5)                       # |a| up to about 1e6 everywhere
    rows[1, 5::97] *= np.float32(3.0e5)                # a few huge entries among ordinary ones
    rows[2] *= np.float32(1.0e30)                      # far beyond: sums near 1e33 still fit f32
    rows[3, k // 2] = np.float32(70000.0)              # just past the largest f16
    c = T.GpuTensor.zeros(dev, (n,), "f32")
    for r in range(4):
        a = np.ascontiguousarray(rows[r])
        truth = O.gemm_f64(a.reshape(1, k), packed, scales, 1, k, n)[0]
        T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, a), pd, sd, c, n, k)
        got = c.to_host()
        assert np.isfinite(got).all(), r
        assert rel_err(got, truth) < TIGHT, r
    w = T.MarlinWeight.from_device(dev, pd, sd, k, n)
    for m in (1, 2, 4):
        truth = O.gemm_f64(rows[:m], packed, scales, m, k, n)
        cm = T.GpuTensor.zeros(dev, (m, n), "f32")
        T.gemm(dev, w, T.GpuTensor.from_host(dev, np.ascontiguousarray(rows[:m])), m, cm)
        for r in range(m):   # (row by row: the rows differ by 30 orders of magnitude)
            assert rel_err(cm.to_host()[r], truth[r]) < TIGHT, (m, r)
    # in range nothing changes: the same bits as before the guard, i.e. as with the values given as exact f16 pairs
    a_in = np.ascontiguousarray(base[0])
    T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, a_in), pd, sd, c, n, k)
    first = c.to_host()
    a_in[7] = np.float32(64999.0)
    T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, a_in), pd, sd, c, n, k)
    assert rel_err(c.to_host(), O.gemm_f64(a_in.reshape(1, k), packed, scales, 1, k, n)[0]) < TIGHT
    assert np.isfinite(first).all()
    w.free()


@pytest.mark.parametrize("k,n", [(3584, 608), (1184, 200)])
def test_f32_rows_of_any_size_from_five_rows_on(dev, k, n):
    # The reference's only quantized GEMM for M > 1 takes `const float *A` and multiplies in f32 (quantize.rs:186-246,
    # 1825-1858), so any finite f32 row is a valid input.  From five rows on the activations are converted once per
    # launch, a workgroup per row, with a power of two per row that keeps the row inside the f16 range (and a tiny row
    # out of the subnormals); the store multiplies the row's sums back.  Rows of 1e6, of 1e30, of 1e-6 and of 1e-30 next
    # to ordinary ones, a single huge entry among ordinary ones, at 8 and 32 rows (both batched-decode kernels, both
    # row-block heights) against the exact-weight f64 product; and at 64 rows (the prefill GEMM, which rounds the scaled
    # activations to one f16 term: values that are f16 numbers times a power of two, so that the rounding is exact)
    # against the f64 product on the FP16 Q4 unpack.  The gated store scales before the gate.
    packed, scales, _ = synth(k, n, 1, 9800 + k)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    factors = [2.5e5, 1.0, 1.0e30, 1.0e-6, 1.0, 1.0e-30, 3.0, 7.0e4]
    for m in (8, 32):
        rows = O.synth_normal_f32(m * k, 9900 + m).reshape(m, k).copy()
        for r in range(m):
            rows[r] *= np.float32(factors[r % len(factors)])
        rows[4, 5::97] *= np.float32(3.0e5)              # a few huge entries among ordinary ones
        truth = O.gemm_f64(rows, packed, scales, m, k, n)
        for splits in (0, 3):
            c = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))
            T.gemm(dev, w, T.GpuTensor.from_host(dev, np.ascontiguousarray(rows)), m, c, splits)
            got = c.to_host()
            assert np.isfinite(got).all(), (m, splits)
            for r in range(m):   # (row by row: the rows differ by sixty orders of magnitude)
                assert rel_err(got[r], truth[r]) < TIGHT, (m, splits, r)
    m = 64
    a16 = O.synth_act_f16(m, k, 9950)
    rows = f16_as_f32(a16).reshape(m, k).copy()
    pow2 = [2.0 ** 18, 1.0, 2.0 ** 100, 2.0 ** -20, 1.0, 2.0 ** -100, 2.0, 2.0 ** 17]
    for r in range(m):
        rows[r] *= np.float32(pow2[r % len(pow2)])
    w16 = O.dequant_f16(packed, scales, k, n).view(np.float16).astype(np.float64).reshape(k, n)
    truth = rows.astype(np.float64) @ w16
    for splits in (0, 2):
        c = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))
        T.gemm(dev, w, T.GpuTensor.from_host(dev, np.ascontiguousarray(rows)), m, c, splits)
        got = c.to_host()
        assert np.isfinite(got).all(), splits
        for r in range(m):   # (the prefill GEMM's bar: f32 sums over all of K inside the MFMAs)
            assert rel_err(got[r], truth[r]) < 1e-3, (splits, r)
    w.free()


@pytest.mark.parametrize("m", [8, 32, 64])
def test_f32_rows_of_any_size_through_the_gated_store(dev, m):
    h, ffn = 640, 224
    gp, gs = O.synth_packed(h, ffn, 1300), O.synth_scales(h, ffn, 1301)
    up, us = O.synth_packed(h, ffn, 1302), O.synth_scales(h, ffn, 1303)
    gd = (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16"))
    ud = (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16"))
    w = T.MarlinWeight.gate_up(dev, gd, ud, h, ffn)
    rows = f16_as_f32(O.synth_act_f16(m, h, 1304)).reshape(m, h).copy()
    for r in range(m):
        rows[r] *= np.float32([2.0 ** 17, 1.0, 2.0 ** -18, 2.0 ** 16][r % 4]) * np.float32(0.02)
    ad = T.GpuTensor.from_host(dev, np.ascontiguousarray(rows))
    for splits in (0, 2):
        out = T.GpuTensor.from_host(dev, np.full((m, ffn), np.nan, np.float32))
        T.gemm_swiglu(dev, w, ad, m, out, splits)
        tmp = T.GpuTensor.zeros(dev, (m, 2 * ffn), "f32")
        T.gemm(dev, w, ad, m, tmp, splits)
        seq = T.GpuTensor.zeros(dev, (m, ffn), "f32")
        T.swiglu_rows(dev, tmp, seq, ffn, m, paired=True)
        got, want = out.to_host(), seq.to_host()
        assert np.isfinite(got).all()
        # (the fused and the two-step launch may run different plans; each row against the other at the bar of one ulp of
        # exp, relative to the row's largest value)
        for r in range(m):
            assert np.abs(got[r] - want[r]).max() <= 1e-5 * np.abs(want[r]).max(), (m, splits, r)
    w.free()


@pytest.mark.parametrize("k,n", [(3584, 608), (18944, 192), (1184, 200)])
def test_f32_rows_of_tiny_magnitude(dev, k, n):
    # Rows whose values are all far below the f16 normal range (scaled by 1e-6, 1e-20): the residual term of the two-term
    # form would fall into the f16 subnormals and the result would keep a few bits; the kernels scale such a stretch up
    # by a power of two first.  The drop-in entry and twm_gemm at one to four rows.
    packed, scales, _ = synth(k, n, 1, 8700 + k)
    pd, sd = T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales, "f16")
    w = T.MarlinWeight.from_device(dev, pd, sd, k, n)
    base = O.synth_normal_f32(4 * k, 8750 + k).reshape(4, k)
    for scale in (1.0e-6, 1.0e-20):
        rows = np.ascontiguousarray(base * np.float32(scale))
        rows[3] = base[3]                                     # an ordinary row beside them
        rows[2, ::2] = base[2, ::2] * np.float32(1.0e-3)      # tiny and small values mixed
        truth = O.gemm_f64(rows, packed, scales, 4, k, n)
        c = T.GpuTensor.zeros(dev, (n,), "f32")
        for r in range(4):
            T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, np.ascontiguousarray(rows[r])), pd, sd, c, n, k)
            assert rel_err(c.to_host(), truth[r]) < TIGHT, (scale, r)
        for m in (1, 2, 4):
            cm = T.GpuTensor.zeros(dev, (m, n), "f32")
            T.gemm(dev, w, T.GpuTensor.from_host(dev, np.ascontiguousarray(rows[:m])), m, cm)
            for r in range(m):
                assert rel_err(cm.to_host()[r], truth[r]) < TIGHT, (scale, m, r)
    w.free()


def test_gemm_tw_marlin_m1_from_buffer_and_errors(dev):
    k, n = 128, 64
    packed, scales, a16 = synth(k, n, 1, 9)
    a = f16_as_f32(a16)
    slab_p = np.concatenate([np.zeros(4096, np.uint8), packed])
    slab_s = np.concatenate([np.zeros(100, np.uint16), scales])
    c = T.GpuTensor.zeros(dev, (n,), "f32")
    T.gemm_tw_marlin_m1_from_buffer(dev, T.GpuTensor.from_host(dev, a), T.GpuTensor.from_host(dev, slab_p), 4096,
                                    T.GpuTensor.from_host(dev, slab_s, "f16"), 100, c, n, k)
    assert rel_err(c.to_host(), O.gemm_f64(a, packed, scales, 1, k, n)[0]) < TIGHT
    try:
        dev.set_option("m1_exact", 1)
        T.gemm_tw_marlin_m1_from_buffer(dev, T.GpuTensor.from_host(dev, a), T.GpuTensor.from_host(dev, slab_p), 4096,
                                        T.GpuTensor.from_host(dev, slab_s, "f16"), 100, c, n, k)
    finally:
        dev.set_option("m1_exact", 0)
    assert np.array_equal(c.to_host(), O.gemv_ref_order(a, packed, scales, 1, k, n, 1)[0])
    # an offset that keeps only the 4-byte alignment the reference's own kernel needs (it reads a record as four
    # 32-bit words, quantize.rs:1227-1228), with and without the reference's split-K: the f32 kernel takes over
    for kk, nn in ((128, 64), (2048, 96)):
        pk, sc_, a16b = synth(kk, nn, 1, 10 + kk)
        ab = f16_as_f32(a16b)
        slab = np.concatenate([np.zeros(36, np.uint8), pk])
        cb = T.GpuTensor.from_host(dev, np.full(nn, np.nan, np.float32))
        T.gemm_tw_marlin_m1_from_buffer(dev, T.GpuTensor.from_host(dev, ab), T.GpuTensor.from_host(dev, slab), 36,
                                        T.GpuTensor.from_host(dev, sc_, "f16"), 0, cb, nn, kk)
        assert rel_err(cb.to_host(), O.gemm_f64(ab, pk, sc_, 1, kk, nn)[0]) < TIGHT
        dev.set_option("m1_align16", 1)                  # a caller can ask to be told instead of taking the slow kernel
        try:
            with pytest.raises(T.DeviceError) as e3:
                T.gemm_tw_marlin_m1_from_buffer(dev, T.GpuTensor.from_host(dev, ab), T.GpuTensor.from_host(dev, slab), 36,
                                                T.GpuTensor.from_host(dev, sc_, "f16"), 0, cb, nn, kk)
            assert e3.value.code == T._lib.SHAPE_ERROR and "16-byte" in str(e3.value)
        finally:
            dev.set_option("m1_align16", 0)
        with pytest.raises(T.DeviceError) as e2:         # not even 4-byte aligned: a fault in the reference
            T.gemm_tw_marlin_m1_from_buffer(dev, T.GpuTensor.from_host(dev, ab), T.GpuTensor.from_host(dev, slab), 35,
                                            T.GpuTensor.from_host(dev, sc_, "f16"), 0, cb, nn, kk)
        assert e2.value.code == T._lib.SHAPE_ERROR
    with pytest.raises(T.DeviceError) as e:              # the reference asserts k % 32 == 0 (quantize.rs:1311)
        T.gemm_tw_marlin_m1(dev, c, c, c, c, n, 100)
    assert e.value.code == T._lib.SHAPE_ERROR
    with pytest.raises(T.DeviceError):
        T.MarlinWeight.upload(dev, packed, scales, 100, n)


# ---------------------------------------------------------------- the repacked fast path

def run_gemm(dev, w, a16, m, n, splits=0, a_f32=False):
    a_dev = T.GpuTensor.from_host(dev, f16_as_f32(a16)) if a_f32 else T.GpuTensor.from_host(dev, a16, "f16")
    c = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))   # NaN canary: every output must be written
    T.gemm(dev, w, a_dev, m, c, splits)
    out = c.to_host()
    a_dev.free()
    c.free()
    return out


@pytest.mark.parametrize("name", ["lcg_k64_n8_m1", "lcg_k128_n64_m4", "synth_k128_n64_m1",
                                  "synth_k256_n80_m5", "synth_k160_n33_m17"])
def test_gemm_matches_golden(dev, name):
    d = np.load(os.path.join(GOLD, name + ".npz"))
    k, n, m = int(d["k"]), int(d["n"]), int(d["m"])
    w = T.MarlinWeight.upload(dev, d["packed"], d["scales"], k, n)
    for a_f32 in (False, True):
        got = run_gemm(dev, w, d["a_f16"], m, n, a_f32=a_f32)
        if m <= EXACT_MAX_M:
            assert rel_err(got, d["c_f64"]) < TIGHT, (name, a_f32)
            if m > 16:   # option: the 32-row batched-decode kernel on the FP16 Q4 unpack (the fixture's dequant_f16)
                w16 = d["dequant_f16"].view(np.float16).astype(np.float64).reshape(k, n)
                exact = f16_as_f32(d["a_f16"]).astype(np.float64).reshape(m, k) @ w16
                dev.set_option("batch_rounded", 1)
                try:
                    assert rel_err(run_gemm(dev, w, d["a_f16"], m, n, a_f32=a_f32), exact) < TIGHT, (name, a_f32)
                finally:
                    dev.set_option("batch_rounded", 0)
        else:
            # M > 32 runs the MFMAs on the FP16 Q4 unpack (the fixture's dequant_f16), like the reference's
            # dequant-then-matmul; against the f32-weight result the weight rounding (2^-12 each) shows
            w16 = d["dequant_f16"].view(np.float16).astype(np.float64).reshape(k, n)
            exact = f16_as_f32(d["a_f16"]).astype(np.float64).reshape(m, k) @ w16
            assert rel_err(got, exact) < TIGHT, (name, a_f32)
            assert np.abs(got - d["c_f64"]).max() / np.abs(d["c_f64"]).max() < 1e-3
    w.free()


@pytest.mark.parametrize("m", [1, 4, 64])
def test_reference_gemm_q4_0_correctness_case(dev, m):
    # The reference's own test of the quantized GEMM (gemm_q4_0_correctness, quantize.rs:3043-3106): its
    # generators for A and B, B quantized on the GPU, result against the full-precision product with
    # NRMSE < 0.15 (the quantization error of group-32 Q4) -- here also against the oracle on the quantized
    # weights at the library's own bar.  M = 64 is the reference's shape; 1 and 4 run the decode kernels.
    n, k = 64, 128
    a = (((np.arange(m * k) * 7 + 13) % 100).astype(np.float32) * np.float32(0.01) - np.float32(0.5)).reshape(m, k)
    b = (((np.arange(k * n) * 11 + 3) % 100).astype(np.float32) * np.float32(0.01) - np.float32(0.5)).reshape(k, n)
    packed, scales = T.quantize_f32_to_tw_marlin(dev, T.GpuTensor.from_host(dev, b), k, n)
    ph, sh = packed.to_host(), scales.to_host()
    w = T.MarlinWeight.from_device(dev, packed, scales, k, n)
    c = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))
    T.gemm(dev, w, T.GpuTensor.from_host(dev, a), m, c)
    got = c.to_host().reshape(m, n).astype(np.float64)
    full = a.astype(np.float64) @ b.astype(np.float64)
    nrmse = np.sqrt(((got - full) ** 2).sum() / max((full ** 2).sum(), 1e-10))
    assert nrmse < 0.15
    if m <= EXACT_MAX_M:
        assert rel_err(got, O.gemm_f64(a, ph, sh, m, k, n)) < TIGHT
    else:   # the prefill GEMM: f16 activations and the FP16 Q4 unpack
        w16 = O.dequant_f16(ph, sh, k, n).view(np.float16).astype(np.float64).reshape(k, n)
        assert rel_err(got, a.astype(np.float16).astype(np.float64) @ w16) < TIGHT
    if m == 1:
        c1 = T.GpuTensor.zeros(dev, (n,), "f32")
        T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, a), packed, scales, c1, n, k)
        assert rel_err(c1.to_host(), O.gemm_f64(a, ph, sh, 1, k, n)[0]) < TIGHT
    w.free()


def test_gemv_closed_forms(dev):
    k, n = 256, 96
    scales = O.synth_scales(k, n, 77)
    a16 = O.synth_act_f16(1, k, 78)
    w0 = T.MarlinWeight.upload(dev, np.full((k // 32) * n * 16, 0x88, np.uint8), scales, k, n)
    assert np.all(run_gemm(dev, w0, a16, 1, n) == 0)                 # all weights exactly zero
    one = np.full((k // 32) * n, np.float16(1.0).view(np.uint16), np.uint16)
    w1 = T.MarlinWeight.upload(dev, np.full((k // 32) * n * 16, 0x99, np.uint8), one, k, n)
    assert np.allclose(run_gemm(dev, w1, a16, 1, n), f16_as_f32(a16).astype(np.float64).sum(), atol=1e-3)
    packed = O.synth_packed(k, n, 79)
    w2 = T.MarlinWeight.upload(dev, packed, scales, k, n)
    deq = O.dequant_f32(packed, scales, k, n)
    for kk in (0, 1, 7, 8, 31, 32, 100, 255):                        # one-hot A picks a dequantised row, exactly
        e = np.zeros((1, k), np.float16)
        e[0, kk] = 1.0
        assert np.array_equal(run_gemm(dev, w2, e.view(np.uint16), 1, n)[0], deq[kk]), kk
    for w in (w0, w1, w2):
        w.free()


SHAPES_05B = [(896, 1152), (896, 896), (896, 9728), (4864, 896)]
SHAPES_7B = [(3584, 4608), (3584, 3584), (3584, 37888), (18944, 3584)]


@pytest.mark.parametrize("k,n", [(4096, 4096)] + SHAPES_05B + SHAPES_7B)
def test_gemv_m1_benchmark_shapes(dev, k, n):
    packed, scales, a16 = synth(k, n, 1, k * 7 + n)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    truth = O.gemm_f64(f16_as_f32(a16), packed, scales, 1, k, n)
    got = run_gemm(dev, w, a16, 1, n)
    err = rel_err(got, truth)
    print("M=1 %5d->%5d splits=%d rel_err=%.2e" % (k, n, T.pick_splits(k, n, 1), err), flush=True)
    assert err < TIGHT and err < TOL
    if k * n <= 3584 * 4608:
        # the other reading of "dequant-then-matmul": the product with the FP16 Q4 unpack, f16(scale * (q - 8)).
        # Its weights carry a rounding of 2^-12 each, which the decode kernels do not make; measured against the
        # largest output the two agree far inside the tolerance
        w16 = O.dequant_f16(packed, scales, k, n).view(np.float16).astype(np.float64).reshape(k, n)
        t16 = f16_as_f32(a16).astype(np.float64).reshape(1, k) @ w16
        assert np.abs(got - t16).max() / np.abs(t16).max() < 1e-3
    w.free()


@pytest.mark.parametrize("m", [2, 3, 4, 5, 8, 15, 16, 17, 31, 32])
def test_batched_decode_small_k(dev, m):
    k, n = 896, 1152
    packed, scales, a16 = synth(k, n, m, 1000 + m)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    truth = gemm_truth(a16, packed, scales, m, k, n)
    for splits in (0, 1, 3):
        assert rel_err(run_gemm(dev, w, a16, m, n, splits), truth) < TIGHT, splits
    w.free()


@pytest.mark.parametrize("m,k,n", [(4, 3584, 4608), (8, 3584, 37888), (16, 18944, 3584), (32, 3584, 4608)])
def test_batched_decode_7b_shapes(dev, m, k, n):
    packed, scales, a16 = synth(k, n, m, 2000 + m)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    truth = gemm_truth(a16, packed, scales, m, k, n)
    got = run_gemm(dev, w, a16, m, n)
    assert rel_err(got, truth) < TIGHT
    # every row of the batch agrees with the same row run alone (another kernel variant and
    # summation order, so agreement is to f32 rounding, not bitwise)
    alone = run_gemm(dev, w, a16[m - 1:m], 1, n)
    assert rel_err(alone[0], got[m - 1]) < TIGHT
    w.free()


def test_split_k_choice_does_not_change_the_result(dev):
    # the one-lane-per-column kernel on whole tiles, every tile width, many split factors
    k, n = 4096, 4096
    packed, scales, a16 = synth(k, n, 1, 31)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    truth = O.gemm_f64(f16_as_f32(a16), packed, scales, 1, k, n)
    try:
        for kernel in (2,):
            dev.set_option("kernel", kernel)
            for nt in (1, 2):
                dev.set_option("nt", nt)
                for splits in (1, 2, 5, 8, 32):
                    got = run_gemm(dev, w, a16, 1, n, splits)
                    assert rel_err(got, truth) < TIGHT, (kernel, nt, splits)
                # same launch twice is bitwise repeatable (ordered reduction, no float atomics)
                assert np.array_equal(run_gemm(dev, w, a16, 1, n, 8), run_gemm(dev, w, a16, 1, n, 8))
            if kernel == 2:
                dev.set_option("nt", 1)
                for waves in (1, 2, 4, 8, 16):
                    dev.set_option("waves", waves)
                    for splits in (1, 3, 32):
                        assert rel_err(run_gemm(dev, w, a16, 1, n, splits), truth) < TIGHT, (waves, splits)
                dev.set_option("waves", 0)
    finally:
        for key in ("kernel", "nt", "waves"):
            dev.set_option(key, 0)
    w.free()


def test_sub_tile_kernel_variants(dev):
    # the M <= 4 kernel on 16- and 32-column sub-tiles, forced through the options: every row count and activation
    # type, one pass per wave and the loop over passes, with and without a cross-workgroup split-K, on ragged N
    # and on a K that ends inside a 128-deep chunk
    try:
        for k, n in ((3584 + 32, 1000), (1184, 160), (256, 72)):
            packed, scales, a16 = synth(k, n, 16, 4100 + n)
            w = T.MarlinWeight.upload(dev, packed, scales, k, n)
            for m in (1, 2, 3, 4, 5, 8, 13, 16):       # from five rows on: f16 rows only, two to four row groups
                truth = gemm_truth(a16[:m], packed, scales, m, k, n)
                for sub in (16, 32):
                    dev.set_option("sub", sub)
                    for waves in (1, 4, 16):
                        dev.set_option("waves", waves)
                        for splits in (0, 3):
                            for a_f32 in ((False, True) if m <= 4 else (False,)):
                                got = run_gemm(dev, w, a16[:m], m, n, splits, a_f32)
                                assert rel_err(got, truth) < TIGHT, (k, n, m, sub, waves, splits, a_f32)
            w.free()
        # the drop-in entry point on the reference's arrays
        for k, n in ((3584 + 32, 1000), (1184, 160)):
            packed, scales, a16 = synth(k, n, 1, 4200 + n)
            a = f16_as_f32(a16).reshape(1, k) * np.float32(1.0 + 2.0 ** -13)    # not f16 values
            truth = O.gemm_f64(a, packed, scales, 1, k, n)
            pd, sd = T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales, "f16")
            ad = T.GpuTensor.from_host(dev, a)
            for sub in (0, 1, 16, 32):
                dev.set_option("sub", sub)
                for waves in (0, 1, 4, 16):
                    dev.set_option("waves", waves)
                    for sp in (0, 3):
                        dev.set_option("m1_splits", sp)
                        c = T.GpuTensor.from_host(dev, np.full((1, n), np.nan, np.float32))
                        T.gemm_tw_marlin_m1(dev, ad, pd, sd, c, n, k)
                        assert rel_err(c.to_host(), truth) < TIGHT, (k, n, sub, waves, sp)
    finally:
        for key in ("sub", "waves", "m1_splits"):
            dev.set_option(key, 0)


def test_sub_tile_gated_store(dev):
    # the gated store on sub-tiles: bit for bit the unfused columns of the same paired handle under the same plan
    h, ffn = 2304, 96
    gp, gs = O.synth_packed(h, ffn, 4300), O.synth_scales(h, ffn, 4301)
    up, us = O.synth_packed(h, ffn, 4302), O.synth_scales(h, ffn, 4303)
    gd = (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16"))
    ud = (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16"))
    w = T.MarlinWeight.gate_up(dev, gd, ud, h, ffn)
    try:
        for m in (1, 2, 4, 7, 16):
            a16 = O.synth_act_f16(m, h, 4304 + m)
            a = f16_as_f32(a16).reshape(m, h)
            tg, tu = O.gemm_f64(a, gp, gs, m, h, ffn), O.gemm_f64(a, up, us, m, h, ffn)
            for act, truth in ((T.ACT_SWIGLU, tg / (1.0 + np.exp(-tg)) * tu), (T.ACT_GEGLU, O.gelu_mul(tg.astype(np.float32), tu.astype(np.float32)))):
                for sub in (16, 32):
                    dev.set_option("sub", sub)
                    for waves, splits in ((4, 0), (16, 0), (4, 3)):
                        dev.set_option("waves", waves)
                        for a_f32 in ((False, True) if m <= 4 else (False,)):
                            ad = T.GpuTensor.from_host(dev, a) if a_f32 else T.GpuTensor.from_host(dev, a16, "f16")
                            out = T.GpuTensor.from_host(dev, np.full((m, ffn), np.nan, np.float32))
                            tmp = T.GpuTensor.zeros(dev, (m, 2 * ffn), "f32")
                            seq = T.GpuTensor.zeros(dev, (m, ffn), "f32")
                            if act == T.ACT_SWIGLU:
                                T.gemm_swiglu(dev, w, ad, m, out, splits)
                                T.gemm(dev, w, ad, m, tmp, splits)
                                T.swiglu_rows(dev, tmp, seq, ffn, m, paired=True)
                                assert np.array_equal(out.to_host(), seq.to_host()), (m, sub, waves, splits, a_f32)
                            else:
                                T.gemm_geglu(dev, w, ad, m, out, splits)
                            assert rel_err(out.to_host(), truth) < TIGHT, (m, act, sub, waves, splits, a_f32)
    finally:
        for key in ("sub", "waves"):
            dev.set_option(key, 0)
        w.free()


def test_five_to_eight_rows_on_wide_matrices(dev):
    # M = 5 .. 8 with f16 rows on more than 128 column tiles: the 64-column lane-per-column kernel with two row
    # groups (f32 rows and forced split factors keep the streaming kernel); both against the oracle
    k, n = 416, 9000
    packed, scales, a16 = synth(k, n, 8, 4500)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    try:
        for m in (5, 6, 7, 8):
            truth = gemm_truth(a16[:m], packed, scales, m, k, n)
            got = run_gemm(dev, w, a16[:m], m, n)
            assert rel_err(got, truth) < TIGHT, m
            dev.set_option("kernel", 3)
            streamed = run_gemm(dev, w, a16[:m], m, n)
            dev.set_option("kernel", 0)
            assert rel_err(streamed, truth) < TIGHT, m
            assert rel_err(got, streamed) < 1e-4, m
            assert rel_err(run_gemm(dev, w, a16[:m], m, n, a_f32=True), truth) < TIGHT, m
            for waves in (1, 16):
                dev.set_option("waves", waves)
                assert rel_err(run_gemm(dev, w, a16[:m], m, n), truth) < TIGHT, (m, waves)
            dev.set_option("waves", 0)
    finally:
        dev.set_option("kernel", 0)
        dev.set_option("waves", 0)
    w.free()
    # the gated store of the same kernel
    h, ffn = 288, 4608
    gp, gs = O.synth_packed(h, ffn, 4510), O.synth_scales(h, ffn, 4511)
    up, us = O.synth_packed(h, ffn, 4512), O.synth_scales(h, ffn, 4513)
    gd = (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16"))
    ud = (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16"))
    wp = T.MarlinWeight.gate_up(dev, gd, ud, h, ffn)
    for m in (5, 8):
        a16 = O.synth_act_f16(m, h, 4514 + m)
        a = f16_as_f32(a16).reshape(m, h)
        tg, tu = O.gemm_f64(a, gp, gs, m, h, ffn), O.gemm_f64(a, up, us, m, h, ffn)
        out = T.GpuTensor.from_host(dev, np.full((m, ffn), np.nan, np.float32))
        T.gemm_swiglu(dev, wp, T.GpuTensor.from_host(dev, a16, "f16"), m, out)
        assert rel_err(out.to_host(), tg / (1.0 + np.exp(-tg)) * tu) < TIGHT, m
    wp.free()


def test_lds_shared_batched_decode_kernel(dev):
    # option "kernel" = 4: one or two tiles per wave ("nt" 1 / 2), two or three column quads per workgroup on one
    # activation tile ("nt" 4 / 3), one / two / four k-slices per workgroup ("waves" 0 / 8 / 16), split-K over
    # workgroups; ragged N and K (K not a multiple of 128), f16 and f32 rows, against the exact-weight truth; 17 .. 32
    # rows also with option "batch_rounded" against the f16-weight truth
    for k, n in ((160, 33), (416, 9000), (3584, 512)):
        packed, scales, a16 = synth(k, n, 32, 5200 + n)
        w = T.MarlinWeight.upload(dev, packed, scales, k, n)
        try:
            dev.set_option("kernel", 4)
            for m, rounded in ((5, 0), (9, 0), (16, 0), (17, 0), (31, 0), (32, 0), (17, 1), (32, 1)):
                dev.set_option("batch_rounded", rounded)
                truth = gemm_truth(a16[:m], packed, scales, m, k, n, rounded=bool(rounded))
                bar = 1e-3 if rounded else TIGHT
                for nt in (1, 2, 3, 4):
                    dev.set_option("nt", nt)
                    for waves in (0, 8, 16):
                        dev.set_option("waves", waves)
                        for splits in ((1, 3) if n > 1000 else (1, 2, 3, 5)):
                            got = run_gemm(dev, w, a16[:m], m, n, splits)
                            assert rel_err(got, truth) < bar, (k, n, m, nt, waves, splits)
                        got32 = run_gemm(dev, w, a16[:m], m, n, 1, a_f32=True)
                        assert rel_err(got32, truth) < bar, (k, n, m, nt, waves, "f32")
                # the same launch twice is bitwise repeatable, split or not
                dev.set_option("nt", 0)
                dev.set_option("waves", 8)
                assert np.array_equal(run_gemm(dev, w, a16[:m], m, n, 3), run_gemm(dev, w, a16[:m], m, n, 3))
                dev.set_option("waves", 0)
        finally:
            for key in ("kernel", "nt", "waves", "batch_rounded"):
                dev.set_option(key, 0)
        # the library's own plan takes this kernel from 17 rows on (and from 9 on wide matrices): same bits as forced
        for m in ((12, 20, 32) if n > 8192 else (20, 32)):
            auto = run_gemm(dev, w, a16[:m], m, n)
            assert rel_err(auto, gemm_truth(a16[:m], packed, scales, m, k, n)) < TIGHT, (k, n, m)
        w.free()
    # the gated store (two tiles per wave: a gate tile and the up tile of the same features in one lane), unsplit and
    # through the split-K partial sums
    h, ffn = 288, 4608
    gp, gs = O.synth_packed(h, ffn, 5210), O.synth_scales(h, ffn, 5211)
    up, us = O.synth_packed(h, ffn, 5212), O.synth_scales(h, ffn, 5213)
    gd = (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16"))
    ud = (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16"))
    wp = T.MarlinWeight.gate_up(dev, gd, ud, h, ffn)
    for m in (12, 17, 32):
        a16 = O.synth_act_f16(m, h, 5214 + m)
        tg, tu = (gemm_truth(a16, gp, gs, m, h, ffn), gemm_truth(a16, up, us, m, h, ffn))
        want = tg / (1.0 + np.exp(-tg)) * tu
        for splits in (0, 2):
            out = T.GpuTensor.from_host(dev, np.full((m, ffn), np.nan, np.float32))
            T.gemm_swiglu(dev, wp, T.GpuTensor.from_host(dev, a16, "f16"), m, out, splits)
            assert rel_err(out.to_host(), want) < TIGHT, (m, splits)
    wp.free()


def test_split_factors_that_do_not_divide_the_k_chunks(dev):
    # 28 k-chunks: 8, 9, 11, 12, 13 ... splits leave trailing splits without any chunk; the launch
    # must fold them away (an empty split used to read past the end of the weight array)
    k, n = 3584, 256
    packed, scales, a16 = synth(k, n, 2, 77)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    truth = O.gemm_f64(f16_as_f32(a16), packed, scales, 2, k, n)
    try:
        for kernel in (2,):
            dev.set_option("kernel", kernel)
            for splits in (5, 8, 9, 11, 12, 13, 15, 20, 27, 28):
                assert rel_err(run_gemm(dev, w, a16, 2, n, splits), truth) < TIGHT, (kernel, splits)
    finally:
        dev.set_option("kernel", 0)
    w.free()


@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 16])
def test_decode_kernels_rows_and_f32_activations(dev, m):
    # K = 1184 is 37 groups: 9 full chunks + one chunk with three zero-padded groups; N = 200 is ragged
    k, n = 1184, 200
    packed, scales, a16 = synth(k, n, m, 3000 + m)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    truth = O.gemm_f64(f16_as_f32(a16), packed, scales, m, k, n)
    try:
        dev.set_option("prefill_min_m", 1 << 30)
        # 2 = one lane per column (M <= 4), 3 = streaming kernel (32-row blocks)
        for kernel in ((2, 3) if m <= 4 else (3,)):
            dev.set_option("kernel", kernel)
            for splits in (0, 1, 2, 3):
                for a_f32 in (False, True):
                    assert rel_err(run_gemm(dev, w, a16, m, n, splits, a_f32), truth) < TIGHT, (kernel, splits, a_f32)
    finally:
        dev.set_option("kernel", 0)
        dev.set_option("prefill_min_m", 33)
    w.free()


@pytest.mark.parametrize("m", [1, 3, 4, 5, 16, 32])
def test_f32_activations_keep_their_precision(dev, m):
    # The reference's decode activations are f32 (generate.rs:2153).  Cutting them to f16 would move
    # near-cancelling outputs of a 3584-deep sum by several percent of their value; the decode kernels take
    # every f32 activation as two f16 terms instead, so the f64 truth on the raw values holds to the same bar.
    k, n = 3584, 1152
    packed, scales, _ = synth(k, n, 1, 4000 + m)
    a_raw = (O.synth_normal_f32(m * k, 4100 + m) * np.float32(1.37)).reshape(m, k)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    truth = O.gemm_f64(a_raw, packed, scales, m, k, n)
    held_to, bar = truth, TIGHT
    for splits in (0, 1, 3):
        c = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))
        T.gemm(dev, w, T.GpuTensor.from_host(dev, a_raw), m, c, splits)
        assert rel_err(c.to_host(), held_to) < bar, splits
    rounded = O.gemm_f64(a_raw.astype(np.float16).astype(np.float32), packed, scales, m, k, n)
    assert rel_err(rounded, truth) > TOL       # what a single f16 term would give: outside the stated tolerance
    w.free()


def test_random_shapes_against_the_oracle(dev):
    # seeded sweep over ragged shapes: K any multiple of 32, N with and without tile padding, M across the three
    # kernels, forced and automatic split-K, f16 and f32 activations
    rng = np.random.default_rng(20250607)
    for case in range(48):
        k = 32 * int(rng.integers(1, 40))
        n = int(rng.choice([1, 7, 15, 16, 17, 63, 64, 65, 100, 129, 200, 333, 512, 600]))
        m = int(rng.choice([1, 2, 3, 4, 5, 9, 16, 17, 31, 32, 33, 47, 64, 70]))
        splits = int(rng.choice([0, 0, 1, 2, 3, 5]))
        a_f32 = bool(rng.integers(0, 2))
        print("case %d: k=%d n=%d m=%d splits=%d f32=%d" % (case, k, n, m, splits, a_f32), flush=True)
        packed, scales, a16 = synth(k, n, m, 5000 + case)
        w = T.MarlinWeight.upload(dev, packed, scales, k, n)
        got = run_gemm(dev, w, a16, m, n, splits, a_f32)
        truth = gemm_truth(a16, packed, scales, m, k, n)
        assert rel_err(got, truth) < (TIGHT if m <= EXACT_MAX_M else 1e-3), (case, k, n, m, splits, a_f32)
        assert np.array_equal(w.dequant_f16().to_host().reshape(-1), O.dequant_f16(packed, scales, k, n).reshape(-1)), case
        if m == 1:
            c = T.GpuTensor.from_host(dev, np.full(n, np.nan, np.float32))
            T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, f16_as_f32(a16)), T.GpuTensor.from_host(dev, packed),
                                T.GpuTensor.from_host(dev, scales, "f16"), c, n, k)
            assert rel_err(c.to_host(), truth[0]) < TIGHT, (case, "drop-in")
        w.free()


def test_random_deep_shapes_against_the_oracle(dev):
    # the same with K from 2048 to 6400, where the planners take sub-tiles, row groups or whole tiles by shape:
    # narrow, middling and wide N (up to 64, 128 and more column tiles), one to sixteen rows
    rng = np.random.default_rng(20251101)
    for case in range(20):
        k = 32 * int(rng.integers(64, 201))
        n = int(rng.choice([16, 72, 200, 1000, 4100, 6000, 8300]))
        m = int(rng.choice([1, 1, 2, 3, 4, 5, 8, 12, 16]))
        a_f32 = bool(rng.integers(0, 2))
        print("case %d: k=%d n=%d m=%d f32=%d" % (case, k, n, m, a_f32), flush=True)
        packed, scales, a16 = synth(k, n, m, 5200 + case)
        w = T.MarlinWeight.upload(dev, packed, scales, k, n)
        truth = gemm_truth(a16, packed, scales, m, k, n)
        assert rel_err(run_gemm(dev, w, a16, m, n, 0, a_f32), truth) < TIGHT, (case, k, n, m, a_f32)
        if m == 1:
            c = T.GpuTensor.from_host(dev, np.full(n, np.nan, np.float32))
            T.gemm_tw_marlin_m1(dev, T.GpuTensor.from_host(dev, f16_as_f32(a16)), T.GpuTensor.from_host(dev, packed),
                                T.GpuTensor.from_host(dev, scales, "f16"), c, n, k)
            assert rel_err(c.to_host(), truth[0]) < TIGHT, (case, "drop-in")
        w.free()


def test_m_larger_than_32_is_tiled_by_the_decode_kernels(dev):
    # with the prefill kernel switched off, any M runs as 32-row blocks of the batched-decode kernel (exact weights;
    # with option "batch_rounded" the FP16 Q4 unpack, the last 6 rows included: one call, one arithmetic), or as
    # 32-row blocks of the streaming kernel
    m, k, n = 70, 256, 128
    packed, scales, a16 = synth(k, n, m, 33)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    try:
        dev.set_option("prefill_min_m", 1 << 30)
        exact = O.gemm_f64(f16_as_f32(a16), packed, scales, m, k, n)
        got = run_gemm(dev, w, a16, m, n)
        assert rel_err(got, exact) < TIGHT
        for lo, hi in ((0, 32), (32, 64), (64, 70)):
            block = run_gemm(dev, w, a16[lo:hi], hi - lo, n)
            if hi - lo > 16:
                assert np.array_equal(got[lo:hi], block)
            else:       # six rows alone take another kernel: the same sums in another order
                assert rel_err(block, got[lo:hi]) < TIGHT
        dev.set_option("batch_rounded", 1)
        got = run_gemm(dev, w, a16, m, n)
        assert rel_err(got, gemm_truth(a16, packed, scales, m, k, n, rounded=True)) < 1e-3
        assert np.abs(got - exact).max() / np.abs(exact).max() < 1e-3
        dev.set_option("batch_rounded", 0)
        dev.set_option("kernel", 3)
        assert rel_err(run_gemm(dev, w, a16, m, n), O.gemm_f64(f16_as_f32(a16), packed, scales, m, k, n)) < TIGHT
    finally:
        dev.set_option("kernel", 0)
        dev.set_option("batch_rounded", 0)
        dev.set_option("prefill_min_m", 33)
    w.free()


@pytest.mark.parametrize("m,k,n", [(17, 256, 128), (32, 3584, 512), (33, 256, 128), (40, 128, 64), (40, 384, 80), (70, 640, 64), (64, 896, 1152),
                                   (128, 1184, 200), (200, 4096, 704), (512, 4096, 1024)])
def test_prefill_kernel_matches_oracle(dev, m, k, n):
    # M > 32 runs the LDS/MFMA prefill kernel (here forced for every M).  Its weights are the reference's FP16 Q4 unpack,
    # f16(scale*(q-8)) (quantize.rs:534-571), so its oracle is A x f16-dequant(W) in f64: tight match.
    # Against the f32-weight matmul the FP16 rounding of the weights (2^-12 relative each) shows on
    # near-cancelling outputs, so that comparison is made relative to the largest output.
    # Ragged M (33, 200), K not a multiple of 128 (1184), N not a multiple of 256 / 64 (200, 704); 1 to 5
    # k-chunks (the k loop is unrolled by three with a remainder); every block form.
    packed, scales, a16 = synth(k, n, m, 4000 + m)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    a = f16_as_f32(a16)
    w16 = O.dequant_f16(packed, scales, k, n).view(np.float16).astype(np.float64)
    exact = a.astype(np.float64) @ w16
    truth = O.gemm_f64(a, packed, scales, m, k, n)
    try:
        dev.set_option("prefill_min_m", 1)
        for bm in (64, 128, 192):   # 192: 128 rows x 192 columns, three tiles per wave
            dev.set_option("prefill_bm", bm)
            for a_f32 in (False, True):
                got = run_gemm(dev, w, a16, m, n, a_f32=a_f32)
                assert rel_err(got, exact) < 1e-3, (bm, a_f32)   # one f32 accumulator over all of K: a few 1e-4 at K = 4096
                assert np.abs(got - truth).max() / np.abs(truth).max() < 1e-3
    finally:
        dev.set_option("prefill_bm", 0)
        dev.set_option("prefill_min_m", 33)
    # with the prefill kernel off: the batched-decode kernel runs the same arithmetic in 32-row blocks under option
    # "batch_rounded"; by default it and the streaming kernel use the exact weights
    try:
        dev.set_option("prefill_min_m", 1 << 30)
        assert rel_err(run_gemm(dev, w, a16, m, n), truth) < TIGHT
        dev.set_option("batch_rounded", 1)
        if m > 16:
            assert rel_err(run_gemm(dev, w, a16, m, n), exact) < 1e-3
        dev.set_option("batch_rounded", 0)
        dev.set_option("kernel", 3)
        assert rel_err(run_gemm(dev, w, a16, m, n), truth) < TIGHT
    finally:
        dev.set_option("kernel", 0)
        dev.set_option("batch_rounded", 0)
        dev.set_option("prefill_min_m", 33)
    w.free()


@pytest.mark.parametrize("m,k,n", [(64, 4096, 704), (100, 1184, 200), (130, 2048, 320)])
def test_prefill_split_k(dev, m, k, n):
    # Few workgroups: K is cut across workgroups, f32 partial sums are added in split order by a second
    # kernel.  Explicit factors (also ones that do not divide the chunk count, and more than there are
    # chunks) and the automatic choice; f32 activations share the scratch with the partials.
    packed, scales, a16 = synth(k, n, m, 5000 + m)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    a = f16_as_f32(a16)
    w16 = O.dequant_f16(packed, scales, k, n).view(np.float16).astype(np.float64)
    exact = a.astype(np.float64) @ w16
    try:
        for bm in (64, 128, 192):   # 192: 128 rows x 192 columns, three tiles per wave
            dev.set_option("prefill_bm", bm)
            base = run_gemm(dev, w, a16, m, n, splits=1)
            assert rel_err(base, exact) < 1e-3
            for splits in (0, 2, 3, 7, 64):
                for a_f32 in (False, True):
                    got = run_gemm(dev, w, a16, m, n, splits=splits, a_f32=a_f32)
                    assert rel_err(got, exact) < 1e-3, (bm, splits, a_f32)
                    assert rel_err(got, base) < 1e-3, (bm, splits, a_f32)      # another summation order
            again = run_gemm(dev, w, a16, m, n, splits=3)
            assert np.array_equal(again, run_gemm(dev, w, a16, m, n, splits=3))   # no atomics: run-to-run identical
    finally:
        dev.set_option("prefill_bm", 0)
    w.free()


def test_empty_inputs(dev):
    w = T.MarlinWeight.upload(dev, np.zeros(0, np.uint8), np.zeros(0, np.uint16), 64, 0)
    c = T.GpuTensor.zeros(dev, (4,), "f32")
    a = T.GpuTensor.zeros(dev, (64,), "f16")
    T.gemm(dev, w, a, 1, c)          # N == 0: nothing to do
    T.gemm(dev, w, a, 0, c)          # M == 0
    w.free()
    w0 = T.MarlinWeight.upload(dev, np.zeros(0, np.uint8), np.zeros(0, np.uint16), 0, 8)
    c8 = T.GpuTensor.from_host(dev, np.ones(8, np.float32))
    T.gemm(dev, w0, a, 1, c8)        # K == 0: the empty sum
    assert np.all(c8.to_host() == 0)
    w0.free()


def test_weight_handle_with_one_copy_builds_the_other_on_demand(dev):
    # A decode-only or prefill-only handle holds 4.5 bits per weight; the other order is built from it, word for word,
    # at the first call that needs it: results and Q4 unpack equal those of a handle made with both copies.
    k, n = 640, 200
    packed, scales = O.synth_packed(k, n, 990), O.synth_scales(k, n, 991)
    both = T.MarlinWeight.upload(dev, packed, scales, k, n)
    assert both.copies == 3
    one_copy = both.nbytes // 2
    a1 = T.GpuTensor.from_host(dev, O.synth_act_f16(1, k, 992), "f16")
    a8 = T.GpuTensor.from_host(dev, O.synth_act_f16(8, k, 993), "f16")
    a40 = T.GpuTensor.from_host(dev, O.synth_act_f16(40, k, 994), "f16")
    def run(w):
        outs = []
        for a, m in ((a1, 1), (a8, 8), (a40, 40)):
            c = T.GpuTensor.zeros(dev, (m, n), "f32")
            T.gemm(dev, w, a, m, c)
            outs.append(c.to_host())
        return outs
    want = run(both)
    want_deq = both.dequant_f16().to_host()
    for first, label in ((T.MarlinWeight.COPY_COLUMN_LANE, "column-lane first"), (T.MarlinWeight.COPY_TILES, "tiles first")):
        dev.set_option("weight_copies", first)
        w = T.MarlinWeight.upload(dev, packed, scales, k, n)
        dev.set_option("weight_copies", 0)
        assert w.copies == first and w.nbytes == one_copy, label
        # a capture may not allocate: the call that needs the missing copy is refused, and says what to do
        m_other, a_other = (40, a40) if first == T.MarlinWeight.COPY_COLUMN_LANE else (1, a1)
        c = T.GpuTensor.zeros(dev, (m_other, n), "f32")
        with pytest.raises(T.DeviceError, match="twm_weight_ensure"):
            T.GraphCapture.record_with_device(dev, lambda: T.gemm(dev, w, a_other, m_other, c))
        assert w.copies == first
        # the export of a one-copy handle is half as long and comes back as it was
        blob = w.export_blob()
        assert blob.size == 64 + one_copy + 96          # header, one copy, the table of measured plans
        w_back = T.MarlinWeight.import_blob(dev, blob)
        assert w_back.copies == first
        got = run(w)
        assert w.copies == 3 and w.nbytes == 2 * one_copy, label
        for g, t in zip(got, want):
            assert np.array_equal(g, t), label
        for src in (0, 1):
            dev.set_option("dequant_src", src)
            assert np.array_equal(w.dequant_f16().to_host(), want_deq), label
            assert np.array_equal(w_back.dequant_f16().to_host(), want_deq), label
        dev.set_option("dequant_src", 0)
        for g, t in zip(run(w_back), want):
            assert np.array_equal(g, t), label
        # drop one again: the handle is back to one copy, and the last copy cannot be dropped
        w.drop(first)
        assert w.copies == 3 - first and w.nbytes == one_copy
        with pytest.raises(T.DeviceError):
            w.drop(3 - first)
        for g, t in zip(run(w), want):
            assert np.array_equal(g, t), label
        w.free(); w_back.free()
    both.free()


def test_weight_tune_keeps_results_and_travels_with_the_blob(dev):
    # twm_weight_tune (the role of autotune.rs:254-396) times the launch forms and keeps the fastest per bucket of row
    # counts.  Whatever it keeps, results stay inside the same bar against the oracle, a call with an explicit split
    # factor or a knob set is not touched, and the table comes back from an exported blob.
    k, n = 2048, 768
    packed, scales = O.synth_packed(k, n, 1500), O.synth_scales(k, n, 1501)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    ms = [1, 4, 8, 32, 80]
    acts = {m: O.synth_act_f16(m, k, 1510 + m) for m in ms}
    before = {m: run_gemm(dev, w, acts[m], m, n, 0) for m in ms}
    w.tune(ms)
    plans = {m: w.tuned_plan(m) for m in ms}
    print("kept plans:", plans)
    assert w.tuned_plan(2) is None and w.tuned_plan(16) is None       # buckets that were not asked for
    for m in ms:
        got = run_gemm(dev, w, acts[m], m, n, 0)
        if m <= 32:
            truth = O.gemm_f64(f16_as_f32(acts[m]), packed, scales, m, k, n)
            assert rel_err(got, truth) < TIGHT, (m, plans[m])
        else:   # the prefill GEMM: weights of the FP16 Q4 unpack, f32 accumulation in whatever K-split order
            w16 = O.dequant_f16(packed, scales, k, n).view(np.float16).astype(np.float64).reshape(k, n)
            truth = acts[m].view(np.float16).astype(np.float64).reshape(m, k) @ w16
            assert rel_err(got, truth) < 1e-3 and rel_err(before[m], truth) < 1e-3, (m, plans[m])
        # forced calls do not look at the table
        assert np.array_equal(run_gemm(dev, w, acts[m], m, n, 1), run_gemm(dev, w, acts[m], m, n, 1))
    blob = w.export_blob()
    w2 = T.MarlinWeight.import_blob(dev, blob)
    for m in ms:
        assert w2.tuned_plan(m) == plans[m]
        assert np.array_equal(run_gemm(dev, w2, acts[m], m, n, 0), run_gemm(dev, w, acts[m], m, n, 0))
    # tuning again with no row counts changes nothing; an entry outside the option ranges is dropped at import
    w.tune([])
    assert {m: w.tuned_plan(m) for m in ms} == plans
    bad = blob.copy()
    bad[-96:-88] = np.array([1, 9, 0, 0, 0, 0, 0, 0], np.uint8)         # bucket 0: kernel 9 does not exist
    w3 = T.MarlinWeight.import_blob(dev, bad)
    assert w3.tuned_plan(1) is None
    for x in (w, w2, w3):
        x.free()


def test_tune_on_upload_option(dev):
    # option "tune_on_upload": a new handle is tuned at once (1 = the decode row counts, 2 = the prefill ones too); whatever
    # the tuner keeps, results stay inside the bar, and a handle made with the option off has no measured plans
    k, n = 1024, 640
    packed, scales = O.synth_packed(k, n, 1600), O.synth_scales(k, n, 1601)
    lib = T._lib.load()
    assert lib.twm_ctx_set_option(dev.handle, b"tune_on_upload", 3) == T._lib.SHAPE_ERROR
    plain = T.MarlinWeight.upload(dev, packed, scales, k, n)
    assert all(plain.tuned_plan(m) is None for m in (1, 4, 8, 16, 32, 128))
    try:
        dev.set_option("tune_on_upload", 2)
        w = T.MarlinWeight.upload(dev, packed, scales, k, n)
        fused = T.MarlinWeight.fuse_n(dev, [plain, plain])
    finally:
        dev.set_option("tune_on_upload", 0)
    print("kept plans:", {m: w.tuned_plan(m) for m in (1, 4, 8, 16, 32, 128, 512, 2048)})
    for m in (1, 8, 32):
        a16 = O.synth_act_f16(m, k, 1610 + m)
        truth = O.gemm_f64(f16_as_f32(a16), packed, scales, m, k, n)
        assert rel_err(run_gemm(dev, w, a16, m, n, 0), truth) < TIGHT, (m, w.tuned_plan(m))
        got2 = run_gemm(dev, fused, a16, m, 2 * n, 0)
        assert rel_err(got2[:, :n], truth) < TIGHT and rel_err(got2[:, n:], truth) < TIGHT, (m, fused.tuned_plan(m))
    for x in (plain, w, fused):
        x.free()


def test_repacked_weight_blob_round_trip_through_a_warp_file(dev, tmp_path):
    from tensorwarp_amd import warp_cache as W
    k, n, ffn = 640, 200, 96
    packed, scales, a16 = synth(k, n, 3, 1000)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    gp, gs = O.synth_packed(k, ffn, 1001), O.synth_scales(k, ffn, 1002)
    up, us = O.synth_packed(k, ffn, 1003), O.synth_scales(k, ffn, 1004)
    wp = T.MarlinWeight.gate_up(dev, (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16")),
                                (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16")), k, ffn)
    blob, blob_p = w.export_blob(), wp.export_blob()
    assert blob.size == 64 + w.nbytes + 96 and bytes(blob[:8]) == b"TWMWGT01"
    path = tmp_path / "model.warp"
    W.save_warp_cache(path, '{"layout": "gfx950"}', [("l0.w", W.DTYPE_U8, blob.shape, blob),
                                                    ("l0.gate_up", W.DTYPE_U8, blob_p.shape, blob_p)])
    _, tensors = W.load_warp_cache(path)
    w2 = T.MarlinWeight.import_blob(dev, tensors[0].array())
    wp2 = T.MarlinWeight.import_blob(dev, tensors[1].array())
    assert (w2.k, w2.n, w2.paired) == (k, n, False) and (wp2.k, wp2.n, wp2.paired) == (k, 2 * ffn, True)
    ad = T.GpuTensor.from_host(dev, a16, "f16")
    for m in (1, 3):
        c1, c2 = T.GpuTensor.zeros(dev, (m, n), "f32"), T.GpuTensor.zeros(dev, (m, n), "f32")
        T.gemm(dev, w, ad, m, c1)
        T.gemm(dev, w2, ad, m, c2)
        assert np.array_equal(c1.to_host(), c2.to_host())
        s1, s2 = T.GpuTensor.zeros(dev, (m, ffn), "f32"), T.GpuTensor.zeros(dev, (m, ffn), "f32")
        T.gemm_swiglu(dev, wp, ad, m, s1)
        T.gemm_swiglu(dev, wp2, ad, m, s2)
        assert np.array_equal(s1.to_host(), s2.to_host())
    assert np.array_equal(w2.dequant_f16().to_host(), O.dequant_f16(packed, scales, k, n).reshape(k, n))
    assert np.array_equal(w2.export_blob(), blob)
    # refusals: flipped payload byte, truncated blob, other layout number, foreign bytes
    bad = blob.copy()
    bad[64 + 1234] ^= 1
    short = blob[:-16]
    other = blob.copy()
    other[8] ^= 0x40
    for b in (bad, short, other, np.zeros(64, np.uint8), np.zeros(10, np.uint8)):
        with pytest.raises(T.DeviceError):
            T.MarlinWeight.import_blob(dev, b)
    empty = T.MarlinWeight.upload(dev, np.zeros(0, np.uint8), np.zeros(0, np.uint16), 64, 0)
    e2 = T.MarlinWeight.import_blob(dev, empty.export_blob())
    assert (e2.k, e2.n) == (64, 0)
    for x in (w, w2, wp, wp2, empty, e2):
        x.free()


# ---------------------------------------------------------------- expert banks (MoE decode)

def make_bank(dev, k, n, experts, seed, pair=False, pad_bytes=0, pad_scales=0):
    """Expert matrices back to back in two buffers with optional slack between experts, as the reference's
    experts_gu_raw / experts_gu_scales."""
    G = k // 32
    pb, sb = G * n * 16 + pad_bytes, G * n + pad_scales
    packed = [O.synth_packed(k, n, seed + 2 * e) for e in range(experts)]
    scales = [O.synth_scales(k, n, seed + 2 * e + 1) for e in range(experts)]
    pbuf = np.full(experts * pb, 0xEE, np.uint8)
    sbuf = np.full(experts * sb, 0x7BFF, np.uint16)
    for e in range(experts):
        pbuf[e * pb:e * pb + G * n * 16] = packed[e]
        sbuf[e * sb:e * sb + G * n] = scales[e]
    bank = T.ExpertBank.from_device(dev, T.GpuTensor.from_host(dev, pbuf), T.GpuTensor.from_host(dev, sbuf, "f16"),
                                    pb, sb, k, n, experts, pair_gate_up=pair)
    return bank, packed, scales


def geglu_close(got, g, u, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return bool(np.all(np.abs(got - want) <= 6e-7 * np.abs(np.asarray(g, np.float64) * np.asarray(u, np.float64)) + 1e-30))


def test_geglu_rows(dev):
    batch, dim = 8, 96
    gu = (O.synth_normal_f32(batch * 2 * dim, 1020) * np.float32(2.5)).reshape(batch, 2 * dim)
    g, u = np.ascontiguousarray(gu[:, :dim]), np.ascontiguousarray(gu[:, dim:])
    out = T.GpuTensor.zeros(dev, (batch, dim), "f32")
    T.batched_marlin_split_geglu(dev, T.GpuTensor.from_host(dev, gu), out, dim, batch)
    assert geglu_close(out.to_host(), g, u, O.gelu_mul(g, u))
    j = np.arange(dim)
    col = (j // 32) * 64 + j % 32
    paired = np.zeros_like(gu)
    paired[:, col], paired[:, col + 32] = g, u
    out2 = T.GpuTensor.zeros(dev, (batch, dim), "f32")
    T.batched_marlin_split_geglu(dev, T.GpuTensor.from_host(dev, paired), out2, dim, batch, paired=True)
    assert np.array_equal(out2.to_host(), out.to_host())


@pytest.mark.parametrize("k,dim,experts,top_k", [(2816, 704, 12, 8), (256, 32, 3, 2), (1184, 96, 5, 4), (64, 64, 4, 1)])
def test_bank_gate_up_and_fused_geglu(dev, k, dim, experts, top_k):
    # batched_marlin_gate_up + batched_marlin_split_geglu (moe_q4_generate.rs:618-631), Gemma MoE shape first
    n = 2 * dim
    ids_h = np.array([(5 * s + 3) % experts for s in range(top_k)], np.float32)
    ids = T.GpuTensor.from_host(dev, ids_h)
    a16 = O.synth_act_f16(1, k, 1030)
    a32 = f16_as_f32(a16).reshape(1, k)
    plain, packed, scales = make_bank(dev, k, n, experts, 1040, pad_bytes=32, pad_scales=8)
    out = T.GpuTensor.from_host(dev, np.full((top_k, n), np.nan, np.float32))
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), plain, ids, out, top_k)
    truth = O.bank_gemv_f64(a32, packed, scales, ids_h, k, n)
    assert rel_err(out.to_host(), truth) < TIGHT
    # f16 and f32 activations bit for bit; the same row from the dense kernel on one expert, to f32 rounding
    out16 = T.GpuTensor.zeros(dev, (top_k, n), "f32")
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a16, "f16"), plain, ids, out16, top_k)
    assert np.array_equal(out16.to_host(), out.to_host())
    e0 = int(ids_h[0])
    w0 = T.MarlinWeight.upload(dev, packed[e0], scales[e0], k, n)
    c0 = T.GpuTensor.zeros(dev, (n,), "f32")
    T.gemm(dev, w0, T.GpuTensor.from_host(dev, a16, "f16"), 1, c0, 1)
    assert rel_err(out.to_host()[0], c0.to_host()) < 1e-4      # (another plan, another order of the f32 sum)
    # device-indexed single expert (gemm_tw_marlin_m1_indirect): one slot, ids pointer at the wanted entry
    one = T.GpuTensor.zeros(dev, (n,), "f32")
    last = T.GpuTensor.from_host(dev, ids_h[top_k - 1:top_k].copy())
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), plain, last, one, 1)
    assert np.array_equal(one.to_host(), out.to_host()[top_k - 1])
    # fused GEGLU on the paired bank = unfused rows + split_geglu, bit for bit
    pairedb, _, _ = make_bank(dev, k, n, experts, 1040, pair=True)
    seq = T.GpuTensor.zeros(dev, (top_k, dim), "f32")
    T.batched_marlin_split_geglu(dev, out, seq, dim, top_k)
    fused = T.GpuTensor.from_host(dev, np.full((top_k, dim), np.nan, np.float32))
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), pairedb, ids, fused, top_k, act=T.ACT_GEGLU)
    assert np.array_equal(fused.to_host(), seq.to_host())
    tg, tu = truth[:, :dim], truth[:, dim:]
    want = 0.5 * tg * (1.0 + np.tanh(0.7978845608 * (tg + 0.044715 * tg ** 3))) * tu
    assert rel_err(fused.to_host(), want) < TIGHT
    sw = T.GpuTensor.zeros(dev, (top_k, dim), "f32")
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), pairedb, ids, sw, top_k, act=T.ACT_SWIGLU)
    assert rel_err(sw.to_host(), tg / (1.0 + np.exp(-tg)) * tu) < TIGHT
    with pytest.raises(T.DeviceError):
        T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), plain, ids, fused, top_k, act=T.ACT_GEGLU)
    for x in (plain, pairedb, w0):
        x.free()


@pytest.mark.parametrize("k,n,experts,top_k", [(704, 2816, 12, 8), (64, 40, 3, 3), (1184, 200, 4, 16), (4096, 128, 2, 1)])
def test_bank_down_axpy_adds_in_slot_order(dev, k, n, experts, top_k):
    ids_h = np.array([(7 * s + 1) % experts for s in range(top_k)], np.float32)
    wts_h = (np.abs(O.synth_normal_f32(top_k, 1050)) * np.float32(0.3) + np.float32(0.01)).astype(np.float32)
    a16 = O.synth_act_f16(top_k, k, 1051)
    a32 = f16_as_f32(a16).reshape(top_k, k)
    acc0 = O.synth_normal_f32(n, 1052)
    bank, packed, scales = make_bank(dev, k, n, experts, 1060)
    ids, wts = T.GpuTensor.from_host(dev, ids_h), T.GpuTensor.from_host(dev, wts_h)
    acc = T.GpuTensor.from_host(dev, acc0)
    T.batched_marlin_down_axpy(dev, T.GpuTensor.from_host(dev, a32), bank, ids, wts, acc, top_k)
    rows = O.bank_gemv_f64(a32, packed, scales, ids_h, k, n)
    truth = acc0.astype(np.float64) + (wts_h.astype(np.float64)[:, None] * rows).sum(axis=0)
    assert rel_err(acc.to_host(), truth) < TIGHT
    # equal, bit for bit, to the per-slot rows of the batched GEMV combined on the host in slot order in f32
    per = T.GpuTensor.zeros(dev, (top_k, n), "f32")
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), bank, ids, per, top_k, per_slot_rows=True)
    ph = per.to_host().reshape(top_k, n)
    assert rel_err(ph, rows) < TIGHT
    acc2 = T.GpuTensor.from_host(dev, acc0)
    T.batched_marlin_down_axpy(dev, T.GpuTensor.from_host(dev, a16, "f16"), bank, ids, wts, acc2, top_k)
    assert np.array_equal(acc2.to_host(), acc.to_host())          # run to run and f16 / f32 activations alike
    if top_k <= 16:
        with pytest.raises(T.DeviceError):
            T.batched_marlin_down_axpy(dev, T.GpuTensor.from_host(dev, np.zeros((17, k), np.float32)), bank,
                                       T.GpuTensor.from_host(dev, np.zeros(17, np.float32)),
                                       T.GpuTensor.from_host(dev, np.zeros(17, np.float32)), acc2, 17)
    bank.free()


def test_bank_kernels_on_both_sub_tile_widths(dev):
    # 16- and 32-column sub-tiles, one pass per wave and the loop over passes (forced through the options)
    k, dim, experts, top_k = 1184, 96, 5, 4
    n = 2 * dim
    ids_h = np.array([(3 * s + 1) % experts for s in range(top_k)], np.float32)
    ids = T.GpuTensor.from_host(dev, ids_h)
    a32 = f16_as_f32(O.synth_act_f16(1, k, 4400)).reshape(1, k) * np.float32(1.0 + 2.0 ** -13)
    plain, packed, scales = make_bank(dev, k, n, experts, 4410)
    pairedb, _, _ = make_bank(dev, k, n, experts, 4410, pair=True)
    truth = O.bank_gemv_f64(a32, packed, scales, ids_h, k, n)
    tg, tu = truth[:, :dim], truth[:, dim:]
    gated = tg / (1.0 + np.exp(-tg)) * tu
    # down projection of the gated rows: (top_k, dim) -> k outputs
    down, dpacked, dscales = make_bank(dev, dim, k, experts, 4420)
    wts_h = np.array([0.4, 0.3, 0.2, 0.1], np.float32)
    wts = T.GpuTensor.from_host(dev, wts_h)
    rows = gated.astype(np.float32)
    per_slot = np.stack([O.bank_gemv_f64(rows[s:s + 1], dpacked, dscales, ids_h[s:s + 1], dim, k)[0] for s in range(top_k)])
    down_truth = (wts_h.astype(np.float64)[:, None] * per_slot).sum(0)
    try:
        for sub in (16, 32):
            dev.set_option("sub", sub)
            for waves in (0, 1, 2, 16):
                dev.set_option("waves", waves)
                out = T.GpuTensor.from_host(dev, np.full((top_k, n), np.nan, np.float32))
                T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), plain, ids, out, top_k)
                assert rel_err(out.to_host(), truth) < TIGHT, (sub, waves)
                fused = T.GpuTensor.from_host(dev, np.full((top_k, dim), np.nan, np.float32))
                T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), pairedb, ids, fused, top_k, act=T.ACT_SWIGLU)
                assert rel_err(fused.to_host(), gated) < TIGHT, (sub, waves)
                acc = T.GpuTensor.zeros(dev, (k,), "f32")
                T.batched_marlin_down_axpy(dev, T.GpuTensor.from_host(dev, rows), down, ids, wts, acc, top_k)
                assert rel_err(acc.to_host(), down_truth) < TIGHT, (sub, waves)
    finally:
        dev.set_option("sub", 0)
        dev.set_option("waves", 0)
    for b in (plain, pairedb, down):
        b.free()


def test_bank_ignores_ids_outside_the_bank(dev):
    k, n, experts = 128, 64, 3
    bank, packed, scales = make_bank(dev, k, n, experts, 1070)
    ids_h = np.array([1.0, -1.0, 3.0, 2.0, np.nan], np.float32)
    a32 = f16_as_f32(O.synth_act_f16(1, k, 1071)).reshape(1, k)
    out = T.GpuTensor.from_host(dev, np.full((5, n), np.nan, np.float32))
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), bank, T.GpuTensor.from_host(dev, ids_h), out, 5)
    got = out.to_host().reshape(5, n)
    assert not got[1].any() and not got[2].any() and not got[4].any()
    assert rel_err(got[[0, 3]], O.bank_gemv_f64(a32, packed, scales, [1, 2], k, n)) < TIGHT
    bank.free()


def test_bank_from_offset_tables_with_unequal_spacing(dev):
    # gemm_tw_marlin_m1_indirect's addressing (quantize_indirect.rs:196-197): expert e at packed_base + packed_offsets[e]
    # bytes and scales_base + scales_offsets[e] elements, the experts in any order and with gaps of any size
    k, n, experts = 256, 96, 4
    G = k // 32
    packed = [O.synth_packed(k, n, 1080 + 2 * e) for e in range(experts)]
    scales = [O.synth_scales(k, n, 1081 + 2 * e) for e in range(experts)]
    order, gaps_p, gaps_s = [2, 0, 3, 1], [4, 260, 0, 12], [1, 0, 7, 33]
    pbuf, sbuf = np.full(4 * (G * n * 16 + 300), 0xEE, np.uint8), np.full(4 * (G * n + 50), 0x7BFF, np.uint16)
    poff, soff = np.zeros(experts, np.uint32), np.zeros(experts, np.uint32)
    pp = ss = 0
    for e, gp, gs in zip(order, gaps_p, gaps_s):
        pp, ss = pp + gp, ss + gs
        poff[e], soff[e] = pp, ss
        pbuf[pp:pp + G * n * 16] = packed[e]
        sbuf[ss:ss + G * n] = scales[e]
        pp, ss = pp + G * n * 16, ss + G * n
    pd, sd = T.GpuTensor.from_host(dev, pbuf), T.GpuTensor.from_host(dev, sbuf, "f16")
    pod, sod = T.GpuTensor.from_host(dev, poff.view(np.int32), "i32"), T.GpuTensor.from_host(dev, soff.view(np.int32), "i32")
    bank = T.ExpertBank.from_device_offsets(dev, pd, pod, sd, sod, k, n, experts)
    ids = [3, 0, 2, 1, 3]
    a32 = f16_as_f32(O.synth_act_f16(1, k, 1090)).reshape(1, k)
    out = T.GpuTensor.zeros(dev, (len(ids), n), "f32")
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), bank, T.GpuTensor.from_host(dev, np.array(ids, np.float32)), out, len(ids))
    assert rel_err(out.to_host().reshape(len(ids), n), O.bank_gemv_f64(a32, packed, scales, ids, k, n)) < TIGHT
    # the bank equals the one built from equal strides, byte for byte in its results
    bank2, _, _ = make_bank(dev, k, n, 1, 1080)
    o1, o2 = T.GpuTensor.zeros(dev, (1, n), "f32"), T.GpuTensor.zeros(dev, (1, n), "f32")
    zero = T.GpuTensor.from_host(dev, np.zeros(1, np.float32))
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), bank, zero, o1, 1)
    T.batched_marlin_gate_up(dev, T.GpuTensor.from_host(dev, a32), bank2, zero, o2, 1)
    assert np.array_equal(o1.to_host(), o2.to_host())
    # a record offset that is not a multiple of four bytes is the reference kernel's own limit (it reads 32-bit words)
    poff_bad = poff.copy(); poff_bad[1] += 2
    with pytest.raises(T.DeviceError):
        T.ExpertBank.from_device_offsets(dev, pd, T.GpuTensor.from_host(dev, poff_bad.view(np.int32), "i32"), sd, sod, k, n, experts)
    bank.free(); bank2.free()


@pytest.mark.parametrize("k,dim,experts,top_k", [(2816, 704, 12, 8), (96, 20, 3, 3), (1184, 100, 4, 20), (4096, 64, 2, 1)])
def test_expert_launches_on_the_reference_slabs(dev, k, dim, experts, top_k):
    # The reference's three MoE launches with its own arguments (moe_batched_marlin.rs:153-232): all experts' TW-Marlin
    # arrays in two slabs, per-expert strides, ids and weights on the device; nothing is repacked.  The strides are
    # larger than the arrays (a gap of junk between experts), f32 activations that are not f16 values.
    n, G = 2 * dim, k // 32
    gap_p, gap_s = 48, 5
    pbe, spe = G * n * 16 + gap_p, G * n + gap_s
    packed = [O.synth_packed(k, n, 5100 + 2 * e) for e in range(experts)]
    scales = [O.synth_scales(k, n, 5101 + 2 * e) for e in range(experts)]
    pbuf, sbuf = np.full(experts * pbe, 0xEE, np.uint8), np.full(experts * spe, 0x7BFF, np.uint16)
    for e in range(experts):
        pbuf[e * pbe:e * pbe + G * n * 16] = packed[e]
        sbuf[e * spe:e * spe + G * n] = scales[e]
    pd, sd = T.GpuTensor.from_host(dev, pbuf), T.GpuTensor.from_host(dev, sbuf, "f16")
    ids_h = np.array([(5 * s + 1) % experts for s in range(top_k)], np.float32)
    wts_h = (np.abs(O.synth_normal_f32(top_k, 5150)) * np.float32(0.3) + np.float32(0.01)).astype(np.float32)
    ids, wts = T.GpuTensor.from_host(dev, ids_h), T.GpuTensor.from_host(dev, wts_h)
    a32 = O.synth_normal_f32(k, 5151).reshape(1, k)
    # gate + up
    gu = T.GpuTensor.zeros(dev, (top_k, n), "f32")
    T.batched_marlin_gate_up_slabs(dev, T.GpuTensor.from_host(dev, a32), pd, sd, ids, gu, pbe, spe, n, k, top_k)
    rows = O.bank_gemv_f64(a32, packed, scales, ids_h, k, n)
    guh = gu.to_host().reshape(top_k, n)
    assert rel_err(guh, rows) < TIGHT
    # split + GEGLU, the plain [gate | up] order
    act = T.GpuTensor.zeros(dev, (top_k, dim), "f32")
    T.batched_marlin_split_geglu(dev, gu, act, dim, top_k)
    g64, u64 = guh[:, :dim].astype(np.float64), guh[:, dim:].astype(np.float64)
    want = 0.5 * g64 * (1.0 + np.tanh(0.7978845608 * (g64 + 0.044715 * g64 ** 3))) * u64
    assert rel_err(act.to_host().reshape(top_k, dim), want) < 1e-5
    # down + weighted sum on a [dim -> hidden] slab: the roles of K and N swap, so build a second pair of slabs
    kd, nd = (dim + 31) // 32 * 32, 72
    Gd = kd // 32
    pbe_d, spe_d = Gd * nd * 16 + 16, Gd * nd + 3
    packed_d = [O.synth_packed(kd, nd, 5200 + 2 * e) for e in range(experts)]
    scales_d = [O.synth_scales(kd, nd, 5201 + 2 * e) for e in range(experts)]
    pbuf_d, sbuf_d = np.full(experts * pbe_d, 0xEE, np.uint8), np.full(experts * spe_d, 0x7BFF, np.uint16)
    for e in range(experts):
        pbuf_d[e * pbe_d:e * pbe_d + Gd * nd * 16] = packed_d[e]
        sbuf_d[e * spe_d:e * spe_d + Gd * nd] = scales_d[e]
    ad = O.synth_normal_f32(top_k * kd, 5250).reshape(top_k, kd)
    acc0 = O.synth_normal_f32(nd, 5251)
    acc = T.GpuTensor.from_host(dev, acc0)
    pdd, sdd = T.GpuTensor.from_host(dev, pbuf_d), T.GpuTensor.from_host(dev, sbuf_d, "f16")
    T.batched_marlin_down_axpy_slabs(dev, T.GpuTensor.from_host(dev, ad), pdd, sdd, ids, wts, acc, pbe_d, spe_d, nd, kd, top_k)
    rows_d = O.bank_gemv_f64(ad, packed_d, scales_d, ids_h, kd, nd)
    truth = acc0.astype(np.float64) + (wts_h.astype(np.float64)[:, None] * rows_d).sum(axis=0)
    assert rel_err(acc.to_host(), truth) < TIGHT
    acc2 = T.GpuTensor.from_host(dev, acc0)
    T.batched_marlin_down_axpy_slabs(dev, T.GpuTensor.from_host(dev, ad), pdd, sdd, ids, wts, acc2, pbe_d, spe_d, nd, kd, top_k)
    assert np.array_equal(acc2.to_host(), acc.to_host())          # slot order: run to run identical
    # the same numbers as a bank built from the same slabs (other kernels, other order of the f32 sum)
    bank = T.ExpertBank.from_device(dev, pdd, sdd, pbe_d, spe_d, kd, nd, experts)
    acc3 = T.GpuTensor.from_host(dev, acc0)
    for s0 in range(0, top_k, 16):
        cnt = min(16, top_k - s0)
        T.batched_marlin_down_axpy(dev, T.GpuTensor.from_host(dev, ad[s0:s0 + cnt]), bank,
                                   T.GpuTensor.from_host(dev, ids_h[s0:s0 + cnt]), T.GpuTensor.from_host(dev, wts_h[s0:s0 + cnt]), acc3, cnt)
    assert rel_err(acc3.to_host(), truth) < TIGHT
    bank.free()


def test_indirect_gemv_reads_the_offset_tables_on_the_device(dev):
    # gemm_tw_marlin_m1_indirect (quantize_indirect.rs:228-253): the expert through packed_offsets[idx] / scales_offsets[idx]
    k, n, experts = 256, 96, 4
    G = k // 32
    packed = [O.synth_packed(k, n, 5300 + 2 * e) for e in range(experts)]
    scales = [O.synth_scales(k, n, 5301 + 2 * e) for e in range(experts)]
    order, gaps_p, gaps_s = [2, 0, 3, 1], [4, 260, 0, 12], [1, 0, 7, 33]
    pbuf, sbuf = np.full(4 * (G * n * 16 + 300), 0xEE, np.uint8), np.full(4 * (G * n + 50), 0x7BFF, np.uint16)
    poff, soff = np.zeros(experts, np.uint32), np.zeros(experts, np.uint32)
    pp = ss = 0
    for e, gp, gs in zip(order, gaps_p, gaps_s):
        pp, ss = pp + gp, ss + gs
        poff[e], soff[e] = pp, ss
        pbuf[pp:pp + G * n * 16] = packed[e]
        sbuf[ss:ss + G * n] = scales[e]
        pp, ss = pp + G * n * 16, ss + G * n
    pd, sd = T.GpuTensor.from_host(dev, pbuf), T.GpuTensor.from_host(dev, sbuf, "f16")
    pod, sod = T.GpuTensor.from_host(dev, poff.view(np.int32), "i32"), T.GpuTensor.from_host(dev, soff.view(np.int32), "i32")
    a32 = O.synth_normal_f32(k, 5350).reshape(1, k)
    ad = T.GpuTensor.from_host(dev, a32)
    c = T.GpuTensor.zeros(dev, (n,), "f32")
    for e in range(experts):
        T.gemm_tw_marlin_m1_indirect(dev, ad, pd, pod, sd, sod, e, c, n, k)
        assert rel_err(c.to_host(), O.gemm_f64(a32, packed[e], scales[e], 1, k, n)[0]) < TIGHT, e
    with pytest.raises(T.DeviceError):
        T.gemm_tw_marlin_m1_indirect(dev, ad, pd, pod, sd, sod, -1, c, n, k)


# ---------------------------------------------------------------- fused projections

def test_plan_description_follows_the_context_options(dev):
    # twm_plan_describe with a context: the options that force a launch form show in the description, and the
    # described form is the one that runs (same result bits as forcing it by hand is not observable from outside;
    # the split factor is: it changes the summation order)
    k, n = 3584, 3584
    assert dev.plan(k, n, 1).startswith("k_gemv4s: 16-column sub-tiles, 8 waves")
    dev.set_option("sub", 1)
    try:
        assert dev.plan(k, n, 1).startswith("k_gemv4: 1 x 64-column tiles per workgroup")
    finally:
        dev.set_option("sub", 0)
    dev.set_option("kernel", 3)
    try:
        assert dev.plan(k, n, 16).startswith("k_stream:")
    finally:
        dev.set_option("kernel", 0)
    dev.set_option("prefill_min_m", 8)
    try:
        assert dev.plan(k, n, 16).startswith("k_prefill:")
    finally:
        dev.set_option("prefill_min_m", 33)
    assert dev.plan(k, n, 16).startswith("k_gemv4s:")
    assert dev.plan(3584, 37888, 1, gated=True).startswith("k_gemv4s: 32-column sub-tiles")
    assert dev.plan(18944, 3584, 1, dtype="f32") == "k_gemv4s: 16-column sub-tiles, 4 waves, 1 K-split; column-lane copy"
    # the drop-in on the reference's arrays: its own planner and options
    assert dev.plan_m1(3584, 37888) == "k_gemv4s: 16-column sub-tiles, 8 waves, 1 K-split; reference arrays"
    dev.set_option("m1_exact", 1)
    try:
        assert dev.plan_m1(3584, 37888).startswith("k_ref_gemv: one thread per column")
    finally:
        dev.set_option("m1_exact", 0)
    dev.set_option("sub", 1)
    dev.set_option("m1_splits", 2)
    try:
        assert dev.plan_m1(18944, 3584) == "k_gemv4: 1 x 64-column tiles per workgroup, 16 waves, 2 K-splits; reference arrays"
    finally:
        dev.set_option("sub", 0)
        dev.set_option("m1_splits", 0)


def test_fusing_handles_equals_fusing_the_arrays(dev):
    # fuse_tw_marlin_n (quantize.rs:1018-1063) on repacked handles: block copies of both copies; the results of every
    # kernel family are bit-identical to those of a handle made from the fused arrays
    k, ns = 1184, [128, 64, 200]      # K not a multiple of 128; the last part is ragged
    host = [(O.synth_packed(k, n, 5400 + i), O.synth_scales(k, n, 5450 + i)) for i, n in enumerate(ns)]
    devp = [(T.GpuTensor.from_host(dev, p), T.GpuTensor.from_host(dev, s, "f16")) for p, s in host]
    parts = [T.MarlinWeight.from_device(dev, p, s, k, n) for (p, s), n in zip(devp, ns)]
    fused = T.MarlinWeight.fuse_n(dev, parts)
    fp, fs = O.fuse_tw_marlin_n(host, k, ns)
    ref = T.MarlinWeight.upload(dev, fp, fs, k, sum(ns))
    assert fused.n == sum(ns) and fused.copies == 3
    for m in (1, 4, 8, 32, 96):
        a16 = O.synth_act_f16(m, k, 5500 + m)
        a_dev = T.GpuTensor.from_host(dev, a16, "f16")
        c1, c2 = T.GpuTensor.zeros(dev, (m, sum(ns)), "f32"), T.GpuTensor.zeros(dev, (m, sum(ns)), "f32")
        T.gemm(dev, fused, a_dev, m, c1)
        T.gemm(dev, ref, a_dev, m, c2)
        assert np.array_equal(c1.to_host(), c2.to_host()), m
    truth = O.gemm_f64(f16_as_f32(O.synth_act_f16(1, k, 5501)), fp, fs, 1, k, sum(ns))
    c = T.GpuTensor.zeros(dev, (1, sum(ns)), "f32")
    T.gemm(dev, fused, T.GpuTensor.from_host(dev, O.synth_act_f16(1, k, 5501), "f16"), 1, c)
    assert rel_err(c.to_host().reshape(1, -1), truth) < TIGHT
    # a part in the middle that is not a multiple of 64 columns wide cannot be block-copied
    with pytest.raises(T.DeviceError):
        T.MarlinWeight.fuse_n(dev, [parts[2], parts[0]])
    # handles with one copy: the fused handle follows the option, missing copies of the parts are built
    dev.set_option("weight_copies", 2)
    one = T.MarlinWeight.fuse_n(dev, parts)
    dev.set_option("weight_copies", 0)
    assert one.copies == 2
    c3 = T.GpuTensor.zeros(dev, (1, sum(ns)), "f32")
    T.gemm(dev, one, T.GpuTensor.from_host(dev, O.synth_act_f16(1, k, 5501), "f16"), 1, c3)
    assert np.array_equal(c3.to_host(), c.to_host())
    for w in parts + [fused, ref, one]:
        w.free()


def test_fused_qkv_and_gate_up_equal_separate_projections(dev):
    # fused-vs-unfused equality, the check the reference makes for F32 weights only
    # (transformer.rs:2230-2287), here on TW-Marlin weights and bit for bit
    h, kv, ffn = 896, 128, 4864
    names = {"wq": (h, h), "wk": (h, kv), "wv": (h, kv), "wo": (h, h), "wg": (h, ffn), "wu": (h, ffn), "wd": (ffn, h)}
    host, pairs = {}, {}
    for i, (nm, (k, n)) in enumerate(names.items()):
        host[nm] = (O.synth_packed(k, n, 300 + i), O.synth_scales(k, n, 400 + i))
        pairs[nm] = (T.GpuTensor.from_host(dev, host[nm][0]), T.GpuTensor.from_host(dev, host[nm][1], "f16"))
    layer = T.TWMarlinWeights(dev, h, kv, ffn, pairs)
    layer.fuse_projections()
    fp, fs = O.fuse_tw_marlin_n([host["wq"], host["wk"], host["wv"]], h, [h, kv, kv])
    assert np.array_equal(layer.wqkv_packed.to_host(), fp) and np.array_equal(layer.wqkv_scales.to_host(), fs)
    rp = layer.repack_for_decode()
    a16 = O.synth_act_f16(1, h, 500)
    a_dev = T.GpuTensor.from_host(dev, a16, "f16")
    # (1) fused GEMV + split kernels, the reference's sequence (generate.rs:2152-2155)
    qkv = T.GpuTensor.zeros(dev, (h + 2 * kv,), "f32")
    T.gemm(dev, rp["qkv"], a_dev, 1, qkv, 1)
    q, kk, v = (T.GpuTensor.zeros(dev, (h,), "f32"), T.GpuTensor.zeros(dev, (kv,), "f32"),
                T.GpuTensor.zeros(dev, (kv,), "f32"))
    T.split_qkv(dev, qkv, q, kk, v, h, kv, 1)
    # (2) the split folded into the GEMV's store
    q2, k2, v2 = (T.GpuTensor.zeros(dev, (h,), "f32"), T.GpuTensor.zeros(dev, (kv,), "f32"),
                  T.GpuTensor.zeros(dev, (kv,), "f32"))
    T.gemm_split(dev, rp["qkv"], a_dev, 1, [q2, k2, v2], [h, kv, kv], 1)
    # (3) three separate projections
    for nm, fused, direct in (("wq", q, q2), ("wk", kk, k2), ("wv", v, v2)):
        k_, n_ = names[nm]
        w = T.MarlinWeight.from_device(dev, pairs[nm][0], pairs[nm][1], k_, n_)
        sep = T.GpuTensor.zeros(dev, (n_,), "f32")
        T.gemm(dev, w, a_dev, 1, sep, 1)
        assert np.array_equal(sep.to_host(), fused.to_host()), nm
        assert np.array_equal(sep.to_host(), direct.to_host()), nm
        truth = O.gemm_f64(f16_as_f32(a16), host[nm][0], host[nm][1], 1, k_, n_)[0]
        assert rel_err(sep.to_host(), truth) < TIGHT
    # gate+up with M = 3 and automatic split-K
    a3 = O.synth_act_f16(3, h, 501)
    a3d = T.GpuTensor.from_host(dev, a3, "f16")
    g, u = T.GpuTensor.zeros(dev, (3, ffn), "f32"), T.GpuTensor.zeros(dev, (3, ffn), "f32")
    T.gemm_split(dev, rp["gate_up"], a3d, 3, [g, u], [ffn, ffn])
    tg = O.gemm_f64(f16_as_f32(a3), host["wg"][0], host["wg"][1], 3, h, ffn)
    tu = O.gemm_f64(f16_as_f32(a3), host["wu"][0], host["wu"][1], 3, h, ffn)
    assert rel_err(g.to_host(), tg) < TIGHT and rel_err(u.to_host(), tu) < TIGHT
    with pytest.raises(T.DeviceError):
        T.gemm_split(dev, rp["gate_up"], a3d, 3, [g, u], [ffn, ffn - 1])


def test_layer_container_carries_norms_and_adds_biases(dev):
    # TWMarlinWeights (quantize.rs:1067-1086) with its norm vectors and optional Q/K/V biases: qkv() is the fused GEMV of
    # the decode step with the biases of generate.rs:2162-2165 added in the store; a layer without biases gives the plain sums
    h, kv, ffn = 640, 128, 1280
    names = {"wq": (h, h), "wk": (h, kv), "wv": (h, kv), "wo": (h, h), "wg": (h, ffn), "wu": (h, ffn), "wd": (ffn, h)}
    host = {nm: (O.synth_packed(k, n, 1600 + i), O.synth_scales(k, n, 1700 + i)) for i, (nm, (k, n)) in enumerate(names.items())}
    pairs = {nm: (T.GpuTensor.from_host(dev, p), T.GpuTensor.from_host(dev, s_, "f16")) for nm, (p, s_) in host.items()}
    bq, bk, bv = (O.synth_normal_f32(x, 1800 + j) for j, x in enumerate((h, kv, kv)))
    norm = T.GpuTensor.from_host(dev, np.ones(h, np.float32))
    layer = T.TWMarlinWeights(dev, h, kv, ffn, pairs, attn_norm=norm, ffn_norm=norm,
                              bq=T.GpuTensor.from_host(dev, bq), bk=T.GpuTensor.from_host(dev, bk), bv=T.GpuTensor.from_host(dev, bv))
    plain = T.TWMarlinWeights(dev, h, kv, ffn, pairs)
    assert layer.attn_norm is norm and plain.bq is None
    a16 = O.synth_act_f16(1, h, 1900)
    ad = T.GpuTensor.from_host(dev, a16, "f16")
    outs = {}
    for label, lw in (("biased", layer), ("plain", plain)):
        lw.repack_for_decode()
        q, kk, v = (T.GpuTensor.zeros(dev, (x,), "f32") for x in (h, kv, kv))
        lw.qkv(ad, 1, q, kk, v)
        outs[label] = [t.to_host() for t in (q, kk, v)]
    for got_b, got_p, nm, b in zip(outs["biased"], outs["plain"], ("wq", "wk", "wv"), (bq, bk, bv)):
        k_, n_ = names[nm]
        truth = O.gemm_f64(f16_as_f32(a16), host[nm][0], host[nm][1], 1, k_, n_)[0]
        assert rel_err(got_p, truth) < TIGHT
        assert np.array_equal(got_b, got_p + b)      # one f32 add on top of the unbiased result


@pytest.mark.parametrize("m,splits", [(1, 0), (1, 4), (3, 0), (12, 0), (12, 2), (40, 0), (70, 2)])
def test_gemm_split_bias_adds_bq_bk_bv_in_the_store(dev, m, splits):
    # q = gemv + bq etc. (the add the reference makes in its bias + RoPE kernel): one f32 add per element on
    # top of the unbiased result, so the comparison with numpy's f32 add is bit for bit, on every kernel
    h, kv = 640, 128
    ns = [h, kv, kv]
    packed, scales, a16 = synth(h, sum(ns), m, 970 + m)
    w = T.MarlinWeight.upload(dev, packed, scales, h, sum(ns))
    ad = T.GpuTensor.from_host(dev, a16, "f16")
    plain = [T.GpuTensor.zeros(dev, (m, n), "f32") for n in ns]
    T.gemm_split(dev, w, ad, m, plain, ns, splits)
    bias_h = [O.synth_normal_f32(n, 980 + i) for i, n in enumerate(ns)]
    bias_h[1] = None                                             # K without a bias
    bias_d = [T.GpuTensor.from_host(dev, b) if b is not None else None for b in bias_h]
    outs = [T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32)) for n in ns]
    T.gemm_split(dev, w, ad, m, outs, ns, splits, biases=bias_d)
    for o, p, b in zip(outs, plain, bias_h):
        want = p.to_host() if b is None else (p.to_host() + b[None, :]).astype(np.float32)
        assert np.array_equal(o.to_host(), want)
    w.free()


def test_gemm_split_bias_with_empty_k(dev):
    ns = [64, 32]
    w = T.MarlinWeight.upload(dev, np.zeros(0, np.uint8), np.zeros(0, np.uint16), 0, 96)
    a = T.GpuTensor.zeros(dev, (1,), "f16")
    b0 = O.synth_normal_f32(64, 990)
    outs = [T.GpuTensor.from_host(dev, np.full((2, n), np.nan, np.float32)) for n in ns]
    T.gemm_split(dev, w, a, 2, outs, ns, 0, biases=[T.GpuTensor.from_host(dev, b0), None])
    assert np.array_equal(outs[0].to_host(), np.stack([b0, b0])) and not outs[1].to_host().any()
    w.free()


@pytest.mark.parametrize("m", [12, 24, 40, 130])
def test_gemm_split_batched_and_prefill_rows(dev, m):
    # segment stores of the streaming kernel (M = 12, 24), of the MFMA GEMM (M = 40, 130) and of the
    # split-K reduce kernel: gemm_split equals slicing the fused result, bit for bit, for every split factor
    k, ns = 1184, [96, 40, 168]
    n = sum(ns)
    packed, scales, a16 = synth(k, n, m, 7000 + m)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    a_dev = T.GpuTensor.from_host(dev, a16, "f16")
    truth = gemm_truth(a16, packed, scales, m, k, n)
    for splits in (0, 1, 3):
        whole = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))
        T.gemm(dev, w, a_dev, m, whole, splits)
        got = whole.to_host()
        assert rel_err(got, truth) < TIGHT, splits
        parts = [T.GpuTensor.from_host(dev, np.full((m, ni), np.nan, np.float32)) for ni in ns]
        T.gemm_split(dev, w, a_dev, m, parts, ns, splits)
        off = 0
        for pt, ni in zip(parts, ns):
            assert np.array_equal(pt.to_host(), got[:, off:off + ni]), (splits, off)
            off += ni
    w.free()


# ---------------------------------------------------------------- graph capture / replay

def test_layer_graph_replays_match_eager(dev):
    # the four projections of a Qwen-0.5B-shaped layer as one graph; replayed several times
    # with eager work and synchronisations in between, every replay checked against eager
    shapes = {"qkv": (896, 1152), "o": (896, 896), "gate_up": (896, 9728), "down": (4864, 896)}
    ws, acts, outs, eager = {}, {}, {}, {}
    for i, (nm, (k, n)) in enumerate(shapes.items()):
        p, s, a16 = synth(k, n, 1, 600 + i)
        ws[nm] = T.MarlinWeight.upload(dev, p, s, k, n)
        acts[nm] = T.GpuTensor.from_host(dev, a16, "f16")
        outs[nm] = T.GpuTensor.zeros(dev, (n,), "f32")
        T.gemm(dev, ws[nm], acts[nm], 1, outs[nm])
        eager[nm] = outs[nm].to_host()
        truth = O.gemm_f64(f16_as_f32(a16), p, s, 1, k, n)[0]
        assert rel_err(eager[nm], truth) < TIGHT

    def body():
        for nm in shapes:
            T.gemm(dev, ws[nm], acts[nm], 1, outs[nm])

    graph = T.GraphCapture.record_with_device(dev, body)
    for rep in range(4):
        for nm, (k, n) in shapes.items():
            outs[nm].copy_from_host(np.full(n, np.nan, np.float32))
        graph.replay()
        dev.synchronize()
        for nm in shapes:
            assert np.array_equal(outs[nm].to_host(), eager[nm]), (rep, nm)
        T.gemm(dev, ws["down"], acts["down"], 1, outs["down"], 7)      # eager work between replays
        dev.synchronize()
    graph.destroy()


def test_graph_of_fused_epilogues_and_expert_banks(dev):
    # SwiGLU GEMV (split-K inside the launch), biased QKV split, the MoE block (fused GEGLU, then down + weighted
    # sum onto an accumulator that the graph itself clears) and the argmax, captured together and replayed with
    # eager work in between; every replay must reproduce the eager results bit for bit
    h, ffn, kv = 2048, 96, 64
    gp, gs = O.synth_packed(h, ffn, 1100), O.synth_scales(h, ffn, 1101)
    up, us = O.synth_packed(h, ffn, 1102), O.synth_scales(h, ffn, 1103)
    wgu = T.MarlinWeight.gate_up(dev, (T.GpuTensor.from_host(dev, gp), T.GpuTensor.from_host(dev, gs, "f16")),
                                 (T.GpuTensor.from_host(dev, up), T.GpuTensor.from_host(dev, us, "f16")), h, ffn)
    qp, qs, a16 = synth(h, h + 2 * kv, 1, 1104)
    wqkv = T.MarlinWeight.upload(dev, qp, qs, h, h + 2 * kv)
    x = T.GpuTensor.from_host(dev, a16, "f16")
    biases = [T.GpuTensor.from_host(dev, O.synth_normal_f32(n, 1105 + i)) for i, n in enumerate((h, kv, kv))]
    dim, experts, top_k = 64, 6, 4
    gub, _, _ = make_bank(dev, h, 2 * dim, experts, 1110, pair=True)
    db, _, _ = make_bank(dev, dim, h, experts, 1130)
    ids = T.GpuTensor.from_host(dev, np.array([4, 0, 5, 2], np.float32))
    wts = T.GpuTensor.from_host(dev, np.array([0.4, 0.3, 0.2, 0.1], np.float32))
    act = T.GpuTensor.zeros(dev, (ffn,), "f32")
    q, kk, v = (T.GpuTensor.zeros(dev, (n,), "f32") for n in (h, kv, kv))
    geglu = T.GpuTensor.zeros(dev, (top_k, dim), "f32")
    moe_acc = T.GpuTensor.zeros(dev, (h,), "f32")
    token = T.GpuTensor.from_host(dev, np.zeros(1, np.int32))

    def body():
        T.gemm_swiglu(dev, wgu, x, 1, act)
        T.gemm_split(dev, wqkv, x, 1, [q, kk, v], [h, kv, kv], 0, biases=biases)
        T.batched_marlin_gate_up(dev, x, gub, ids, geglu, top_k, act=T.ACT_GEGLU)
        dev._l.twm_memset_zero(dev.handle, moe_acc.ptr, h * 4)
        T.batched_marlin_down_axpy(dev, geglu, db, ids, wts, moe_acc, top_k)
        T.argmax(dev, moe_acc, token, 1, h)

    body()
    dev.synchronize()
    bufs = {"act": act, "q": q, "k": kk, "v": v, "geglu": geglu, "moe": moe_acc, "token": token}
    eager = {nm: t.to_host().copy() for nm, t in bufs.items()}
    assert int(eager["token"][0]) == int(np.argmax(eager["moe"])) and np.isfinite(eager["moe"]).all()
    graph = T.GraphCapture.record_with_device(dev, body)
    for rep in range(4):
        for nm, t in bufs.items():
            if nm != "token":
                t.copy_from_host(np.full(t.numel, np.nan, np.float32))
        graph.replay()
        dev.synchronize()
        for nm, t in bufs.items():
            assert np.array_equal(t.to_host(), eager[nm]), (rep, nm)
        T.gemm_swiglu(dev, wgu, x, 1, act, 3)                 # eager work between replays
        dev.synchronize()
    graph.destroy()
    for wobj in (wgu, wqkv, gub, db):
        wobj.free()


def test_graph_of_batched_and_prefill_launches():
    # The multi-kernel paths (f32 -> f16 conversion, split-K partials + ordered reduce) captured in a graph
    # as their FIRST use in a fresh context, then replayed with eager work in between; every replay must
    # reproduce the eager result bit for bit (no memset nodes, no allocation, deterministic sums).
    with T.WarpDevice(0) as d:
        k, n = 2048, 320
        packed, scales, a16 = synth(k, n, 130, 8100)
        w = T.MarlinWeight.upload(d, packed, scales, k, n)
        cases = []
        for m, a_f32, splits in ((12, False, 3), (24, True, 0), (40, True, 2), (130, False, 0)):
            bits = a16[:m]
            a_dev = T.GpuTensor.from_host(d, f16_as_f32(bits)) if a_f32 else T.GpuTensor.from_host(d, bits, "f16")
            cases.append((m, a_dev, T.GpuTensor.zeros(d, (m, n), "f32"), splits, bits))

        def body():
            for m, a_dev, c, splits, _ in cases:
                T.gemm(d, w, a_dev, m, c, splits)

        graph = T.GraphCapture.record_with_device(d, body)
        graph.replay()
        d.synchronize()
        first = [c.to_host() for _, _, c, _, _ in cases]
        for (m, _, _, _, bits), got in zip(cases, first):
            assert rel_err(got, gemm_truth(bits, packed, scales, m, k, n)) < TIGHT, m
        for rep in range(3):
            for _, _, c, _, _ in cases:
                c.copy_from_host(np.full(c.shape, np.nan, np.float32))
            body()                                   # eager, between replays
            d.synchronize()
            for (_, _, c, _, _), want in zip(cases, first):
                assert np.array_equal(c.to_host(), want), ("eager", rep)
                c.copy_from_host(np.full(c.shape, np.nan, np.float32))
            graph.replay()
            d.synchronize()
            for (_, _, c, _, _), want in zip(cases, first):
                assert np.array_equal(c.to_host(), want), ("replay", rep)
        graph.destroy()
        w.free()


def test_instruction_mix_probe_runs_and_orders_its_rows(dev):
    # the profiling aid behind bench.py --mfma-mix: matrix instructions alone run near the FP16 peak, every added part
    # of a prefill block's instruction mix costs throughput, and bad arguments are errors, not launches
    import ctypes as C
    lib, tf = T._lib.load(), C.c_float()
    got = {}
    for parts in (0, 7):
        assert lib.twm_debug_mfma_mix(dev.handle, 0, parts, 1, 4096, C.byref(tf)) == T._lib.OK, lib.twm_last_error()
        got[parts] = tf.value
    assert 1500 < got[0] < 2600 and 500 < got[7] < got[0], got
    assert lib.twm_debug_mfma_mix(dev.handle, 1, 19, 1, 4096, C.byref(tf)) == T._lib.OK, lib.twm_last_error()
    assert 500 < tf.value < 2600, tf.value
    assert lib.twm_debug_mfma_mix(dev.handle, 0, 4, 1, 4096, C.byref(tf)) == T._lib.UNSUPPORTED_OP
    assert lib.twm_debug_mfma_mix(dev.handle, 0, 0, 3, 4096, C.byref(tf)) == T._lib.SHAPE_ERROR
    assert lib.twm_debug_mfma_mix(dev.handle, 1, 0, 2, 4096, C.byref(tf)) == T._lib.SHAPE_ERROR
    assert lib.twm_debug_mfma_mix(dev.handle, 0, 0, 1, 100, C.byref(tf)) == T._lib.SHAPE_ERROR


def test_gemm_with_f16_result_rows(dev):
    # twm_gemm_f16out = the f32 result of twm_gemm rounded to nearest even, bit for bit: decode rows, batched rows, prefill
    # rows, f16 and f32 activations, and a row count whose f32 results exceed the staging half of the scratch (row blocks)
    for k, n, ms in ((256, 200, (1, 3, 8, 32, 100)), (3584, 37888, (1, 300))):
        packed, scales = O.synth_packed(k, n, 1700), O.synth_scales(k, n, 1701)
        w = T.MarlinWeight.upload(dev, packed, scales, k, n)
        for m in ms:
            a16 = O.synth_act_f16(m, k, 1710 + m)
            for a_f32 in (False, True):
                a_dev = T.GpuTensor.from_host(dev, f16_as_f32(a16)) if a_f32 else T.GpuTensor.from_host(dev, a16, "f16")
                c32 = T.GpuTensor.from_host(dev, np.full((m, n), np.nan, np.float32))
                c16 = T.GpuTensor.from_host(dev, np.full((m, n), 0x7E00, np.uint16), "f16")     # NaN canary
                T.gemm(dev, w, a_dev, m, c32)
                T.gemm_f16out(dev, w, a_dev, m, c16)
                want = c32.to_host().astype(np.float16).view(np.uint16)
                got = c16.to_host().view(np.uint16).reshape(m, n)
                if n == 200:
                    assert np.array_equal(got, want), (k, n, m, a_f32)
                else:
                    # (row blocks and half the scratch may mean another K-split than twm_gemm's on all rows at once: the
                    # f32 sums then differ in their last bits, and a few of them round to the neighbouring f16)
                    gf, wf = got.view(np.float16).astype(np.float32), want.view(np.float16).astype(np.float32)
                    assert (got != want).mean() < 1e-3 and np.abs(gf - wf).max() <= 1e-3 * np.abs(wf).max(), (k, n, m, a_f32)
                for t in (a_dev, c32, c16):
                    t.free()
        w.free()
    # in a captured graph (the call allocates nothing), replayed with eager work in between; empty calls are no-ops
    k, n = 512, 320
    packed, scales = O.synth_packed(k, n, 1720), O.synth_scales(k, n, 1721)
    w = T.MarlinWeight.upload(dev, packed, scales, k, n)
    acts = {m: T.GpuTensor.from_host(dev, O.synth_act_f16(m, k, 1730 + m), "f16") for m in (1, 8, 40)}
    outs = {m: T.GpuTensor.from_host(dev, np.zeros((m, n), np.uint16), "f16") for m in acts}
    eager = {}
    for m in acts:
        T.gemm_f16out(dev, w, acts[m], m, outs[m])
        eager[m] = outs[m].to_host().view(np.uint16).copy()
    graph = T.GraphCapture.record_with_device(dev, lambda: [T.gemm_f16out(dev, w, acts[m], m, outs[m]) for m in acts])
    for rep in range(3):
        for m in acts:
            outs[m].copy_from_host(np.full((m, n), 0x7E00, np.uint16))
        graph.replay()
        dev.synchronize()
        for m in acts:
            assert np.array_equal(outs[m].to_host().view(np.uint16), eager[m]), (rep, m)
        T.gemm_f16out(dev, w, acts[8], 8, outs[8], 2)        # eager work between replays
        dev.synchronize()
    graph.destroy()
    T.gemm_f16out(dev, w, acts[1], 0, outs[1])
    lib = T._lib.load()
    assert lib.twm_gemm_f16out(dev.handle, None, None, T._lib.F16, 1, None, 0) == T._lib.INVALID_HANDLE
    assert lib.twm_gemm_f16out(dev.handle, w.handle, acts[1].ptr, 7, 1, outs[1].ptr, 0) == T._lib.UNSUPPORTED_OP
    w.free()

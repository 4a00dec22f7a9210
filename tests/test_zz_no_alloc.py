"""twm_gemm_tw_marlin_m1_noalloc (the entry point for callers that cannot allocate) against twm_gemm_tw_marlin_m1,
through the C ABI: bit-identical outputs, on calls in a row, the later ones with smaller inputs.  The first two shapes
are ones whose default plan cuts K over workgroups, so their launches park partial sums in the library's static scratch
and count arrivals there; before every call the whole scratch is poisoned (every byte 0xFF: NaN partial sums, counters
at 2^32 - 1), so that a call which relied on what was left there, or whose scratch address was wrong, fails."""
import ctypes as C

import numpy as np
import pytest

import tensorwarp_amd as T
from oracle import twm_oracle as O

pytestmark = pytest.mark.gpu


def f16_as_f32(bits):
    return bits.view(np.float16).astype(np.float32)


def test_noalloc_entry_point_matches_the_context_entry_point():
    lib = T._lib.load()
    with T.WarpDevice(0) as dev:
        stream = lib.twm_ctx_stream(dev.handle)
        # 32768 -> 100 (ragged N): four K-splits through the scratch; then the smaller 16384 -> 256: two; then a shape
        # that does not split at all
        for k, n, splits in ((32768, 100, 4), (16384, 256, 2), (896, 1152, 1)):
            print("no-alloc case K=%d N=%d" % (k, n), flush=True)
            buf = C.create_string_buffer(256)
            assert lib.twm_plan_describe_m1(None, k, n, buf, 256) == T._lib.OK
            assert ("%d K-split" % splits) in buf.value.decode(), buf.value
            packed, scales = O.synth_packed(k, n, 9000 + n), O.synth_scales(k, n, 9001 + n)
            a = f16_as_f32(O.synth_act_f16(1, k, 9002 + n)) * np.float32(1.25) + np.float32(1e-3)
            pd, sd, ad = T.GpuTensor.from_host(dev, packed), T.GpuTensor.from_host(dev, scales, "f16"), T.GpuTensor.from_host(dev, a)
            want = T.GpuTensor.from_host(dev, np.full(n, np.nan, np.float32))
            got = T.GpuTensor.from_host(dev, np.full(n, np.nan, np.float32))
            T.gemm_tw_marlin_m1(dev, ad, pd, sd, want, n, k)
            assert lib.twm_noalloc_scratch_fill(stream, 0xFF) == T._lib.OK, lib.twm_last_error()
            rc = lib.twm_gemm_tw_marlin_m1_noalloc(stream, ad.ptr, pd.ptr, sd.ptr, got.ptr, n, k)
            assert rc == T._lib.OK, lib.twm_last_error()
            dev.synchronize()
            w, g = want.to_host(), got.to_host()
            assert not np.isnan(g).any()
            assert np.array_equal(g, w), (k, n)
            truth = O.gemm_f64(a.reshape(1, k), packed, scales, 1, k, n)[0]
            denom = np.maximum(np.abs(truth), 1e-3 * np.abs(truth).max())
            assert (np.abs(g - truth) / denom).max() < 2e-4
            for t in (pd, sd, ad, want, got):
                t.free()
        # sizes beyond the stated maximum are refused before anything is launched
        assert lib.twm_gemm_tw_marlin_m1_noalloc(stream, None, None, None, None, (1 << 20) + 64, 64) == T._lib.SHAPE_ERROR
        assert b"beyond" in lib.twm_last_error()
        assert lib.twm_gemm_tw_marlin_m1_noalloc(stream, None, None, None, None, 64, 100) == T._lib.SHAPE_ERROR

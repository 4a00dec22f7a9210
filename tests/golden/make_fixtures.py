"""Writes the golden fixtures in this directory.

The vectors come from a numpy restatement of the TW-Marlin format that is
independent of the C oracle: vectorised numpy float32 / float16 arithmetic
(numpy's float16 is IEEE binary16 with round-to-nearest-even) and float64
matmul.  Both the C oracle and the HIP path are checked against these files, so
a mistake shared by oracle and kernel (nibble order, group stride, zero point)
shows up as a fixture mismatch.

Format facts restated here (reference: crates/loader/src/gemma_moe_q4.rs:218-254,
crates/kernels/src/quantize.rs:1209-1238):
  packed u8[G][N][16], byte i of a record = q[2i] | q[2i+1] << 4
  scales f16[G][N]
  quantizer: amax/7, inv = 7/amax, q = clamp(round_half_away(v*inv) + 8, 0, 15)
  dequant:   w = f32(scale_f16) * (q - 8)

Run:  python tests/golden/make_fixtures.py      (needs numpy only)
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def round_half_away(x):
    x = np.asarray(x, np.float32)
    return np.copysign(np.floor(np.abs(x) + np.float32(0.5)), x).astype(np.float32)


def np_quantize_nk(w_nk):
    """w_nk: [N, K] float32 -> packed u8[G, N, 16], scales float16 [G, N]."""
    n, k = w_nk.shape
    g = k // 32
    v = w_nk.astype(np.float32).reshape(n, g, 32)
    amax = np.max(np.abs(v), axis=2)                       # [N, G]
    scale = (amax / np.float32(7.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = np.where(scale != 0, np.float32(7.0) / amax, np.float32(0.0)).astype(np.float32)
    q = round_half_away(v * inv[:, :, None]).astype(np.int32) + 8
    q = np.clip(q, 0, 15).astype(np.uint8)                 # [N, G, 32]
    byts = (q[:, :, 0::2] | (q[:, :, 1::2] << 4)).astype(np.uint8)   # [N, G, 16]
    packed = np.ascontiguousarray(byts.transpose(1, 0, 2))           # [G, N, 16]
    scales = np.ascontiguousarray(scale.T).astype(np.float16)        # RNE
    return packed, scales


def np_nibbles(packed_gn16):
    """[G, N, 16] bytes -> q int32 [K, N]."""
    g, n, _ = packed_gn16.shape
    lo = (packed_gn16 & 0xF).astype(np.int32)
    hi = (packed_gn16 >> 4).astype(np.int32)
    q = np.empty((g, n, 32), np.int32)
    q[:, :, 0::2] = lo
    q[:, :, 1::2] = hi
    return np.ascontiguousarray(q.transpose(0, 2, 1)).reshape(g * 32, n)


def np_dequant_f32(packed_gn16, scales_gn):
    q = np_nibbles(packed_gn16)
    s = np.repeat(scales_gn.astype(np.float32), 32, axis=0)   # [K, N]
    return (s * (q - 8).astype(np.float32)).astype(np.float32)


def np_dequant_f16(packed_gn16, scales_gn):
    return np_dequant_f32(packed_gn16, scales_gn).astype(np.float16)


def lcg_weights(k, n):
    # the reference test's generator (quantize.rs:3618-3620), laid out [K, N]
    i = np.arange(k * n, dtype=np.int64)
    return (((i * 17 + 3) % 101).astype(np.float32) * np.float32(0.02) - np.float32(1.0)).reshape(k, n)


def lcg_act(m, k):
    # quantize.rs:3054-3056
    i = np.arange(m * k, dtype=np.int64)
    return (((i * 7 + 13) % 100).astype(np.float32) * np.float32(0.01) - np.float32(0.5)).reshape(m, k)


def make_case(name, k, n, m, rng, synthetic):
    if synthetic:
        # benchmark-style synthetic: nibbles uniform 0..15, scales f16(|N(0,1)|*0.02)
        packed = rng.integers(0, 256, size=(k // 32, n, 16), dtype=np.uint8)
        scales = (np.abs(rng.standard_normal((k // 32, n))) * 0.02).astype(np.float32).astype(np.float16)
        a16 = rng.standard_normal((m, k)).astype(np.float32).astype(np.float16)
        w_kn = None
    else:
        w_kn = lcg_weights(k, n)
        packed, scales = np_quantize_nk(np.ascontiguousarray(w_kn.T))
        a16 = lcg_act(m, k).astype(np.float16)
    a32 = a16.astype(np.float32)
    deq32 = np_dequant_f32(packed, scales)
    deq16 = np_dequant_f16(packed, scales)
    c64 = a32.astype(np.float64) @ deq32.astype(np.float64)
    out = dict(k=np.int64(k), n=np.int64(n), m=np.int64(m),
               packed=packed.reshape(-1), scales=scales.view(np.uint16).reshape(-1),
               a_f16=a16.view(np.uint16), dequant_f32=deq32,
               dequant_f16=deq16.view(np.uint16), c_f64=c64)
    if w_kn is not None:
        out["w_kn"] = w_kn
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


def main():
    rng = np.random.default_rng(20240607)
    make_case("lcg_k64_n8_m1", 64, 8, 1, rng, synthetic=False)
    make_case("lcg_k128_n64_m4", 128, 64, 4, rng, synthetic=False)
    make_case("synth_k128_n64_m1", 128, 64, 1, rng, synthetic=True)
    make_case("synth_k256_n80_m5", 256, 80, 5, rng, synthetic=True)    # N not a multiple of 64
    make_case("synth_k160_n33_m17", 160, 33, 17, rng, synthetic=True)  # ragged N, G not a multiple of 4

    # f16 conversion corner cases: value, expected bits (numpy RNE)
    vals = np.array([0.0, -0.0, 1.0, -2.5, 65504.0, 65519.9, 65520.0, 1e6, -1e6,
                     5.9604645e-08, 2.9802322e-08, 2.9802326e-08, 8.9406967e-08,
                     6.1035156e-05, 6.0975552e-05, 1.0009766, 1.00048828125, 1.00146484375,
                     0.0999755859375, 3.1415927, np.inf, -np.inf], np.float32)
    with np.errstate(over="ignore"):
        bits = vals.astype(np.float16).view(np.uint16)
    np.savez_compressed(os.path.join(HERE, "f16_corners.npz"), vals=vals, bits=bits)


if __name__ == "__main__":
    main()

"""ctypes binding of the C oracle (oracle/twm_oracle.c -> libtwm_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtwm_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force or not os.path.exists(_SO):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _lib.twmo_f16_to_f32.restype = C.c_float
        _lib.twmo_f16_to_f32.argtypes = [C.c_uint16]
        _lib.twmo_f32_to_f16.restype = C.c_uint16
        _lib.twmo_f32_to_f16.argtypes = [C.c_float]
        _lib.twmo_gemv_ref_order_mt.restype = C.c_int
        _lib.twmo_max_threads.restype = C.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def f16_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().twmo_f16_to_f32_array(_p(h), _p(out), C.c_size_t(h.size))
    return out


def f32_to_f16(f):
    f = _c(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().twmo_f32_to_f16_array(_p(f), _p(out), C.c_size_t(f.size))
    return out


def quantize_tw_marlin_nk(data_nk, k, n):
    """cpu_quantize_tw_marlin: data row-major [N, K] f32 -> (packed u8[G*N*16], scales u16[G*N])."""
    data = _c(data_nk, np.float32).reshape(n, k)
    g = k // 32
    packed = np.zeros(g * n * 16, np.uint8)
    scales = np.zeros(g * n, np.uint16)
    lib().twmo_quantize_tw_marlin_nk(_p(data), C.c_uint32(k), C.c_uint32(n), _p(packed), _p(scales))
    return packed, scales


def quantize_q4_col_major_nk(data_nk, k, n):
    data = _c(data_nk, np.float32).reshape(n, k)
    out = np.zeros((k // 32) * n * 20, np.uint8)
    lib().twmo_quantize_q4_col_major_nk(_p(data), C.c_uint32(k), C.c_uint32(n), _p(out))
    return out


def quantize_weights_q4_0_kn(w_kn, k, n, block_major=False):
    w = _c(w_kn, np.float32).reshape(k, n)
    out = np.zeros((k // 32) * n * 20, np.uint8)
    lib().twmo_quantize_weights_q4_0_kn(_p(w), C.c_uint32(k), C.c_uint32(n), _p(out),
                                        C.c_int(1 if block_major else 0))
    return out


def q4_0_roundtrip(x):
    x = _c(x, np.float32)
    out = np.zeros_like(x)
    lib().twmo_q4_0_roundtrip(_p(x), _p(out), C.c_size_t(x.size))
    return out


def reorder_to_tw_marlin(q4, k, n):
    q4 = _c(q4, np.uint8)
    g = k // 32
    packed = np.zeros(g * n * 16, np.uint8)
    scales = np.zeros(g * n, np.uint16)
    lib().twmo_reorder_to_tw_marlin(_p(q4), C.c_uint32(k), C.c_uint32(n), _p(packed), _p(scales))
    return packed, scales


def fuse_tw_marlin_n(mats, k, ns):
    """mats: list of (packed, scales); returns fused (packed, scales)."""
    cnt = len(mats)
    g = k // 32
    total = int(sum(ns))
    pk = [_c(m[0], np.uint8) for m in mats]
    sc = [_c(m[1], np.uint16) for m in mats]
    pp = (C.c_void_p * cnt)(*[p.ctypes.data for p in pk])
    sp = (C.c_void_p * cnt)(*[s.ctypes.data for s in sc])
    nsa = np.asarray(ns, np.uint32)
    packed = np.zeros(g * total * 16, np.uint8)
    scales = np.zeros(g * total, np.uint16)
    lib().twmo_fuse_tw_marlin_n(pp, sp, C.c_uint32(k), _p(nsa), C.c_uint32(cnt), _p(packed), _p(scales))
    return packed, scales


def split_qkv(qkv, h, kv, batch):
    qkv = _c(qkv, np.float32)
    q = np.zeros(batch * h, np.float32)
    kk = np.zeros(batch * kv, np.float32)
    v = np.zeros(batch * kv, np.float32)
    lib().twmo_split_qkv(_p(qkv), _p(q), _p(kk), _p(v), C.c_uint32(h), C.c_uint32(kv), C.c_uint32(batch))
    return q, kk, v


def split_gate_up(gu, ffn, batch):
    gu = _c(gu, np.float32)
    g = np.zeros(batch * ffn, np.float32)
    u = np.zeros(batch * ffn, np.float32)
    lib().twmo_split_gate_up(_p(gu), _p(g), _p(u), C.c_uint32(ffn), C.c_uint32(batch))
    return g, u


def silu_mul(gate, up):
    gate, up = _c(gate, np.float32), _c(up, np.float32)
    out = np.zeros(gate.size, np.float32)
    lib().twmo_silu_mul(_p(gate), _p(up), _p(out), C.c_size_t(gate.size))
    return out.reshape(gate.shape)


def gelu_mul(gate, up):
    gate, up = _c(gate, np.float32), _c(up, np.float32)
    out = np.zeros(gate.size, np.float32)
    lib().twmo_gelu_mul(_p(gate), _p(up), _p(out), C.c_size_t(gate.size))
    return out.reshape(gate.shape)


def bank_gemv_f64(a, packed_bank, scales_bank, ids, k, n):
    """batched_marlin_gate_up (moe_batched_marlin.rs:20-74) as f64 truth: row s = A_s x dequant(expert ids[s]).
    a: [1, K] shared or [slots, K]; packed_bank [E][G*N*16], scales_bank [E][G*N]; invalid ids give zeros."""
    a = np.asarray(a, np.float32).reshape(-1, k)
    out = np.zeros((len(ids), n), np.float64)
    for s, e in enumerate(ids):
        e = int(e)
        if 0 <= e < len(packed_bank):
            row = a[s if a.shape[0] > 1 else 0].reshape(1, k)
            out[s] = gemm_f64(row, packed_bank[e], scales_bank[e], 1, k, n)[0]
    return out


def pair_gate_up(gate_packed, gate_scales, up_packed, up_scales, k, ffn):
    po = np.zeros((k // 32) * 2 * ffn * 16, np.uint8)
    so = np.zeros((k // 32) * 2 * ffn, np.uint16)
    lib().twmo_pair_gate_up(_p(_c(gate_packed, np.uint8)), _p(_c(gate_scales, np.uint16)),
                            _p(_c(up_packed, np.uint8)), _p(_c(up_scales, np.uint16)),
                            C.c_uint32(k), C.c_uint32(ffn), _p(po), _p(so))
    return po, so


def argmax(x, rows, cols):
    x = _c(x, np.float32)
    out = np.zeros(rows, np.int32)
    lib().twmo_argmax(_p(x), C.c_uint32(rows), C.c_uint32(cols), _p(out))
    return out


def dequant_f32(packed, scales, k, n):
    out = np.empty((k, n), np.float32)
    lib().twmo_dequant_f32(_p(_c(packed, np.uint8)), _p(_c(scales, np.uint16)),
                           C.c_uint32(k), C.c_uint32(n), _p(out))
    return out


def dequant_f16(packed, scales, k, n):
    out = np.empty((k, n), np.uint16)
    lib().twmo_dequant_f16(_p(_c(packed, np.uint8)), _p(_c(scales, np.uint16)),
                           C.c_uint32(k), C.c_uint32(n), _p(out))
    return out


def dequant_q4_0_to_f16(q4, k, n):
    out = np.empty((k, n), np.uint16)
    lib().twmo_dequant_q4_0_to_f16(_p(_c(q4, np.uint8)), C.c_uint32(k), C.c_uint32(n), _p(out))
    return out


def cpu_gemm(a, b, m, n, k):
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    c = np.zeros((m, n), np.float32)
    lib().twmo_cpu_gemm(_p(a), _p(b), _p(c), C.c_size_t(m), C.c_size_t(n), C.c_size_t(k))
    return c


def gemv_ref_order(a, packed, scales, m, k, n, splits=1):
    a = _c(a, np.float32)
    c = np.zeros((m, n), np.float32)
    lib().twmo_gemv_ref_order(_p(a), _p(_c(packed, np.uint8)), _p(_c(scales, np.uint16)), _p(c),
                              C.c_uint32(m), C.c_uint32(k), C.c_uint32(n), C.c_uint32(splits))
    return c


def gemv_ref_order_mt(a, packed, scales, m, k, n):
    a = _c(a, np.float32)
    c = np.zeros((m, n), np.float32)
    used = lib().twmo_gemv_ref_order_mt(_p(a), _p(_c(packed, np.uint8)), _p(_c(scales, np.uint16)),
                                        _p(c), C.c_uint32(m), C.c_uint32(k), C.c_uint32(n))
    return c, used


def gemm_tile_order(a, packed, scales, m, k, n):
    a = _c(a, np.float32)
    c = np.zeros((m, n), np.float32)
    lib().twmo_gemm_tile_order(_p(a), _p(_c(packed, np.uint8)), _p(_c(scales, np.uint16)), _p(c),
                               C.c_uint32(m), C.c_uint32(k), C.c_uint32(n))
    return c


def gemm_f64(a, packed, scales, m, k, n):
    a = _c(a, np.float32)
    c = np.zeros((m, n), np.float64)
    lib().twmo_gemm_f64(_p(a), _p(_c(packed, np.uint8)), _p(_c(scales, np.uint16)), _p(c),
                        C.c_uint32(m), C.c_uint32(k), C.c_uint32(n))
    return c


def linear_dense(a, packed, scales, m, k, n):
    """Reference CPU semantics: unpack to dense f32 [K,N], then cpu_gemm."""
    a = _c(a, np.float32)
    dense = np.empty((k, n), np.float32)
    c = np.zeros((m, n), np.float32)
    lib().twmo_linear_dense(_p(a), _p(_c(packed, np.uint8)), _p(_c(scales, np.uint16)), _p(dense),
                            _p(c), C.c_uint32(m), C.c_uint32(k), C.c_uint32(n))
    return c


def pick_splits(k, n):
    nb, sp, kb = C.c_uint32(), C.c_uint32(), C.c_uint32()
    lib().twmo_pick_splits(C.c_uint32(k), C.c_uint32(n), C.byref(nb), C.byref(sp), C.byref(kb))
    return nb.value, sp.value, kb.value


def max_threads():
    return lib().twmo_max_threads()


# ---- deterministic synthetic inputs (identical on every machine) ----

def synth_packed(k, n, seed):
    out = np.empty((k // 32) * n * 16, np.uint8)
    lib().twmo_fill_packed(_p(out), C.c_size_t(out.size), C.c_uint64(seed))
    return out


def synth_scales(k, n, seed):
    out = np.empty((k // 32) * n, np.uint16)
    lib().twmo_fill_scales_f16(_p(out), C.c_size_t(out.size), C.c_uint64(seed))
    return out


def synth_act_f16(m, k, seed):
    out = np.empty(m * k, np.uint16)
    lib().twmo_fill_act_f16(_p(out), C.c_size_t(out.size), C.c_uint64(seed))
    return out.reshape(m, k)


def synth_normal_f32(count, seed):
    out = np.empty(count, np.float32)
    lib().twmo_fill_normal_f32(_p(out), C.c_size_t(out.size), C.c_uint64(seed))
    return out

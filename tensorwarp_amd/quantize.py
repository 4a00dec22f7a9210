"""Host-side mirror of the reference's quantized-linear interface, over the C ABI.

Names, argument order and error behaviour follow crates/kernels/src/quantize.rs,
device.rs, tensor.rs, cuda_graph.rs and ops.rs of the reference so that tests read
like the reference's own; every function is a thin call into libtwmarlin_hip.so.
numpy is used only to move host bytes in and out.
"""
import ctypes as C

import numpy as np

from . import _lib

BLOCK_SIZE = 32           # quantize.rs `BLOCK_SIZE`
Q4_0_BLOCK_BYTES = 20     # quantize.rs `Q4_0_BLOCK_BYTES`


class DeviceError(RuntimeError):
    """device.rs:278-292 `DeviceError`; `.code` is the c_api.rs `WarpError` value."""

    def __init__(self, code, message):
        super().__init__("[%d] %s" % (code, message))
        self.code = code


def _check(rc):
    if rc != _lib.OK:
        raise DeviceError(rc, _lib.load().twm_last_error().decode())


class WarpDevice:
    """device.rs `WarpDevice` + cache.rs `KernelCache`: one context, one stream."""

    def __init__(self, ordinal=0):
        self._l = _lib.load()
        self.handle = self._l.twm_ctx_create(ordinal)
        if not self.handle:
            raise DeviceError(_lib.DEVICE_ERROR, self._l.twm_last_error().decode())

    def close(self):
        if self.handle:
            self._l.twm_ctx_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def synchronize(self):
        _check(self._l.twm_ctx_sync(self.handle))

    def summary(self):
        buf = C.create_string_buffer(256)
        _check(self._l.twm_ctx_info(self.handle, buf, 256))
        return buf.value.decode()

    def with_stream(self, hip_stream):
        _check(self._l.twm_ctx_set_stream(self.handle, hip_stream))

    def set_option(self, key, value):
        _check(self._l.twm_ctx_set_option(self.handle, key.encode(), int(value)))

    def plan(self, k, n, m, dtype="f16", gated=False):
        """What gemm() would launch for a K x N weight and m rows under this context's options, as a line of text."""
        buf = C.create_string_buffer(256)
        _check(self._l.twm_plan_describe(self.handle, k, n, m, _lib.F32 if dtype == "f32" else _lib.F16, int(gated), buf, 256))
        return buf.value.decode()

    def plan_m1(self, k, n):
        """What gemm_tw_marlin_m1() would launch on the reference's K x N arrays under this context's options."""
        buf = C.create_string_buffer(256)
        _check(self._l.twm_plan_describe_m1(self.handle, k, n, buf, 256))
        return buf.value.decode()

    # timing
    def event(self):
        ev = self._l.twm_event_create(self.handle)
        if not ev:
            raise DeviceError(_lib.DEVICE_ERROR, self._l.twm_last_error().decode())
        return ev

    def record(self, ev):
        _check(self._l.twm_event_record(self.handle, ev))

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        _check(self._l.twm_event_elapsed_ms(self.handle, start, stop, C.byref(ms)))
        return ms.value

    def event_destroy(self, ev):
        _check(self._l.twm_event_destroy(self.handle, ev))


_NP_DTYPES = {"f32": np.float32, "f16": np.uint16, "u8": np.uint8, "i32": np.int32}


class GpuTensor:
    """tensor.rs `GpuTensor<T>`: an owned device allocation with a shape.  f16 data
    travels as raw uint16 bit patterns on the host side."""

    def __init__(self, device, shape, dtype):
        self.device = device
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = dtype
        self.numel = int(np.prod(self.shape)) if self.shape else 1
        self.nbytes = self.numel * np.dtype(_NP_DTYPES[dtype]).itemsize
        self.ptr = device._l.twm_malloc(device.handle, self.nbytes)
        if not self.ptr:
            raise DeviceError(_lib.MEMORY_ERROR, device._l.twm_last_error().decode())

    @classmethod
    def zeros(cls, device, shape, dtype):
        t = cls(device, shape, dtype)
        if t.nbytes:
            t.copy_from_host(np.zeros(t.numel, _NP_DTYPES[dtype]))
        return t

    @classmethod
    def from_host(cls, device, array, dtype=None):
        array = np.ascontiguousarray(array)
        if dtype is None:
            dtype = {np.dtype(np.float32): "f32", np.dtype(np.uint16): "f16", np.dtype(np.float16): "f16",
                     np.dtype(np.uint8): "u8", np.dtype(np.int32): "i32"}[array.dtype]
        if array.dtype == np.float16:
            array = array.view(np.uint16)
        t = cls(device, array.shape, dtype)
        t.copy_from_host(array)
        return t

    def copy_from_host(self, array):
        array = np.ascontiguousarray(array, dtype=_NP_DTYPES[self.dtype])
        assert array.nbytes == self.nbytes
        _check(self.device._l.twm_memcpy_h2d(self.device.handle, self.ptr, array.ctypes.data, self.nbytes))

    def to_host(self):
        out = np.empty(self.shape, _NP_DTYPES[self.dtype])
        _check(self.device._l.twm_memcpy_d2h(self.device.handle, out.ctypes.data, self.ptr, self.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.device._l.twm_free(self.device.handle, self.ptr)
            self.ptr = None


def _require_k(k):
    # the reference asserts (quantize.rs:1311); here the library reports SHAPE_ERROR
    if k % BLOCK_SIZE != 0:
        raise DeviceError(_lib.SHAPE_ERROR, "K (%d) must be divisible by %d" % (k, BLOCK_SIZE))


def pick_splits_reference(k, n):
    """quantize.rs:1314-1325 -> (n_blocks, splits, k_blocks_per_split)."""
    nb, sp, kb = C.c_uint32(), C.c_uint32(), C.c_uint32()
    _lib.load().twm_pick_splits_reference(k, n, C.byref(nb), C.byref(sp), C.byref(kb))
    return nb.value, sp.value, kb.value


def pick_splits(k, n, m=1):
    return _lib.load().twm_pick_splits(k, n, m)


def quantize_weights_q4_0(device, weights, k, n):
    """quantize.rs:414 — weights: GpuTensor f32 [K,N] -> GpuTensor u8 (Q4_0 column-major blocks)."""
    _require_k(k)
    out = GpuTensor(device, ((k // BLOCK_SIZE) * n * Q4_0_BLOCK_BYTES,), "u8")
    _check(device._l.twm_quantize_weights_q4_0(device.handle, weights.ptr, k, n, out.ptr))
    return out


def reorder_to_tw_marlin(device, col_major_q4, k, n):
    """quantize.rs:912 -> (packed GpuTensor u8, scales GpuTensor f16)."""
    _require_k(k)
    g = k // BLOCK_SIZE
    packed = GpuTensor(device, (g * n * 16,), "u8")
    scales = GpuTensor(device, (g * n,), "f16")
    _check(device._l.twm_reorder_to_tw_marlin(device.handle, col_major_q4.ptr, k, n, packed.ptr, scales.ptr))
    return packed, scales


def quantize_f32_to_tw_marlin(device, weights, k, n, weights_are_nk=False):
    """quantize.rs:1171 (weights [K,N]); weights_are_nk=True gives cpu_quantize_tw_marlin
    (gemma_moe_q4.rs:218) on a [N,K] matrix."""
    _require_k(k)
    g = k // BLOCK_SIZE
    packed = GpuTensor(device, (g * n * 16,), "u8")
    scales = GpuTensor(device, (g * n,), "f16")
    _check(device._l.twm_quantize_f32_to_tw_marlin(device.handle, weights.ptr, 1 if weights_are_nk else 0, k, n,
                                                   packed.ptr, scales.ptr))
    return packed, scales


def fuse_tw_marlin_n(device, matrices, k, ns):
    """quantize.rs:1018 — matrices: [(packed, scales), ...] GpuTensors; ns: their N."""
    _require_k(k)
    cnt = len(matrices)
    total = int(sum(ns))
    g = k // BLOCK_SIZE
    packed = GpuTensor(device, (g * total * 16,), "u8")
    scales = GpuTensor(device, (g * total,), "f16")
    pp = (C.c_void_p * cnt)(*[m[0].ptr for m in matrices])
    sp = (C.c_void_p * cnt)(*[m[1].ptr for m in matrices])
    nsa = (C.c_uint32 * cnt)(*[int(x) for x in ns])
    _check(device._l.twm_fuse_tw_marlin_n(device.handle, pp, sp, k, nsa, cnt, packed.ptr, scales.ptr))
    return packed, scales


def dequant_to_f16(device, packed, scales, k, n):
    """quantize.rs:580 `dequant_q4_to_f16` for TW-Marlin arrays -> GpuTensor f16 [K,N]."""
    _require_k(k)
    out = GpuTensor(device, (k, n), "f16")
    _check(device._l.twm_dequant_to_f16(device.handle, packed.ptr, scales.ptr, k, n, out.ptr))
    return out


def dequant_to_f32(device, packed, scales, k, n):
    _require_k(k)
    out = GpuTensor(device, (k, n), "f32")
    _check(device._l.twm_dequant_to_f32(device.handle, packed.ptr, scales.ptr, k, n, out.ptr))
    return out


def split_qkv(device, qkv, q, k, v, h, kv_dim, batch):
    """ops.rs:2300"""
    _check(device._l.twm_split_qkv(device.handle, qkv.ptr, q.ptr, k.ptr, v.ptr, h, kv_dim, batch))


def split_gate_up(device, gate_up, gate, up, ffn_dim, batch):
    """ops.rs:2324"""
    _check(device._l.twm_split_gate_up(device.handle, gate_up.ptr, gate.ptr, up.ptr, ffn_dim, batch))


def fused_silu_mul(device, gate, up, out):
    """ops.rs:1139 — out = silu(gate) * up, elementwise f32."""
    _check(device._l.twm_silu_mul(device.handle, gate.ptr, up.ptr, out.ptr, gate.numel))


def swiglu_rows(device, gate_up, out, ffn_dim, batch, paired=False):
    """split_gate_up + fused_silu_mul in one pass; paired=True reads the order of pair_gate_up."""
    _check(device._l.twm_swiglu_rows(device.handle, gate_up.ptr, batch, ffn_dim, int(paired), out.ptr))


def pair_gate_up(device, gate, up, k, ffn_dim):
    """(packed, scales) of gate and up -> TW-Marlin arrays [K/32][2*ffn] with the columns interleaved in runs
    of 32 (gate, up, gate, ...), the order the fused SwiGLU GEMV reads."""
    g = k // 32
    po = GpuTensor(device, (g * 2 * ffn_dim * 16,), "u8")
    so = GpuTensor(device, (g * 2 * ffn_dim,), "f16")
    _check(device._l.twm_pair_gate_up(device.handle, gate[0].ptr, gate[1].ptr, up[0].ptr, up[1].ptr, k, ffn_dim,
                                      po.ptr, so.ptr))
    return po, so


def argmax(device, input, output, rows, cols):
    """missing_ops.rs:42 — input f32 [rows, cols], output i32 [rows]."""
    _check(device._l.twm_argmax_f32(device.handle, input.ptr, rows, cols, output.ptr))


def gemm_tw_marlin_m1(device, a, packed, scales, c, n, k):
    """quantize.rs:1301 — a: f32 [1,K]; packed/scales: reference TW-Marlin arrays; c: f32 [1,N]."""
    _check(device._l.twm_gemm_tw_marlin_m1(device.handle, a.ptr, packed.ptr, scales.ptr, c.ptr, n, k))


def gemm_tw_marlin_m1_from_buffer(device, a, packed_buf, packed_offset, scales_buf, scales_offset, c, n, k):
    """quantize.rs:1731"""
    _check(device._l.twm_gemm_tw_marlin_m1_from_buffer(device.handle, a.ptr, packed_buf.ptr, packed_offset,
                                                       scales_buf.ptr, scales_offset, c.ptr, n, k))


class MarlinWeight:
    """One projection repacked for gfx950 (twm_weight)."""

    def __init__(self, device, handle, k, n):
        self.device, self.handle, self.k, self.n = device, handle, k, n

    @classmethod
    def upload(cls, device, packed_host, scales_host, k, n):
        packed_host = np.ascontiguousarray(packed_host, np.uint8)
        scales_host = np.ascontiguousarray(scales_host).view(np.uint16)
        h = device._l.twm_weight_upload(device.handle, packed_host.ctypes.data, scales_host.ctypes.data, k, n)
        if not h:
            raise DeviceError(_lib.SHAPE_ERROR if k % 32 else _lib.DEVICE_ERROR, device._l.twm_last_error().decode())
        return cls(device, h, k, n)

    @classmethod
    def from_device(cls, device, packed, scales, k, n):
        h = device._l.twm_weight_from_device(device.handle, packed.ptr, scales.ptr, k, n)
        if not h:
            raise DeviceError(_lib.SHAPE_ERROR if k % 32 else _lib.DEVICE_ERROR, device._l.twm_last_error().decode())
        return cls(device, h, k, n)

    @classmethod
    def fuse_n(cls, device, parts):
        """fuse_tw_marlin_n (quantize.rs:1018) on handles: the parts' columns side by side in a new handle."""
        import ctypes
        arr = (ctypes.c_void_p * len(parts))(*[p.handle for p in parts])
        h = device._l.twm_weight_fuse_n(device.handle, arr, len(parts))
        if not h:
            raise DeviceError(_lib.SHAPE_ERROR, device._l.twm_last_error().decode())
        return cls(device, h, parts[0].k, sum(p.n for p in parts))

    @classmethod
    def gate_up(cls, device, gate, up, k, ffn_dim):
        """Paired gate/up weight for gemm_swiglu; gate and up are (packed, scales) device pairs."""
        h = device._l.twm_weight_gate_up(device.handle, gate[0].ptr, gate[1].ptr, up[0].ptr, up[1].ptr, k, ffn_dim)
        if not h:
            raise DeviceError(_lib.SHAPE_ERROR if (k % 32 or ffn_dim % 32) else _lib.DEVICE_ERROR,
                              device._l.twm_last_error().decode())
        return cls(device, h, k, 2 * ffn_dim)

    @property
    def paired(self):
        return bool(self.device._l.twm_weight_is_paired(self.handle))

    @property
    def nbytes(self):
        return self.device._l.twm_weight_bytes(self.handle)

    COPY_TILES, COPY_COLUMN_LANE = 1, 2

    @property
    def copies(self):
        """Mask of the repacked orders the handle holds now (COPY_TILES | COPY_COLUMN_LANE)."""
        return self.device._l.twm_weight_copies(self.handle)

    def tune(self, ms):
        """autotune.rs:254-396 — measure the launch forms for these row counts and keep the fastest per bucket."""
        arr = (C.c_uint32 * len(ms))(*ms)
        _check(self.device._l.twm_weight_tune(self.device.handle, self.handle, arr, len(ms)))

    def tuned_plan(self, m):
        """The kept plan for m rows: dict of the option values, or None when the planners' choice runs."""
        v = (C.c_int * 8)()
        _check(self.device._l.twm_weight_tuned_plan(self.handle, m, v))
        keys = ("valid", "kernel", "nt", "waves", "sub", "sub_waves", "splits", "prefill_bm")
        return dict(zip(keys[1:], list(v)[1:])) if v[0] else None

    def ensure(self, copies):
        _check(self.device._l.twm_weight_ensure(self.device.handle, self.handle, copies))

    def drop(self, copies):
        _check(self.device._l.twm_weight_drop(self.device.handle, self.handle, copies))

    def export_blob(self):
        """The repacked weight as a uint8 array (header + device bytes) for an on-disk cache."""
        size = self.device._l.twm_weight_blob_bytes(self.handle)
        blob = np.empty(size, np.uint8)
        _check(self.device._l.twm_weight_export(self.device.handle, self.handle, blob.ctypes.data, size))
        return blob

    @classmethod
    def import_blob(cls, device, blob):
        blob = np.ascontiguousarray(blob, np.uint8)
        h = device._l.twm_weight_import(device.handle, blob.ctypes.data, blob.size)
        if not h:
            raise DeviceError(_lib.SHAPE_ERROR, device._l.twm_last_error().decode())
        k, n = C.c_uint32(), C.c_uint32()
        device._l.twm_weight_dims(h, C.byref(k), C.byref(n))
        return cls(device, h, k.value, n.value)

    def dequant_f16(self):
        out = GpuTensor(self.device, (self.k, self.n), "f16")
        _check(self.device._l.twm_weight_dequant_f16(self.device.handle, self.handle, out.ptr))
        return out

    def free(self):
        if self.handle:
            self.device._l.twm_weight_destroy(self.handle)
            self.handle = None


def gemm(device, weight, a, m, c, splits=0):
    """C[M,N] f32 = A[M,K] (f16 or f32) x dequant(weight). M=1 is gemm_tw_marlin_m1."""
    dt = _lib.F16 if a.dtype == "f16" else _lib.F32
    _check(device._l.twm_gemm(device.handle, weight.handle, a.ptr, dt, m, c.ptr, splits))


def gemm_f16out(device, weight, a, m, c16, splits=0):
    """gemm() with f16 result rows: c16[M,N] = f16(the f32 result), rounded by the library's cast kernel."""
    dt = _lib.F16 if a.dtype == "f16" else _lib.F32
    _check(device._l.twm_gemm_f16out(device.handle, weight.handle, a.ptr, dt, m, c16.ptr, splits))


def gemm_swiglu(device, weight, a, m, out, splits=0):
    """out[M, ffn] = silu(A x W_gate) * (A x W_up) on a MarlinWeight.gate_up weight: gemm_tw_marlin_m1 +
    split_gate_up + fused_silu_mul of the decode step (and of prefill) with the gate applied in the GEMM's store."""
    dt = _lib.F16 if a.dtype == "f16" else _lib.F32
    _check(device._l.twm_gemm_swiglu(device.handle, weight.handle, a.ptr, dt, m, out.ptr, splits))


def gemm_geglu(device, weight, a, m, out, splits=0):
    """gemm_swiglu with the Gemma gate: out = gelu_tanh(A x W_gate) * (A x W_up)."""
    dt = _lib.F16 if a.dtype == "f16" else _lib.F32
    _check(device._l.twm_gemm_geglu(device.handle, weight.handle, a.ptr, dt, m, out.ptr, splits))


def gemm_split(device, weight, a, m, outs, ns, splits=0, biases=None):
    """Fused projection whose column ranges land in separate buffers (gemm + split_qkv/split_gate_up);
    biases: optional list of f32 [ns[i]] tensors (or None entries) added in the store (bq/bk/bv)."""
    cnt = len(outs)
    dt = _lib.F16 if a.dtype == "f16" else _lib.F32
    op = (C.c_void_p * cnt)(*[o.ptr for o in outs])
    nsa = (C.c_uint32 * cnt)(*[int(x) for x in ns])
    if biases is None:
        _check(device._l.twm_gemm_split(device.handle, weight.handle, a.ptr, dt, m, op, nsa, cnt, splits))
        return
    bp = (C.c_void_p * cnt)(*[(b.ptr if b is not None else None) for b in biases])
    _check(device._l.twm_gemm_split_bias(device.handle, weight.handle, a.ptr, dt, m, op, bp, nsa, cnt, splits))


class TWMarlinWeights:
    """quantize.rs:1067-1166 `TWMarlinWeights`: the seven projections of one layer as
    (packed, scales) device pairs, plus the fused QKV / gate+up made by fuse_projections."""

    NAMES = ("wq", "wk", "wv", "wo", "wg", "wu", "wd")

    def __init__(self, device, hidden_size, kv_dim, ffn_dim, pairs, attn_norm=None, ffn_norm=None, bq=None, bk=None, bv=None):
        self.device, self.h, self.kv, self.ffn = device, hidden_size, kv_dim, ffn_dim
        for name in self.NAMES:
            p, s = pairs[name]
            setattr(self, name + "_packed", p)
            setattr(self, name + "_scales", s)
        # the rest of the reference's struct (quantize.rs:1068-1080): the two norm vectors, which this path only
        # carries, and the optional Q/K/V biases, which qkv() adds in the GEMV's store
        self.attn_norm, self.ffn_norm = attn_norm, ffn_norm
        self.bq, self.bk, self.bv = bq, bk, bv
        self.wqkv_packed = self.wqkv_scales = self.wgu_packed = self.wgu_scales = None
        self.repacked = {}

    def qkv(self, a, m, q, k, v, splits=0):
        """The fused QKV projection of the decode step (generate.rs:2152-2165): one GEMV whose store writes q, k and v
        and adds bq / bk / bv where the layer has them (repack_for_decode first)."""
        biases = [self.bq, self.bk, self.bv] if (self.bq is not None or self.bk is not None or self.bv is not None) else None
        gemm_split(self.device, self.repacked["qkv"], a, m, [q, k, v], [self.h, self.kv, self.kv], splits, biases=biases)

    def fuse_projections(self):
        """quantize.rs:1138"""
        d, h, kv, ffn = self.device, self.h, self.kv, self.ffn
        self.wqkv_packed, self.wqkv_scales = fuse_tw_marlin_n(
            d, [(self.wq_packed, self.wq_scales), (self.wk_packed, self.wk_scales), (self.wv_packed, self.wv_scales)],
            h, [h, kv, kv])
        self.wgu_packed, self.wgu_scales = fuse_tw_marlin_n(
            d, [(self.wg_packed, self.wg_scales), (self.wu_packed, self.wu_scales)], h, [ffn, ffn])

    def repack_for_decode(self):
        """Builds the gfx950 tile-order weights for the four GEMVs of the fused decode path."""
        d, h, kv, ffn = self.device, self.h, self.kv, self.ffn
        if self.wqkv_packed is None:
            self.fuse_projections()
        self.repacked = {
            "qkv": MarlinWeight.from_device(d, self.wqkv_packed, self.wqkv_scales, h, h + 2 * kv),
            "o": MarlinWeight.from_device(d, self.wo_packed, self.wo_scales, h, h),
            "gate_up": MarlinWeight.from_device(d, self.wgu_packed, self.wgu_scales, h, 2 * ffn),
            "down": MarlinWeight.from_device(d, self.wd_packed, self.wd_scales, ffn, h),
        }
        return self.repacked


class ExpertBank:
    """All experts of one MoE projection, repacked (twm_bank): the buffers and strides that
    moe_batched_marlin.rs hands to its batched kernels."""

    def __init__(self, device, handle, k, n, num_experts, paired):
        self.device, self.handle, self.k, self.n, self.num_experts, self.paired = device, handle, k, n, num_experts, paired

    @classmethod
    def from_device(cls, device, packed_buf, scales_buf, packed_bytes_per_expert, scales_per_expert, k, n, num_experts,
                    pair_gate_up=False):
        h = device._l.twm_bank_from_device(device.handle, packed_buf.ptr, scales_buf.ptr, packed_bytes_per_expert,
                                           scales_per_expert, k, n, num_experts, int(pair_gate_up))
        if not h:
            raise DeviceError(_lib.SHAPE_ERROR, device._l.twm_last_error().decode())
        return cls(device, h, k, n, num_experts, bool(pair_gate_up))

    @classmethod
    def from_device_offsets(cls, device, packed_buf, packed_offsets, scales_buf, scales_offsets, k, n, num_experts,
                            pair_gate_up=False):
        """Experts at packed_buf + packed_offsets[e] (bytes) and scales_buf + scales_offsets[e] (elements), u32 device
        tables: the arguments of gemm_tw_marlin_m1_indirect (quantize_indirect.rs:228-253)."""
        h = device._l.twm_bank_from_device_offsets(device.handle, packed_buf.ptr, scales_buf.ptr, packed_offsets.ptr,
                                                   scales_offsets.ptr, k, n, num_experts, int(pair_gate_up))
        if not h:
            raise DeviceError(_lib.SHAPE_ERROR, device._l.twm_last_error().decode())
        return cls(device, h, k, n, num_experts, bool(pair_gate_up))

    @property
    def nbytes(self):
        return self.device._l.twm_bank_bytes(self.handle)

    def free(self):
        if self.handle:
            self.device._l.twm_bank_destroy(self.handle)
            self.handle = None


ACT_NONE, ACT_GEGLU, ACT_SWIGLU = 0, 1, 2


def batched_marlin_gate_up(device, input, bank, topk_ids, output, top_k, act=ACT_NONE, per_slot_rows=False):
    """moe_batched_marlin.rs:153 — output[s] = input x W[topk_ids[s]] for all slots in one launch; with act the
    gate is applied in the store and output is [top_k, N/2] (replaces batched_marlin_split_geglu as well)."""
    dt = _lib.F16 if input.dtype == "f16" else _lib.F32
    _check(device._l.twm_bank_gemv(device.handle, bank.handle, input.ptr, dt, bank.k if per_slot_rows else 0,
                                   topk_ids.ptr, top_k, act, output.ptr))


def batched_marlin_gate_up_slabs(device, input, packed_buf, scales_buf, topk_ids, output, packed_bytes_per_expert,
                                 scales_per_expert, n, k, top_k):
    """moe_batched_marlin.rs:153 with the reference's own arguments: the experts' TW-Marlin arrays as they lie in the
    two slabs, expert x at x * packed_bytes_per_expert / x * scales_per_expert; nothing is repacked."""
    _check(device._l.twm_batched_marlin_gate_up(device.handle, input.ptr, packed_buf.ptr, scales_buf.ptr, topk_ids.ptr,
                                                output.ptr, packed_bytes_per_expert, scales_per_expert, n, k, top_k))


def batched_marlin_down_axpy_slabs(device, geglu_all, packed_buf, scales_buf, topk_ids, topk_weights, acc,
                                   packed_bytes_per_expert, scales_per_expert, n, k, top_k):
    """moe_batched_marlin.rs:184 with the reference's own arguments (slot order instead of float atomics)."""
    _check(device._l.twm_batched_marlin_down_axpy(device.handle, geglu_all.ptr, packed_buf.ptr, scales_buf.ptr, topk_ids.ptr,
                                                  topk_weights.ptr, acc.ptr, packed_bytes_per_expert, scales_per_expert,
                                                  n, k, top_k))


def gemm_tw_marlin_m1_indirect(device, a, packed_buf, packed_offsets, scales_buf, scales_offsets, expert_idx, c, n, k):
    """quantize_indirect.rs:228 — C = A x W[expert_idx], the expert found through the two u32 device tables."""
    _check(device._l.twm_gemm_tw_marlin_m1_indirect(device.handle, a.ptr, packed_buf.ptr, packed_offsets.ptr, scales_buf.ptr,
                                                    scales_offsets.ptr, int(expert_idx), c.ptr, n, k))


def batched_marlin_split_geglu(device, gate_up, output, moe_dim, top_k, paired=False):
    """moe_batched_marlin.rs:215"""
    _check(device._l.twm_geglu_rows(device.handle, gate_up.ptr, top_k, moe_dim, int(paired), output.ptr))


def batched_marlin_down_axpy(device, geglu_all, bank, topk_ids, topk_weights, acc, top_k):
    """moe_batched_marlin.rs:184 — acc += sum_s topk_weights[s] * (geglu_all[s] x W[topk_ids[s]]), slot order."""
    dt = _lib.F16 if geglu_all.dtype == "f16" else _lib.F32
    _check(device._l.twm_bank_down_axpy(device.handle, bank.handle, geglu_all.ptr, dt, topk_ids.ptr, topk_weights.ptr,
                                        top_k, acc.ptr))


class GraphCapture:
    """cuda_graph.rs:72-118"""

    def __init__(self, device, handle):
        self.device, self.handle = device, handle

    @classmethod
    def record_with_device(cls, device, fn):
        _check(device._l.twm_graph_begin(device.handle))
        err = None
        try:
            fn()
        except Exception as e:  # end the capture before reporting, as the reference does (cuda_graph.rs:101-108)
            err = e
        h = device._l.twm_graph_end(device.handle)
        if err is not None:
            if h:
                device._l.twm_graph_destroy(h)
            raise err
        if not h:
            raise DeviceError(_lib.DEVICE_ERROR, device._l.twm_last_error().decode())
        return cls(device, h)

    def replay(self):
        _check(self.device._l.twm_graph_launch(self.device.handle, self.handle))

    def destroy(self):
        if self.handle:
            self.device._l.twm_graph_destroy(self.handle)
            self.handle = None

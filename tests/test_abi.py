"""CPU-side checks of the C ABI: the library loads, exports every symbol that
include/twmarlin.h declares, and fails cleanly (no abort) without a GPU or with bad
handles.  No compute is launched here."""
import ctypes as C
import os
import re

import pytest

import tensorwarp_amd as T
from tensorwarp_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "twmarlin.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(twm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = header_symbols()
    assert len(names) >= 40
    for name in names:
        assert hasattr(lib, name), name


def test_ctypes_table_matches_header():
    assert sorted(_lib.SIGNATURES) == header_symbols()


def test_version_and_error_codes():
    lib = _lib.load()
    assert lib.twm_version() == b"0.1.0"
    # c_api.rs:41-50 WarpError values
    assert (_lib.OK, _lib.DEVICE_ERROR, _lib.MEMORY_ERROR, _lib.SHAPE_ERROR, _lib.UNSUPPORTED_OP,
            _lib.INVALID_HANDLE) == (0, 1, 2, 3, 4, 5)


def test_null_handles_are_rejected_not_crashed():
    lib = _lib.load()
    assert lib.twm_ctx_sync(None) == _lib.INVALID_HANDLE
    assert b"null" in lib.twm_last_error()
    assert lib.twm_gemm(None, None, None, _lib.F16, 1, None, 0) == _lib.INVALID_HANDLE
    assert lib.twm_gemm_f16out(None, None, None, _lib.F16, 1, None, 0) == _lib.INVALID_HANDLE
    assert lib.twm_gemm_tw_marlin_m1(None, None, None, None, None, 64, 64) == _lib.INVALID_HANDLE
    assert lib.twm_graph_begin(None) == _lib.INVALID_HANDLE
    assert lib.twm_graph_launch(None, None) == _lib.INVALID_HANDLE
    assert lib.twm_malloc(None, 16) is None
    assert lib.twm_debug_mfma_mix(None, 0, 0, 1, 64, None) == _lib.INVALID_HANDLE
    assert lib.twm_weight_upload(None, None, None, 64, 64) is None
    assert lib.twm_weight_bytes(None) == 0
    # the fused stores, the weight cache and the expert banks
    assert lib.twm_gemm_swiglu(None, None, None, _lib.F16, 1, None, 0) == _lib.INVALID_HANDLE
    assert lib.twm_gemm_geglu(None, None, None, _lib.F16, 1, None, 0) == _lib.INVALID_HANDLE
    assert lib.twm_gemm_split_bias(None, None, None, _lib.F16, 1, None, None, None, 1, 0) == _lib.INVALID_HANDLE
    assert lib.twm_silu_mul(None, None, None, None, 4) == _lib.INVALID_HANDLE
    assert lib.twm_pair_gate_up(None, None, None, None, None, 64, 64, None, None) == _lib.INVALID_HANDLE
    assert lib.twm_weight_gate_up(None, None, None, None, None, 64, 64) is None
    assert lib.twm_weight_is_paired(None) == 0
    assert lib.twm_weight_fuse_n(None, None, 0) is None
    assert lib.twm_weight_blob_bytes(None) == 0
    assert lib.twm_weight_export(None, None, None, 0) == _lib.INVALID_HANDLE
    assert lib.twm_weight_import(None, None, 0) is None
    assert lib.twm_bank_from_device(None, None, None, 0, 0, 64, 64, 1, 0) is None
    assert lib.twm_bank_bytes(None) == 0
    assert lib.twm_bank_gemv(None, None, None, _lib.F32, 0, None, 1, 0, None) == _lib.INVALID_HANDLE
    assert lib.twm_bank_down_axpy(None, None, None, _lib.F32, None, None, 1, None) == _lib.INVALID_HANDLE
    assert lib.twm_geglu_rows(None, None, 1, 32, 0, None) == _lib.INVALID_HANDLE
    assert lib.twm_batched_marlin_gate_up(None, None, None, None, None, None, 0, 0, 64, 64, 1) == _lib.INVALID_HANDLE
    assert lib.twm_batched_marlin_down_axpy(None, None, None, None, None, None, None, 0, 0, 64, 64, 1) == _lib.INVALID_HANDLE
    assert lib.twm_batched_marlin_split_geglu(None, None, None, 32, 1) == _lib.INVALID_HANDLE
    assert lib.twm_gemm_tw_marlin_m1_indirect(None, None, None, None, None, None, 0, None, 64, 64) == _lib.INVALID_HANDLE
    assert lib.twm_argmax_f32(None, None, 1, 1, None) == _lib.INVALID_HANDLE
    lib.twm_ctx_destroy(None)
    lib.twm_weight_destroy(None)
    lib.twm_bank_destroy(None)
    lib.twm_graph_destroy(None)


@pytest.mark.parametrize("shape,want", [
    ((4096, 4096), (16, 16, 8)), ((896, 1152), (5, 1, 28)), ((896, 896), (4, 1, 28)),
    ((896, 9728), (38, 1, 28)), ((4864, 896), (4, 19, 8)), ((3584, 4608), (18, 14, 8)),
    ((3584, 3584), (14, 14, 8)), ((3584, 37888), (148, 1, 112)), ((18944, 3584), (14, 19, 32)),
    ((4096, 11008), (43, 6, 22)), ((11008, 4096), (16, 16, 22))])
def test_reference_split_k_rule(shape, want):
    # quantize.rs:1317-1325 worked by hand for the benchmark shapes
    assert T.pick_splits_reference(*shape) == want


def test_library_split_choice_is_sane():
    for k, n in [(4096, 4096), (896, 1152), (3584, 37888), (18944, 3584), (4864, 896), (32, 16)]:
        for m in (1, 8, 32):
            sp = T.pick_splits(k, n, m)
            chunks = (k // 32 + 3) // 4
            assert 1 <= sp <= max(chunks, 1)


def test_no_gpu_means_clean_failure():
    lib = _lib.load()
    if lib.twm_device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(T.DeviceError) as e:
        T.WarpDevice(0)
    assert e.value.code == _lib.DEVICE_ERROR
    assert lib.twm_last_error_kind() == 1        # TWM_KIND_INIT: DeviceError::Init (device.rs:278-292)


def test_error_kinds_of_argument_errors():
    # an error that never reached the device maps to no DeviceError variant; the new entries reject null handles
    lib = _lib.load()
    assert lib.twm_ctx_sync(None) == _lib.INVALID_HANDLE and lib.twm_last_error_kind() == 0
    assert lib.twm_stream_create(None) is None and lib.twm_last_error_kind() == 0
    assert lib.twm_stream_sync(None, None) == _lib.INVALID_HANDLE
    assert lib.twm_stream_destroy(None, None) == _lib.INVALID_HANDLE
    assert lib.twm_cast_f32_to_f16(None, None, None, 4) == _lib.INVALID_HANDLE
    assert lib.twm_cast_f16_to_f32(None, None, None, 4) == _lib.INVALID_HANDLE


def test_product_package_does_not_touch_the_oracle():
    pkg = os.path.join(ROOT, "tensorwarp_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("no CPU fallback", ""), f


def test_bench_refuses_more_than_one_gpu():
    # one GPU per box: bench.py --gpus N (N != 1) exits with a message before touching any device
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0
    assert "ONE GPU" in res.stderr

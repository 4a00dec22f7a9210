"""The launch planners, through twm_plan_describe: no GPU is touched (the library is only loaded).

What twm_gemm runs for the benchmark shapes is pinned here as text, so that a change of a planner's rule shows up
as a changed line in this file, and the invariants every plan must keep are checked over a sweep of shapes."""
import ctypes
import re

import numpy as np
import pytest

from tensorwarp_amd import _lib


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def describe(lib, k, n, m, dtype=None, gated=0):
    buf = ctypes.create_string_buffer(256)
    rc = lib.twm_plan_describe(None, k, n, m, _lib.F16 if dtype is None else dtype, gated, buf, 256)
    assert rc == 0, lib.twm_last_error().decode()
    return buf.value.decode()


QWEN7B = {"qkv": (3584, 4608), "o": (3584, 3584), "gate_up": (3584, 37888), "down": (18944, 3584)}


@pytest.mark.parametrize("name,m,dtype,want", [
    # M = 1, the headline: sub-tiles everywhere; gate_up one pass per wave (28 chunks / 4 = 7 passes on eight waves), down the pass loop
    ("qkv", 1, "f16", "k_gemv4s: 32-column sub-tiles, 16 waves, 1 K-split; column-lane copy"),
    ("o", 1, "f16", "k_gemv4s: 16-column sub-tiles, 8 waves, 1 K-split; column-lane copy"),
    ("gate_up", 1, "f16", "k_gemv4s: 16-column sub-tiles, 8 waves, 1 K-split; column-lane copy"),
    ("down", 1, "f16", "k_gemv4s: 16-column sub-tiles, 4 waves, 1 K-split; column-lane copy"),
    # one row of f32 activations: the pass loop on four waves where K is deep or the matrix wide
    ("gate_up", 1, "f32", "k_gemv4s: 16-column sub-tiles, 4 waves, 1 K-split; column-lane copy"),
    ("down", 1, "f32", "k_gemv4s: 16-column sub-tiles, 4 waves, 1 K-split; column-lane copy"),
    # batched decode
    ("gate_up", 4, "f16", "k_gemv4: 1 x 64-column tiles per workgroup, 8 waves, 1 K-split; column-lane copy"),
    ("down", 4, "f16", "k_gemv4s: 16-column sub-tiles, 4 waves, 1 K-split; column-lane copy"),
    ("o", 16, "f16", "k_gemv4s: 16-column sub-tiles, 8 waves, 1 K-split; column-lane copy"),
    ("down", 16, "f16", "k_stream: 8 waves, 4 K-splits + k_splitk_reduce; 16-column tile copy"),
    ("gate_up", 16, "f16", "k_batch: 3 quads per workgroup, 1 tile per wave, 1 k-slice, 1 K-split; 16-column tile copy"),
    ("gate_up", 32, "f16", "k_batch: 3 quads per workgroup, 1 tile per wave, 1 k-slice, 1 K-split; 16-column tile copy"),
    ("down", 32, "f16", "k_batch: 1 quad per workgroup, 1 tile per wave, 2 k-slices, 4 K-splits + k_splitk_reduce; 16-column tile copy"),
    ("qkv", 32, "f16", "k_batch: 1 quad per workgroup, 1 tile per wave, 2 k-slices, 3 K-splits + k_splitk_reduce; 16-column tile copy"),
])
def test_plans_of_the_qwen7b_projections(lib, name, m, dtype, want):
    k, n = QWEN7B[name]
    assert describe(lib, k, n, m, _lib.F32 if dtype == "f32" else _lib.F16) == want


@pytest.mark.parametrize("k,n,m,want", [
    (4096, 11008, 2048, "k_prefill: 128-row x 192-column blocks, 1 K-split; 16-column tile copy"),   # 928 workgroups, two per CU
    (11008, 4096, 2048, "k_prefill: 128-row x 256-column blocks, 1 K-split; 16-column tile copy"),
    (4096, 11008, 512, "k_prefill: 128-row x 192-column blocks, 1 K-split; 16-column tile copy"),   # 232 workgroups instead of 172
    (11008, 4096, 512, "k_prefill: 128-row x 256-column blocks, 4 K-splits + k_splitk_reduce; 16-column tile copy"),
    (3584, 4608, 2048, "k_prefill: 128-row x 192-column blocks, 1 K-split; 16-column tile copy"),
    (3584, 152064, 1, "k_gemv4: 1 x 64-column tiles per workgroup, 8 waves, 1 K-split; column-lane copy"),
    (896, 1152, 1, "k_gemv4s: 16-column sub-tiles, 4 waves, 1 K-split; column-lane copy"),
])
def test_plans_of_prefill_lm_head_and_small_shapes(lib, k, n, m, want):
    assert describe(lib, k, n, m) == want


def test_the_gated_store_takes_32_column_sub_tiles(lib):
    # 16 gate + 16 up columns per workgroup: with 8 + 8 the stores would be 128-byte runs
    assert describe(lib, 3584, 37888, 1, gated=1).startswith("k_gemv4s: 32-column sub-tiles")
    assert describe(lib, 3584, 37888, 1, gated=0).startswith("k_gemv4s: 16-column sub-tiles")


def test_pick_splits_agrees_with_the_described_plan(lib):
    rng = np.random.default_rng(7)
    for _ in range(400):
        k = 32 * int(rng.integers(1, 700))
        n = int(rng.integers(1, 60000))
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 32]))
        text = describe(lib, k, n, m)
        splits = int(re.search(r"(\d+) K-split", text).group(1))
        assert splits == lib.twm_pick_splits(k, n, m), (k, n, m, text)
        k_chunks = (k // 32 + 3) // 4
        assert 1 <= splits <= max(1, k_chunks), (k, n, m, text)
        # which rows go to which kernel family
        kernel = text.split(":")[0]
        if m <= 4:
            assert kernel in ("k_gemv4", "k_gemv4s"), (k, n, m, text)
            assert "column-lane copy" in text
        if m > 16:
            assert kernel == "k_batch", (k, n, m, text)
        if kernel == "k_gemv4s":
            sub, waves = map(int, re.search(r"(\d+)-column sub-tiles, (\d+) waves", text).groups())
            assert sub in (16, 32) and 1 <= waves <= 16
            if m > 4:   # rows beyond four repeat the MFMA chain: only in the one-pass form
                assert waves * (64 // sub) >= k_chunks, (k, n, m, text)


def test_describe_rejects_what_twm_gemm_rejects(lib):
    buf = ctypes.create_string_buffer(64)
    assert lib.twm_plan_describe(None, 100, 64, 1, _lib.F16, 0, buf, 64) == _lib.SHAPE_ERROR       # K % 32
    assert lib.twm_plan_describe(None, 128, 64, 1, 7, 0, buf, 64) == _lib.UNSUPPORTED_OP           # dtype
    assert lib.twm_plan_describe(None, 128, 64, 1, _lib.F16, 0, None, 0) == _lib.INVALID_HANDLE
    assert lib.twm_plan_describe(None, 128, 64, 0, _lib.F16, 0, buf, 64) == 0 and buf.value == b"nothing to launch"


# ---------------------------------------------------------------- the drop-in on the reference's arrays

def describe_m1(lib, k, n):
    buf = ctypes.create_string_buffer(256)
    rc = lib.twm_plan_describe_m1(None, k, n, buf, 256)
    assert rc == 0, lib.twm_last_error().decode()
    return buf.value.decode()


@pytest.mark.parametrize("k,n,want", [
    # the Qwen-7B layer: 32 columns x 16 waves of one pass on qkv, 16 columns elsewhere (one pass per wave on o and on
    # the wide gate_up, the pass loop on sixteen waves on the deep down)
    (3584, 4608, "k_gemv4s: 32-column sub-tiles, 16 waves, 1 K-split; reference arrays"),
    (3584, 3584, "k_gemv4s: 16-column sub-tiles, 8 waves, 1 K-split; reference arrays"),
    (3584, 37888, "k_gemv4s: 16-column sub-tiles, 8 waves, 1 K-split; reference arrays"),
    (18944, 3584, "k_gemv4s: 16-column sub-tiles, 16 waves, 1 K-split; reference arrays"),
    # 65 .. 255 tiles on a deeper K: 32 columns, waves looping; sixteen up to 128 tiles and 160 chunks, else eight
    (13824, 5120, "k_gemv4s: 32-column sub-tiles, 16 waves, 1 K-split; reference arrays"),
    (28672, 8192, "k_gemv4s: 32-column sub-tiles, 8 waves, 1 K-split; reference arrays"),
    (8192, 10240, "k_gemv4s: 32-column sub-tiles, 8 waves, 1 K-split; reference arrays"),
    # 256 tiles or more beyond K = 4096: whole 64-column tiles
    (8192, 57344, "k_gemv4: 1 x 64-column tiles per workgroup, 8 waves, 1 K-split; reference arrays"),
    # the LM head
    (3584, 152064, "k_gemv4s: 16-column sub-tiles, 8 waves, 1 K-split; reference arrays"),
])
def test_known_drop_in_plans(lib, k, n, want):
    assert describe_m1(lib, k, n) == want


def test_drop_in_plan_invariants(lib):
    for k in (32, 64, 896, 2048, 3584, 4096, 5120, 8192, 11008, 16384, 18944, 28672, 32768, 65536):
        for n in (8, 64, 100, 256, 300, 1024, 1152, 4096, 4608, 6144, 8192, 16384, 22016, 57344):
            text = describe_m1(lib, k, n)
            kernel = text.split(":")[0]
            assert kernel in ("k_gemv4s", "k_gemv4"), text
            waves = int(re.search(r"(\d+) waves", text).group(1))
            splits = int(re.search(r"(\d+) K-split", text).group(1))
            k_chunks = (k // 32 + 3) // 4
            assert 1 <= waves <= 16 and 1 <= splits <= k_chunks, (k, n, text)
            if kernel == "k_gemv4s":
                assert int(re.search(r"(\d+)-column sub-tiles", text).group(1)) in (16, 32)
            # K is cut over workgroups only on a few 16-column sub-tiles with a very deep K each, within the CU count;
            # what the no-allocation entry point's static scratch (16 Ki floats, 256 counters) is sized by
            sub_tiles = (n + 63) // 64 * 4
            if splits > 1:
                assert kernel == "k_gemv4s" and sub_tiles <= 64 and k_chunks // splits >= 64 and sub_tiles * splits <= 256, (k, n, text)
                assert splits * ((n + 63) // 64 * 64) <= 16384 and sub_tiles <= 256
    assert "2 K-splits" in describe_m1(lib, 16384, 256) and "4 K-splits" in describe_m1(lib, 32768, 64)
    assert "1 K-split;" in describe_m1(lib, 8192, 200) and "1 K-split;" in describe_m1(lib, 18944, 3584)


def test_describe_m1_edges(lib):
    buf = ctypes.create_string_buffer(64)
    assert lib.twm_plan_describe_m1(None, 100, 64, buf, 64) == _lib.SHAPE_ERROR      # K % 32, as the call itself
    assert lib.twm_plan_describe_m1(None, 128, 64, None, 0) == _lib.INVALID_HANDLE
    assert lib.twm_plan_describe_m1(None, 128, 0, buf, 64) == 0 and buf.value == b"nothing to launch"
    assert lib.twm_plan_describe_m1(None, 0, 64, buf, 64) == 0 and buf.value == b"k_fill_zero"

"""The launch planners, through twm_plan_describe: no GPU is touched (the library is only loaded).

The plans of the benchmark shapes are held to what every good plan must keep (kernel family and repacked copy of a row
count, no K-split where the columns alone fill the CUs, enough workgroups otherwise), not to their text: a planner's
rule can be refitted without editing this file, and bench.py prints every plan line beside the time it led to.  The
same invariants are checked over a sweep of shapes."""
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


def parse(text):
    """The fields of a plan line."""
    f = {"kernel": text.split(":")[0], "copy": text.rsplit(";", 1)[1].strip(), "text": text}
    for key, pat in (("sub", r"(\d+)-column sub-tiles"), ("waves", r"(\d+) waves"), ("splits", r"(\d+) K-split"),
                     ("quads", r"(\d+) quads? per workgroup"), ("tiles_per_wave", r"(\d+) tiles? per wave"),
                     ("slices", r"(\d+) k-slice"), ("tiles64", r"(\d+) x 64-column tiles"),
                     ("block_rows", r"(\d+)-row x"), ("block_cols", r"x (\d+)-column blocks")):
        m = re.search(pat, text)
        if m:
            f[key] = int(m.group(1))
    return f


def workgroups(f, k, n, m):
    n_pad = (n + 63) // 64 * 64
    if f["kernel"] == "k_gemv4s":
        return n_pad // f["sub"] * f["splits"]
    if f["kernel"] == "k_gemv4":
        return -(-(n_pad // 64) // f["tiles64"]) * f["splits"]
    if f["kernel"] == "k_batch":
        return -(-(n_pad // 64) // (f["quads"] * f["tiles_per_wave"])) * f["splits"]
    if f["kernel"] == "k_stream":
        return n_pad // 64 * f["splits"]
    if f["kernel"] == "k_prefill":
        return -(-m // f["block_rows"]) * -(-n_pad // f["block_cols"]) * f["splits"]
    raise AssertionError(f["text"])


CUS = 256


@pytest.mark.parametrize("name", list(QWEN7B))
@pytest.mark.parametrize("m,dtype", [(1, "f16"), (1, "f32"), (2, "f16"), (4, "f16"), (8, "f16"), (16, "f16"), (32, "f16")])
def test_plans_of_the_qwen7b_projections(lib, name, m, dtype):
    # What every plan of the benchmark layer must keep, whatever rule of a planner produced it (the plan lines themselves
    # are printed by bench.py beside the times they led to): the kernel family of the row count, the repacked copy that
    # family reads, no K-split where the columns alone give a workgroup to at least half the CUs, enough workgroups
    # otherwise, and at one row the sub-tile kernel without a hand-over between workgroups.
    k, n = QWEN7B[name]
    f = parse(describe(lib, k, n, m, _lib.F32 if dtype == "f32" else _lib.F16))
    k_chunks, wgs = (k // 32 + 3) // 4, workgroups(f, k, n, m)
    if m <= 4:
        assert f["kernel"] in ("k_gemv4s", "k_gemv4") and f["copy"] == "column-lane copy", f["text"]
        assert f["splits"] == 1, f["text"]                   # (a hand-over between workgroups costs over a microsecond)
    elif m <= 16:
        assert f["kernel"] in ("k_gemv4s", "k_gemv4", "k_stream", "k_batch"), f["text"]
    else:
        assert f["kernel"] == "k_batch" and f["copy"] == "16-column tile copy", f["text"]
    if m == 1:
        assert f["kernel"] == "k_gemv4s" and wgs >= CUS // 2, f["text"]
        if k_chunks <= 32:                                    # K up to 4096: a wave makes one pass or two, no loop
            assert f["waves"] * (64 // f["sub"]) * 2 >= k_chunks, f["text"]
        else:                                                 # deep K: sixteen columns, few waves, the pass loop
            assert f["sub"] == 16 and f["waves"] in (4, 8, 16), f["text"]
    if f["kernel"] in ("k_stream", "k_batch"):
        assert f["copy"] == "16-column tile copy" and 1 <= f["splits"] <= 16, f["text"]
        unsplit = wgs // f["splits"]
        if f["splits"] > 1:
            assert unsplit < CUS and "k_splitk_reduce" in f["text"], f["text"]   # only where the columns leave CUs idle
            assert k_chunks // f["splits"] >= 7, f["text"]                        # and every range keeps some depth
        if n >= 16384:
            assert f["splits"] == 1 and wgs >= 128, f["text"]                    # wide: the columns are enough


@pytest.mark.parametrize("k,n,m", [(4096, 11008, 2048), (11008, 4096, 2048), (4096, 11008, 512), (11008, 4096, 512),
                                   (3584, 4608, 2048), (3584, 37888, 128), (896, 1152, 64)])
def test_plans_of_prefill(lib, k, n, m):
    f = parse(describe(lib, k, n, m))
    assert f["kernel"] == "k_prefill" and f["copy"] == "16-column tile copy", f["text"]
    assert f["block_rows"] in (64, 128) and f["block_cols"] in (192, 256), f["text"]
    wgs, k_chunks = workgroups(f, k, n, m), (k // 32 + 3) // 4
    if f["splits"] > 1:
        assert wgs // f["splits"] < CUS // 2 and "k_splitk_reduce" in f["text"], f["text"]   # K is cut only to fill idle CUs
        assert k_chunks // f["splits"] >= 2, f["text"]
    if m >= 2048 and n >= 4096:
        assert f["block_rows"] == 128 and f["splits"] == 1 and wgs >= CUS, f["text"]        # enough tiles: the cheapest form per row


def test_plans_of_lm_head_and_small_shapes(lib):
    lm = parse(describe(lib, 3584, 152064, 1))
    assert lm["kernel"] in ("k_gemv4", "k_gemv4s") and lm["splits"] == 1 and workgroups(lm, 3584, 152064, 1) >= 8 * CUS, lm["text"]
    small = parse(describe(lib, 896, 1152, 1))
    assert small["kernel"] == "k_gemv4s" and small["splits"] == 1, small["text"]            # shallow K, one row: sub-tiles


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


@pytest.mark.parametrize("k,n", [(3584, 4608), (3584, 3584), (3584, 37888), (18944, 3584),     # the Qwen-7B layer
                                 (13824, 5120), (28672, 8192), (8192, 10240), (8192, 57344), (3584, 152064)])
def test_drop_in_plans_of_model_shapes(lib, k, n):
    # held to what a good plan keeps, not to its text: the MFMA kernels on the arrays as they are, one launch without a
    # hand-over between workgroups, a workgroup for at least half of the CUs, and up to K = 4096 one pass per wave
    f = parse(describe_m1(lib, k, n))
    assert f["kernel"] in ("k_gemv4s", "k_gemv4") and f["copy"] == "reference arrays" and f["splits"] == 1, f["text"]
    assert workgroups(f, k, n, 1) >= CUS // 2, f["text"]
    if k <= 4096:
        assert f["kernel"] == "k_gemv4s" and f["waves"] * (64 // f["sub"]) >= (k // 32 + 3) // 4, f["text"]


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

"""Pins the oracle's arithmetic building blocks (no GPU).

Each check is independent of the oracle's own formula: numpy's integer / IEEE arithmetic,
brute-force enumeration, or a value table read off the reference (path:line cited).
"""
import itertools

import numpy as np
import pytest

import oracle as orc

INT_TYPES = [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.UINT64]
UCX_TYPES = INT_TYPES + [orc.FLOAT32, orc.FLOAT64]          # src/ucx/kernel.cu:60-98
SHM_TYPES = [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.FLOAT32]  # src/shm/utils.cpp:39-69


def test_dtype_size_table():
    # src/core/common.cpp:19-38 with the enum values of include/megray/common.h:106-118
    expected = {0: 1, 1: 1, 2: 4, 3: 4, 4: 8, 5: 8, 6: 2, 7: 4, 8: 8, 9: 1}
    for dtype, size in expected.items():
        assert orc.dtype_size(dtype) == size
    for bad in (-1, 10, 11, 255):
        assert orc.dtype_size(bad) == 0  # the reference throws "unknown dtype"


def test_ring_add_sub_bruteforce():
    # src/ucx/utils.h:24-30: plain modular arithmetic, including delta >= m
    for m in range(1, 10):
        for n in range(m):
            for d in range(0, 3 * m + 1):
                assert orc.ring_add(n, d, m) == (n + d) % m
                assert orc.ring_sub(n, d, m) == (n - d) % m


def test_chunk_partition_exhaustive():
    # src/ucx/all_reduce.cpp:33-38,48-51: tiles [0,len), sizes differ by <=1, larger first
    for nchunks in range(1, 19):
        for length in range(0, 65):
            sizes, offs = orc.chunk_partition(length, nchunks)
            assert sum(sizes) == length
            assert max(sizes) - min(sizes) <= 1
            assert sizes == sorted(sizes, reverse=True)
            assert sizes.count(max(sizes)) == (length % nchunks or nchunks)
            assert offs == [sum(sizes[:i]) for i in range(nchunks)]


def test_f16_to_f32_all_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([orc.f16_to_f32(b) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    # (NaN payloads are not compared: a float returned through ctypes is widened to double and
    # back, which quiets signalling NaNs)


def _f32_to_f16_vec(values):
    return np.array([orc.f32_to_f16(v) for v in values], dtype=np.uint16)


def test_f32_to_f16_roundtrip_ties_and_neighbours():
    bits = np.arange(65536, dtype=np.uint16)
    halves = bits.view(np.float16)
    finite = np.isfinite(halves)
    f32 = halves.astype(np.float32)
    # exact values survive
    assert np.array_equal(_f32_to_f16_vec(f32[finite]), bits[finite])
    # midpoints between neighbouring halves (the RNE ties) and the floats either side of them
    pos = np.sort(f32[finite & (f32 >= 0)])
    mid = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    cases = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)),
                            np.nextafter(mid, np.float32(-np.inf))])
    cases = np.concatenate([cases, -cases])
    with np.errstate(over="ignore"):
        want = cases.astype(np.float16).view(np.uint16)
    assert np.array_equal(_f32_to_f16_vec(cases), want)
    # overflow edge: 65504 is the largest half, 65520 is the tie that rounds to inf
    edge = np.array([65504.0, 65519.996, 65520.0, 65536.0, 1e30, np.inf, -np.inf, 2.0 ** -25,
                     np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -24, 0.0, -0.0],
                    dtype=np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(_f32_to_f16_vec(edge), edge.astype(np.float16).view(np.uint16))


def test_f32_to_f16_random_bit_patterns():
    rng = np.random.default_rng(7)
    pats = rng.integers(0, 2 ** 32, size=200_000, dtype=np.uint64).astype(np.uint32)
    vals = pats.view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = _f32_to_f16_vec(vals)
    nan = np.isnan(vals)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got[nan].view(np.float16)))


@pytest.mark.parametrize("dtype", [orc.INT8, orc.UINT8])
def test_reduce_bytes_all_pairs(dtype):
    npdt = orc.NP_DTYPE[dtype]
    vals = np.arange(256, dtype=np.uint8).view(npdt)
    a = np.repeat(vals, 256)
    b = np.tile(vals, 256)
    with np.errstate(over="ignore"):
        want_sum = (a.astype(np.int32) + b.astype(np.int32)).astype(np.uint8).view(npdt)  # mod 256
    for fn, types in ((orc.reduce_ucx, UCX_TYPES), (orc.reduce_shm, SHM_TYPES)):
        assert dtype in types
        assert np.array_equal(fn(a, b, dtype, orc.SUM), want_sum)
        assert np.array_equal(fn(a, b, dtype, orc.MAX), np.maximum(a, b))
        assert np.array_equal(fn(a, b, dtype, orc.MIN), np.minimum(a, b))


def _rand(dtype, n, rng):
    npdt = orc.NP_DTYPE[dtype]
    if np.issubdtype(npdt, np.integer):
        raw = rng.integers(0, 2 ** 64, size=n, dtype=np.uint64)
        out = raw.astype(np.dtype(npdt).str.replace("i", "u")).view(npdt)
        info = np.iinfo(npdt)
        out[:4] = [info.max, info.min, info.max, info.min]  # force overflow pairs
        return out
    return (rng.standard_normal(n) * np.exp(rng.uniform(-30, 30, n))).astype(npdt)


@pytest.mark.parametrize("dtype", UCX_TYPES)
def test_reduce_wide_types_vs_numpy(dtype):
    rng = np.random.default_rng(dtype)
    a, b = _rand(dtype, 4099, rng), _rand(dtype, 4099, rng)
    b[:2] = a[:2]  # max+max and min+min overflow
    with np.errstate(over="ignore"):
        want_sum = a + b  # numpy wraps integers, adds floats in IEEE
    fns = [orc.reduce_ucx] + ([orc.reduce_shm] if dtype in SHM_TYPES else [])
    for fn in fns:
        assert np.array_equal(fn(a, b, dtype, orc.SUM).view(np.uint8), want_sum.view(np.uint8))
        assert np.array_equal(fn(a, b, dtype, orc.MAX), np.maximum(a, b))
        assert np.array_equal(fn(a, b, dtype, orc.MIN), np.minimum(a, b))


def test_unsupported_dtypes_and_ops():
    a = np.zeros(4, dtype=np.uint64)
    for dtype in (orc.FLOAT16, orc.CHAR):  # src/ucx/kernel.cu:95-96
        with pytest.raises(NotImplementedError):
            orc.reduce_ucx(a.view(orc.NP_DTYPE[dtype]), a.view(orc.NP_DTYPE[dtype]), dtype, orc.SUM)
    for dtype in (orc.UINT64, orc.FLOAT64, orc.FLOAT16, orc.CHAR):  # src/shm/utils.cpp:66-67
        with pytest.raises(NotImplementedError):
            orc.reduce_shm(a.view(orc.NP_DTYPE[dtype]), a.view(orc.NP_DTYPE[dtype]), dtype, orc.SUM)
    f = np.zeros(4, dtype=np.float32)
    for op in (3, -1, 99):  # src/ucx/kernel.cu:55-56, src/shm/utils.cpp:34-35
        with pytest.raises(NotImplementedError):
            orc.reduce_ucx(f, f, orc.FLOAT32, op)
        with pytest.raises(NotImplementedError):
            orc.reduce_shm(f, f, orc.FLOAT32, op)


def _bits(x):
    return np.asarray(x, dtype=np.float32).view(np.uint32).tolist()


def test_float_tie_and_nan_conventions():
    """(i0 > i1) ? i0 : i1 keeps i1 on ties/unordered (src/ucx/kernel.cu:24-38);
    std::max(a, b) / std::min(a, b) keep a (src/shm/utils.cpp:24-32)."""
    pz, nz, nan, one = np.float32(0.0), np.float32(-0.0), np.float32(np.nan), np.float32(1.0)
    a = np.array([pz, nz, nan, one, nan], dtype=np.float32)
    b = np.array([nz, pz, one, nan, nan], dtype=np.float32)
    for op in (orc.MAX, orc.MIN):
        u = orc.reduce_ucx(a, b, orc.FLOAT32, op)
        s = orc.reduce_shm(a, b, orc.FLOAT32, op)
        # +-0 compare equal: ucx returns the second operand, shm the first
        assert _bits(u[:2]) == _bits(b[:2])
        assert _bits(s[:2]) == _bits(a[:2])
        # a NaN makes the compare false: ucx -> i1, shm -> a
        assert u[2] == one and np.isnan(u[3]) and np.isnan(u[4])
        assert np.isnan(s[2]) and s[3] == one and np.isnan(s[4])


def test_sum_special_values():
    a = np.array([np.inf, -np.inf, np.inf, 1e-45, 3.4e38, -0.0, 0.0], dtype=np.float32)
    b = np.array([1.0, 1.0, -np.inf, 1e-45, 3.4e38, -0.0, -0.0], dtype=np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = a + b
    for fn in (orc.reduce_ucx, orc.reduce_shm):
        got = fn(a, b, orc.FLOAT32, orc.SUM)
        assert np.isnan(got[2]) and np.isnan(want[2])
        keep = [0, 1, 3, 4, 5, 6]
        assert _bits(got[keep]) == _bits(want[keep])  # denormal kept, overflow -> inf, -0 + -0 = -0


def test_oracle_selftest_under_sanitizers():
    """The oracle itself, driven over ragged shapes under AddressSanitizer + UBSan (host only)."""
    import os
    import subprocess
    here = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")
    subprocess.check_call(["make", "-s", "-C", here, "selftest_asan"])
    proc = subprocess.run([os.path.join(here, "selftest_asan")], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "selftest ok" in proc.stdout

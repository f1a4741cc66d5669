"""Synthetic rank buffers for the benchmark and the full-size tests.

Counter based: element i of rank r is a pure function of (seed, r, i), so a buffer can be filled in HBM
and any window of it regenerated on the host without copying it back.  The same integer recipe runs in
numpy (uint64) and in torch (int64, two's-complement wrap), and every floating-point value is produced
by one exact conversion and at most one IEEE multiply or subtract, so host and device agree bit for bit.

    z  = (seed + rank) xor (GOLDEN * i)                       (mod 2^64)
    h  = splitmix64 finaliser of z + GOLDEN

    uniform fp32 in [-1, 1):  float(h >> 40) * 2^-23 - 1      (24 bits, exact)
    uniform fp64 in [-1, 1):  float(h >> 11) * 2^-52 - 1      (53 bits, exact)
    integers:                 the low bits of h, reinterpreted in the target width
    "normal" fp16/fp32:       (sum of the eight 16-bit fields of h and of the finaliser of h) - 262140,
                              times sigma / (65536 * sqrt(8/12)): an Irwin-Hall approximation of
                              normal(0, sigma) that needs no transcendental function
"""
import numpy as np

GOLDEN = 0x9E3779B97F4A7C15
MIX1 = 0xBF58476D1CE4E5B9
MIX2 = 0x94D049BB133111EB
BASE_SEED = 0x4D656752  # "MegR"
_MASK = (1 << 64) - 1
_SLICE = 1 << 24  # elements generated per pass on the device (bounds the temporaries)


def _normal_scale(sigma):
    return np.float32(sigma / (65536.0 * np.sqrt(8.0 / 12.0)))


# ---- numpy -------------------------------------------------------------------------------------

def _mix_np(z):
    z = z + np.uint64(GOLDEN)
    z = (z ^ (z >> np.uint64(30))) * np.uint64(MIX1)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(MIX2)
    return z ^ (z >> np.uint64(31))


def hash_np(seed, rank, start, count):
    idx = np.arange(start, start + count, dtype=np.uint64)
    key = np.uint64((seed + rank) & _MASK)
    return _mix_np(key ^ (idx * np.uint64(GOLDEN)))


def _fields_np(h):
    return ((h & np.uint64(0xFFFF)) + ((h >> np.uint64(16)) & np.uint64(0xFFFF)) +
            ((h >> np.uint64(32)) & np.uint64(0xFFFF)) + (h >> np.uint64(48))).astype(np.int64)


def fill_np(np_dtype, count, rank, kind="uniform", start=0, seed=BASE_SEED, sigma=0.01):
    """Elements [start, start+count) of rank `rank`'s buffer as a numpy array of `np_dtype`."""
    np_dtype = np.dtype(np_dtype)
    h = hash_np(seed, rank, start, count)
    if np_dtype.kind in "iu":
        return h.astype(np.dtype(f"u{np_dtype.itemsize}")).view(np_dtype)
    if kind == "normal":
        s = (_fields_np(h) + _fields_np(_mix_np(h)) - 262140).astype(np.float32)
        return (s * _normal_scale(sigma)).astype(np_dtype)
    if np_dtype == np.float64:
        return (h >> np.uint64(11)).astype(np.float64) * 2.0 ** -52 - 1.0
    u = (h >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -23) - np.float32(1.0)
    return u.astype(np_dtype)


# ---- torch (any device) ------------------------------------------------------------------------

def _s64(c):
    c &= _MASK
    return c - (1 << 64) if c >> 63 else c


def _lsr(z, k):
    return (z >> k) & ((1 << (64 - k)) - 1)


def _mix_t(z):
    z = z + _s64(GOLDEN)
    z = (z ^ _lsr(z, 30)) * _s64(MIX1)
    z = (z ^ _lsr(z, 27)) * _s64(MIX2)
    return z ^ _lsr(z, 31)


def _fields_t(h):
    return (h & 0xFFFF) + (_lsr(h, 16) & 0xFFFF) + (_lsr(h, 32) & 0xFFFF) + _lsr(h, 48)


def _chunk_t(torch, dtype, start, count, rank, kind, seed, sigma, device):
    idx = torch.arange(start, start + count, dtype=torch.int64, device=device)
    h = _mix_t((idx * _s64(GOLDEN)) ^ _s64(seed + rank))
    if not dtype.is_floating_point:
        if dtype == torch.int64:
            return h
        bits = 8 * torch.empty((), dtype=dtype).element_size()
        low = h & ((1 << bits) - 1)
        if dtype != torch.uint8:  # sign-extend so the narrowing conversion is value preserving
            low = (low ^ (1 << (bits - 1))) - (1 << (bits - 1))
        return low.to(dtype)
    if kind == "normal":
        s = (_fields_t(h) + _fields_t(_mix_t(h)) - 262140).to(torch.float32)
        return (s * float(_normal_scale(sigma))).to(dtype)
    if dtype == torch.float64:
        return _lsr(h, 11).to(torch.float64) * 2.0 ** -52 - 1.0
    u = _lsr(h, 40).to(torch.float32) * 2.0 ** -23 - 1.0
    return u.to(dtype)


def fill_torch(dtype, count, rank, kind="uniform", start=0, seed=BASE_SEED, sigma=0.01, device="cuda:0", out=None):
    """The same elements as `fill_np`, generated on `device` into a new tensor (or `out`)."""
    import torch

    if out is None:
        out = torch.empty(count, dtype=dtype, device=device)
    for lo in range(0, count, _SLICE):
        n = min(_SLICE, count - lo)
        out[lo:lo + n] = _chunk_t(torch, dtype, start + lo, n, rank, kind, seed, sigma, device)
    return out

"""Device-memory helpers for the GPU parity tests: torch is only the allocator here."""
import numpy as np
import torch

import oracle as orc

DEV = "cuda:0"


def to_device(arr, offset_bytes=0):
    """numpy array -> uint8 device tensor holding the same bytes, optionally shifted off 256-byte
    alignment by `offset_bytes` (torch allocations are at least 256-byte aligned)."""
    raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
    buf = torch.empty(raw.size + offset_bytes + 64, dtype=torch.uint8, device=DEV)
    view = buf[offset_bytes:offset_bytes + raw.size]
    if raw.size:
        view.copy_(torch.from_numpy(raw.copy()))
    return view


def empty_device(nbytes, offset_bytes=0, fill=0xA5):
    buf = torch.full((nbytes + offset_bytes + 64,), fill, dtype=torch.uint8, device=DEV)
    return buf[offset_bytes:offset_bytes + nbytes]


class Guarded:
    """An output buffer of `nbytes` bytes at `offset_bytes` from a 256-byte boundary, with `margin` bytes of a known
    fill on either side: `intact()` tells whether a kernel wrote outside the buffer."""

    def __init__(self, nbytes, offset_bytes=0, fill=0xA5, margin=256):
        self.fill, self.lo, self.hi = fill, margin + offset_bytes, margin + offset_bytes + nbytes
        self.buf = torch.full((self.hi + margin,), fill, dtype=torch.uint8, device=DEV)
        self.view = self.buf[self.lo:self.hi]

    def intact(self):
        return bool((self.buf[:self.lo] == self.fill).all().item()) and bool((self.buf[self.hi:] == self.fill).all().item())


def to_host(view, np_dtype):
    return view.cpu().numpy().view(np_dtype)


def rand_array(dtype, n, rng, wide=True):
    npdt = orc.NP_DTYPE[dtype]
    if np.issubdtype(npdt, np.integer):
        raw = rng.integers(0, 2 ** 64, size=n, dtype=np.uint64)
        return raw.astype(np.dtype(npdt).str.replace("i", "u")).view(npdt)
    if dtype == orc.FLOAT16:
        return (rng.standard_normal(n) * np.exp(rng.uniform(-6, 6, n))).astype(npdt)
    scale = np.exp(rng.uniform(-20, 20, n)) if wide else 1.0
    return (rng.standard_normal(n) * scale).astype(npdt)


def bits_equal(a, b):
    a = np.ascontiguousarray(a).view(np.uint8)
    b = np.ascontiguousarray(b).view(np.uint8)
    return a.shape == b.shape and bool(np.array_equal(a, b))


def first_mismatch(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    ne = np.nonzero((a.view(np.uint8).reshape(a.size, -1) != b.view(np.uint8).reshape(b.size, -1)).any(axis=1))[0]
    if ne.size == 0:
        return None
    i = int(ne[0])
    return i, a[i], b[i], int(ne.size)

"""Helpers of the GPU parity tests: device buffers as raw bytes, seeded payloads, bit-level comparison."""
import numpy as np
import torch

from oracle import templates as T


def have_gpu():
    return torch.cuda.is_available()


class DevBuf:
    """A device allocation holding the bytes of a numpy array (any dtype), at an optional byte offset
    from a 256-byte aligned base so that misaligned pointers can be tested."""

    def __init__(self, arr=None, nbytes=None, offset=0, fill=0xA5):
        if arr is not None:
            arr = np.ascontiguousarray(arr)
            nbytes = arr.nbytes
        self.nbytes = nbytes
        self.offset = offset
        self.t = torch.full((nbytes + offset + 64,), fill, dtype=torch.uint8, device="cuda:0")
        if arr is not None and nbytes:
            self.t[offset:offset + nbytes] = torch.from_numpy(arr.view(np.uint8).reshape(-1).copy()).to("cuda:0")

    @property
    def ptr(self):
        return self.t.data_ptr() + self.offset

    def get(self, np_dtype):
        return self.t[self.offset:self.offset + self.nbytes].cpu().numpy().view(np_dtype).copy()

    def guard_intact(self, fill=0xA5):
        """The bytes before and after the payload were not written."""
        head = self.t[:self.offset].cpu().numpy()
        tail = self.t[self.offset + self.nbytes:].cpu().numpy()
        return bool((head == fill).all() and (tail == fill).all())


def payload(rng, dtype, n, kind="normal"):
    """Seeded storage-typed payload.  16-bit floats come back as uint16 bit patterns."""
    npd = T.NP_STORAGE[dtype]
    if dtype in (T.FP32, T.FP64):
        if kind == "prod":
            return (0.9 + 0.2 * rng.random(n)).astype(npd)
        if kind == "uniform":
            return (rng.random(n) * 2 - 1).astype(npd)
        return rng.standard_normal(n).astype(npd)
    if dtype in (T.FP16, T.BFP16):
        if kind == "prod":
            f = (0.9 + 0.2 * rng.random(n)).astype(np.float32)
        elif kind == "bits":   # every finite bit pattern, subnormals included
            b = rng.integers(0, 65536, size=n, dtype=np.uint32).astype(np.uint16)
            return b & np.uint16(0xFBFF if dtype == T.FP16 else 0xFF7F)
        else:
            f = rng.standard_normal(n).astype(np.float32)
        return T.narrow16(f, dtype)
    ii = np.iinfo(npd)
    return rng.integers(ii.min, ii.max, size=n, dtype=npd, endpoint=True)


def is_nan_bits(a, dtype):
    if dtype == T.FP16:
        return (a & 0x7FFF) > 0x7C00
    if dtype == T.BFP16:
        return (a & 0x7FFF) > 0x7F80
    if dtype in (T.FP32, T.FP64):
        return np.isnan(a)
    return np.zeros(a.shape, dtype=bool)


def assert_same_bits(got, want, dtype, what=""):
    """Bit-exact, except that NaNs only have to be NaNs (their payload is host-FPU specific)."""
    assert got.shape == want.shape, what
    if got.size == 0:
        return
    gn, wn = is_nan_bits(got, dtype), is_nan_bits(want, dtype)
    assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
    g = got.view(np.uint8).reshape(got.size, -1)[~gn]
    w = want.view(np.uint8).reshape(want.size, -1)[~wn]
    if not np.array_equal(g, w):
        bad = np.nonzero((g != w).any(axis=1))[0]
        raise AssertionError(f"{what}: {bad.size} of {got.size} elements differ, first at {bad[0]}: "
                             f"got {got[~gn][bad[0]]!r} want {want[~wn][bad[0]]!r}")


def fold_oracle(srcs, dtype, op, order, wide):
    """acc = srcs[order[0]]; acc = srcs[k] (+) acc for the rest.  wide=True keeps a 16-bit float
    accumulator in fp32 and narrows once (the fused SUM semantics)."""
    if wide and dtype in (T.FP16, T.BFP16):
        acc = T.widen16(srcs[order[0]], dtype)
        e = T.NumericElems(T.FP32, op)
        for k in order[1:]:
            e.reduce(acc, 0, T.widen16(srcs[k], dtype), 0, acc.size)
        return T.narrow16(acc, dtype)
    acc = np.ascontiguousarray(srcs[order[0]]).copy()
    e = T.NumericElems(dtype, op)
    for k in order[1:]:
        e.reduce(acc, 0, np.ascontiguousarray(srcs[k]), 0, acc.size)
    return acc


def fused_is_wide(dtype, op):
    """16-bit float SUM accumulates in fp32 inside a fused fold; PROD narrows every step; MAX/MIN select."""
    return dtype in (T.FP16, T.BFP16) and op == T.SUM

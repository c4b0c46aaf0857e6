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


def sample_positions(rng, length, k, marks=()):
    """k random positions plus the first and last 70 and 8 either side of every mark (slice boundaries)."""
    parts = [rng.integers(0, length, k), np.arange(min(70, length)), np.arange(max(0, length - 70), length)]
    for m in marks:
        parts.append(np.arange(max(0, m - 8), min(length, m + 8)))
    return np.unique(np.concatenate(parts)).astype(np.int64)


def take(t, pos):
    """The elements of device tensor t at the (sorted) host positions pos, as a numpy array."""
    return t[torch.from_numpy(pos).to(t.device)].cpu().numpy()


TORCH_STORAGE = {T.INT8: torch.int8, T.INT16: torch.int16, T.INT32: torch.int32, T.INT64: torch.int64,
                 T.FP16: torch.float16, T.BFP16: torch.bfloat16, T.FP32: torch.float32, T.FP64: torch.float64}


def device_payload(dtype, n, seed):
    """Seeded payload made on the GPU (sizes where a host-made one would take minutes): integers over their whole
    range, floats standard normal.  Returns the tensor in its storage type."""
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    td = TORCH_STORAGE[dtype]
    if td in (torch.int8, torch.int16, torch.int32):
        ii = torch.iinfo(td)
        return torch.randint(ii.min, ii.max + 1, (n,), device="cuda:0", generator=g, dtype=td)
    if td == torch.int64:
        return torch.randint(-2**62, 2**62, (n,), device="cuda:0", generator=g, dtype=td)
    out = torch.empty(n, device="cuda:0", dtype=td)
    step = 1 << 28                      # through fp32 in pieces: no second full-size buffer
    for at in range(0, n, step):
        m = min(step, n - at)
        out[at:at + m] = torch.randn(m, device="cuda:0", generator=g, dtype=torch.float32).to(td)
    return out


def host_sample(t, pos, dtype):
    """Sampled elements of a device tensor as the oracle's storage type (16-bit floats as bit patterns)."""
    v = take(t.view(torch.int16) if dtype in (T.FP16, T.BFP16) else t, pos)
    return v.view(np.uint16) if dtype in (T.FP16, T.BFP16) else v

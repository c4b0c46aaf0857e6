"""Pins oracle/elem_oracle.c against arithmetic stated independently of it (numpy's IEEE conversions and
integer identities), so that a dropped rounding term, a wrong operand order or a missing wrap fails."""
import ctypes

import numpy as np
import pytest

from oracle import templates as T

L = T.lib()


def reduce_np(dst, src, dtype, op):
    d = np.ascontiguousarray(dst).copy()
    s = np.ascontiguousarray(src)
    assert L.orc_reduce(d.ctypes.data, s.ctypes.data, d.size, dtype, op) == 0
    return d


def test_fp16_decode_all_65536_values():
    bits = np.arange(65536, dtype=np.uint16)
    got = T.widen16(bits, T.FP16)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    # NaNs keep sign and payload (mantissa << 13), wrapper.cc:1042-1049
    exp = ((bits.astype(np.uint32) >> 15) << 31) | (0xFF << 23) | ((bits.astype(np.uint32) & 0x3FF) << 13)
    assert np.array_equal(got.view(np.uint32)[nan], exp[nan])


def test_fp16_encode_dense_sweep_matches_ieee_rne():
    rng = np.random.default_rng(7)
    # every exponent, random mantissas, plus exact ties and the values around each half ulp
    raw = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    halves = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32).view(np.uint32)
    ties = np.concatenate([halves + 0x1000, halves + 0x0FFF, halves + 0x1001, halves])
    allbits = np.concatenate([raw, ties]).astype(np.uint32)
    vals = allbits.view(np.float32)
    keep = ~np.isnan(vals)
    vals = vals[keep]
    got = T.narrow16(vals, T.FP16)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_fp16_encode_nan_stays_nan_with_payload():
    f = np.array([0x7FC00000, 0xFFC00001, 0x7F800001, 0x7F802000], dtype=np.uint32).view(np.float32)
    got = T.narrow16(f, T.FP16)
    assert list(got) == [0x7E00, 0xFE00, 0x7C01, 0x7C01]


def test_fp16_roundtrip_is_identity():
    bits = np.arange(65536, dtype=np.uint16)
    assert np.array_equal(T.narrow16(T.widen16(bits, T.FP16), T.FP16), bits)


def test_bf16_narrow_is_rne_on_integers():
    rng = np.random.default_rng(3)
    u = rng.integers(0, 2**32, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    u = np.concatenate([u, np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF, 0x00008000,
                                     0x80008000, 0x7F800000], dtype=np.uint32)])
    f = u.view(np.float32)
    keep = ~np.isnan(f)
    u, f = u[keep], f[keep]
    got = T.narrow16(f, T.BFP16)
    hi, lo = (u >> 16).astype(np.uint64), (u & 0xFFFF).astype(np.uint64)
    up = (lo > 0x8000) | ((lo == 0x8000) & ((hi & 1) == 1))
    want = ((hi + up) & 0xFFFF).astype(np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(T.widen16(want, T.BFP16).view(np.uint32), want.astype(np.uint32) << 16)


@pytest.mark.parametrize("op", [T.SUM, T.PROD, T.MAX, T.MIN])
def test_int8_all_pairs(op):
    a, b = np.meshgrid(np.arange(-128, 128, dtype=np.int64), np.arange(-128, 128, dtype=np.int64))
    a, b = a.ravel(), b.ravel()
    got = reduce_np(b.astype(np.int8), a.astype(np.int8), T.INT8, op)   # dst=b, src=a
    want = {T.SUM: a + b, T.PROD: a * b, T.MAX: np.maximum(a, b), T.MIN: np.minimum(a, b)}[op]
    want = ((want + 128) % 256 - 128).astype(np.int8)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype,bits", [(T.INT16, 16), (T.INT32, 32), (T.INT64, 64)])
@pytest.mark.parametrize("op", [T.SUM, T.PROD, T.MAX, T.MIN])
def test_wide_ints_wrap_like_python_ints(dtype, bits, op):
    rng = np.random.default_rng(bits + op)
    npd = T.NP_STORAGE[dtype]
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    a = rng.integers(lo, hi, size=2000, dtype=np.int64 if bits < 64 else np.int64, endpoint=True)
    b = rng.integers(lo, hi, size=2000, dtype=np.int64, endpoint=True)
    edge = np.array([lo, hi, -1, 0, 1, hi, lo, lo], dtype=np.int64)
    a = np.concatenate([a, edge]); b = np.concatenate([b, edge[::-1]])
    got = reduce_np(b.astype(npd), a.astype(npd), dtype, op)
    mod = 1 << bits
    want = []
    for x, y in zip(a.tolist(), b.tolist()):
        v = {T.SUM: x + y, T.PROD: x * y, T.MAX: max(x, y), T.MIN: min(x, y)}[op]
        want.append((v - lo) % mod + lo)
    assert got.tolist() == want


def test_uint64_wraps():
    a = np.array([2**64 - 1, 2**63, 5, 0], dtype=np.uint64)
    b = np.array([2, 2**63, 7, 9], dtype=np.uint64)
    assert reduce_np(b, a, T.UINT64, T.SUM).tolist() == [1, 0, 12, 9]
    assert reduce_np(b, a, T.UINT64, T.PROD).tolist() == [2**64 - 2, 0, 35, 0]
    assert reduce_np(b, a, T.UINT64, T.MAX).tolist() == [2**64 - 1, 2**63, 7, 9]
    assert reduce_np(b, a, T.UINT64, T.MIN).tolist() == [2, 2**63, 5, 0]


@pytest.mark.parametrize("dtype,npd", [(T.FP32, np.float32), (T.FP64, np.float64)])
def test_float_ops_are_ieee_binary_ops(dtype, npd):
    rng = np.random.default_rng(11)
    a = rng.standard_normal(10000).astype(npd) * npd(1e3)
    b = rng.standard_normal(10000).astype(npd)
    tiny = np.array([1e-40, -1e-40, 1e-45, 0.0, -0.0], dtype=npd)   # fp32 subnormals must survive
    a = np.concatenate([a, tiny]); b = np.concatenate([b, tiny[::-1].copy()])
    assert np.array_equal(reduce_np(b, a, dtype, T.SUM), a + b)
    assert np.array_equal(reduce_np(b, a, dtype, T.PROD), a * b)
    assert np.array_equal(reduce_np(b, a, dtype, T.MAX), np.where(a < b, b, a))
    assert np.array_equal(reduce_np(b, a, dtype, T.MIN), np.where(b < a, b, a))


def test_float_max_min_operand_order_on_nan_and_signed_zero():
    # std::max(src, dst) returns src unless src < dst: NaN in src wins, NaN in dst loses, equal -> src
    src = np.array([np.nan, 1.0, 0.0, -0.0], dtype=np.float32)
    dst = np.array([1.0, np.nan, -0.0, 0.0], dtype=np.float32)
    mx = reduce_np(dst, src, T.FP32, T.MAX)
    mn = reduce_np(dst, src, T.FP32, T.MIN)
    assert np.isnan(mx[0]) and mx[1] == 1.0 and np.isnan(mn[0]) and mn[1] == 1.0
    assert np.signbit(mx[2]) == False and np.signbit(mx[3]) == True   # equal -> src
    assert np.signbit(mn[2]) == False and np.signbit(mn[3]) == True


@pytest.mark.parametrize("op", [T.SUM, T.PROD])
def test_fp16_pairwise_equals_correctly_rounded_half_arithmetic(op):
    # widen -> fp32 op -> RNE narrow is the correctly rounded half result; numpy's float16 ops are that
    rng = np.random.default_rng(5)
    a = rng.integers(0, 65536, size=400000, dtype=np.uint32).astype(np.uint16)
    b = rng.integers(0, 65536, size=400000, dtype=np.uint32).astype(np.uint16)
    got = reduce_np(b, a, T.FP16, op)
    with np.errstate(all="ignore"):
        fa, fb = a.view(np.float16), b.view(np.float16)
        want = (fa + fb if op == T.SUM else fa * fb)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want.view(np.uint16)[ok])
    assert np.all(np.isnan(got.view(np.float16)[~ok]))


def test_fp16_max_selects_original_bits():
    a = np.array([0x3C00, 0x0001, 0x8001, 0x7BFF], dtype=np.uint16)
    b = np.array([0x4000, 0x0002, 0x8002, 0xFBFF], dtype=np.uint16)
    assert reduce_np(b, a, T.FP16, T.MAX).tolist() == [0x4000, 0x0002, 0x8001, 0x7BFF]
    assert reduce_np(b, a, T.FP16, T.MIN).tolist() == [0x3C00, 0x0001, 0x8002, 0xFBFF]


def test_bf16_sum_is_fp32_add_then_rne():
    rng = np.random.default_rng(9)
    a = rng.integers(0, 0x7F80, size=100000, dtype=np.uint32).astype(np.uint16)
    b = (rng.integers(0, 0x7F80, size=100000, dtype=np.uint32) | 0x8000).astype(np.uint16)
    got = reduce_np(b, a, T.BFP16, T.SUM)
    s = (a.astype(np.uint32) << 16).view(np.float32) + (b.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(got, T.narrow16(s, T.BFP16))


def test_unsupported_type_is_internal_error():
    d = np.zeros(4, dtype=np.uint8)
    assert L.orc_reduce(d.ctypes.data, d.ctypes.data, 4, T.UINT8, T.SUM) == 4   # HCCL_E_INTERNAL


@pytest.mark.parametrize("dtype", [T.INT8, T.INT16, T.INT32, T.INT64, T.UINT64, T.FP16, T.FP32, T.FP64, T.BFP16])
@pytest.mark.parametrize("op", [T.SUM, T.PROD, T.MAX, T.MIN])
def test_parallel_variant_gives_the_same_bits(dtype, op):
    rng = np.random.default_rng(dtype * 4 + op)
    npd = T.NP_STORAGE[dtype]
    n = 50001
    if dtype in (T.FP32, T.FP64):
        a = rng.standard_normal(n).astype(npd); b = rng.standard_normal(n).astype(npd)
    else:
        ii = np.iinfo(npd)
        a = rng.integers(ii.min, ii.max, size=n, dtype=npd, endpoint=True)
        b = rng.integers(ii.min, ii.max, size=n, dtype=npd, endpoint=True)
        if dtype in (T.FP16, T.BFP16):   # keep NaN bit patterns out: their payload is not pinned
            a = a & 0x7BFF if dtype == T.FP16 else a & 0x7F7F
            b = b & 0x7BFF if dtype == T.FP16 else b & 0x7F7F
    d1, d2 = b.copy(), b.copy()
    assert L.orc_reduce(d1.ctypes.data, a.ctypes.data, n, dtype, op) == 0
    assert L.orc_reduce_parallel(d2.ctypes.data, a.ctypes.data, n, dtype, op) == 0
    assert np.array_equal(d1, d2)

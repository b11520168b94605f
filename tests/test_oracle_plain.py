"""The oracle on the unquantized weight types (F32, F16, BF16): what pins it.

ggml's CPU mul_mat converts the f32 activations to the weight's own type and adds fp32 products in double.  Pinned here
by mathematics, not by retyping the C: bfloat16 rounding against an exact-arithmetic statement of round-to-nearest-even
(the nearer of the two neighbouring bfloat16 values, the even one on a tie), the float16 path against numpy's casts, the
dot products against numpy fp64 on the converted operands, exact-integer cases, and the output layout with M != N.
"""
import numpy as np
import pytest

import oracle
from oracle import BF16, F16, F32


def _bf16_nearest_even(x: np.ndarray) -> np.ndarray:
    """bfloat16 bit patterns of finite f32 x: both neighbours on the bfloat16 grid, distances in exact fp64"""
    u = x.view(np.uint32).astype(np.uint64)
    lo = u & 0xFFFF0000
    hi = lo + 0x10000  # next bfloat16 away from zero (may be the pattern of infinity: overflow rounds there)
    f = lambda b: (b.astype(np.uint32)).view(np.float32).astype(np.float64)
    xv = x.astype(np.float64)
    inf_hi = (hi & 0x7FFFFFFF) == 0x7F800000
    # the value infinity stands for when rounding: one step beyond the largest finite bfloat16
    fhi = np.where(inf_hi, np.sign(xv) * 2.0 ** 128, f(np.where(inf_hi, lo, hi)))
    dlo, dhi = np.abs(xv - f(lo)), np.abs(fhi - xv)
    take_hi = (dhi < dlo) | ((dhi == dlo) & (((lo >> 16) & 1) == 1))
    return (np.where(take_hi, hi, lo) >> 16).astype(np.uint16)


def test_bf16_rounding_is_nearest_even_on_every_pattern_and_its_neighbourhood():
    h = np.arange(65536, dtype=np.uint32)
    finite = (h & 0x7FFF) < 0x7F80
    h = h[finite]
    cases = []
    for low in (0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x4000, 0xC000):
        cases.append(((h << 16) | low).astype(np.uint32))
    rng = np.random.default_rng(5)
    r = rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32)
    cases.append(r[(r & 0x7F800000) != 0x7F800000])
    u = np.concatenate(cases)
    x = u.view(np.float32)
    got = oracle.quantize(BF16, x[None, :]).view(np.uint16).reshape(-1)
    assert np.array_equal(got, _bf16_nearest_even(x))
    # widening is exact and narrowing inverts it
    back = np.array([oracle.bf16_to_fp32(int(v)) for v in range(0, 65536, 257)], dtype=np.float32)
    assert np.array_equal(back.view(np.uint32) >> 16, np.arange(0, 65536, 257, dtype=np.uint32))


def test_bf16_nan_stays_a_quiet_nan_and_infinities_stay():
    assert oracle.fp32_to_bf16(float("inf")) == 0x7F80 and oracle.fp32_to_bf16(float("-inf")) == 0xFF80
    v = oracle.fp32_to_bf16(float("nan"))
    assert (v & 0x7F80) == 0x7F80 and (v & 0x7F) != 0 and (v & 0x40)
    top = np.array([0x7F7F0000, 0x7F7F7FFF, 0x7F7F8000], dtype=np.uint32).view(np.float32)
    # the largest bfloat16 stays; just below half a step beyond it rounds back; half a step beyond it rounds to infinity
    assert [oracle.fp32_to_bf16(float(v)) for v in top] == [0x7F7F, 0x7F7F, 0x7F80]


def test_f16_conversion_of_rows_is_numpys_cast():
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.standard_normal(5000).astype(np.float32) * s for s in (1e-8, 1e-5, 1.0, 300.0, 7e4)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = oracle.quantize(F16, x[None, :]).view(np.uint16).reshape(-1)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.quantize(F32, x[None, :]).view(np.float32).reshape(-1), x)


def _to(t, a):
    if t == F32:
        return a.astype(np.float32)
    if t == F16:
        return a.astype(np.float16).astype(np.float32)
    return (_bf16_nearest_even(a.astype(np.float32)).astype(np.uint32) << 16).view(np.float32)


def _bytes(t, a):
    """f32 values already representable in t -> the bytes of a tensor of type t"""
    if t == F32:
        return a.astype(np.float32).view(np.uint8)
    if t == F16:
        return a.astype(np.float16).view(np.uint8)
    return (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)


@pytest.mark.parametrize("t", [F32, F16, BF16])
@pytest.mark.parametrize("k", [1, 7, 64, 1000, 4096])
def test_plain_dot_products_against_fp64(t, k):
    rng = np.random.default_rng(100 * t + k)
    w = _to(t, rng.standard_normal(k).astype(np.float32) * 0.05)
    x = rng.standard_normal(k).astype(np.float32)
    xq = oracle.quantize(t, x[None, :]).reshape(-1)
    got = oracle.vec_dot(t, k, _bytes(t, w), xq)
    want = float(np.dot(w.astype(np.float64), _to(t, x).astype(np.float64)))
    scale = float(np.sqrt(np.dot(w.astype(np.float64) ** 2, _to(t, x).astype(np.float64) ** 2))) + 1e-30
    # products of two 16-bit values are exact in fp32; F32 products are rounded once each (2^-24 relative)
    assert abs(got - want) <= (1e-7 if t != F32 else 1e-6) * max(abs(want), scale)


@pytest.mark.parametrize("t", [F32, F16, BF16])
def test_plain_dot_of_small_integers_is_exact(t):
    """integers up to 256 are exact in all three types: the result is the integer dot product, a dropped or doubled
    term or a wrong operand shows as a different integer"""
    rng = np.random.default_rng(9 + t)
    k = 515
    w = rng.integers(-200, 201, k).astype(np.float32)
    x = rng.integers(-256, 257, k).astype(np.float32)
    got = oracle.vec_dot(t, k, _bytes(t, w), oracle.quantize(t, x[None, :]).reshape(-1))
    assert got == float(np.dot(w.astype(np.int64), x.astype(np.int64)))


@pytest.mark.parametrize("t", [F32, F16, BF16])
def test_plain_mul_mat_layout_and_threads(t):
    rng = np.random.default_rng(40 + t)
    k, m, n = 96, 7, 3
    w = _to(t, rng.standard_normal((m, k)).astype(np.float32))
    x = rng.standard_normal((n, k)).astype(np.float32)
    y = oracle.mul_mat(t, _bytes(t, w).reshape(m, -1), k, m, x)
    assert y.shape == (n, m)
    want = _to(t, x).astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(y - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(y, oracle.mul_mat(t, _bytes(t, w).reshape(m, -1), k, m, x, nthreads=3))
    for i in range(n):
        for r in range(m):
            assert y[i, r] == oracle.vec_dot(t, k, _bytes(t, w[r]), oracle.quantize(t, x[i][None, :]).reshape(-1))


def test_plain_sizes_and_vec_dot_types():
    assert [oracle.type_size(t) for t in (F32, F16, BF16)] == [4, 2, 2]
    assert [oracle.block_size(t) for t in (F32, F16, BF16)] == [1, 1, 1]
    assert [oracle.vec_dot_type(t) for t in (F32, F16, BF16)] == [F32, F16, BF16]
    assert oracle.row_size(F16, 4097) == 8194

"""Pins oracle_gemm_f16_fused (the fused GEMM epilogues of before_dl.py:163-318) without the
reference: numpy float16 arithmetic step by step (an independent restatement in another language
and library), the float64 closed form with scipy's erf, and identities that a dropped term, a
swapped operand or a missing rounding step would break."""
import numpy as np
import pytest
from scipy.special import erf


def _inputs(M, N, K, seed):
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    bias = rng.uniform(-1, 1, N).astype(np.float16)
    r1 = rng.standard_normal((M, N)).astype(np.float16)
    r2 = rng.standard_normal((M, N)).astype(np.float16)
    return a, w, bias, r1, r2


def _numpy_steps(mm_h, bias, r1, r2, kind):
    """numpy float16 scalars round after every operation, like the PrimFunc's fp16 buffers."""
    t = (mm_h + bias).astype(np.float16) if bias is not None else mm_h
    if kind in (1, 2):
        t = (r1 + t).astype(np.float16)
        t = (t + r2).astype(np.float16)
        return t.astype(np.float32) if kind == 2 else t
    if kind == 3:
        m = (t * np.float16(0.70710678118654757)).astype(np.float16)
        e = erf(m.astype(np.float32).astype(np.float64)).astype(np.float32).astype(np.float16)
        h = (e * np.float16(0.5)).astype(np.float16)
        g = (np.float16(0.5) + h).astype(np.float16)
        return (t * g).astype(np.float16)
    return t


@pytest.mark.parametrize("kind", [0, 1, 2, 3])
@pytest.mark.parametrize("M,N,K", [(1, 7, 8), (5, 33, 40), (17, 64, 256)])
def test_matches_numpy_float16_step_by_step(oracle, kind, M, N, K):
    a, w, bias, r1, r2 = _inputs(M, N, K, 10 * kind + M)
    mm_h = oracle.c.gemm(a, w)                         # pinned separately (test_oracle_matmul.py)
    got = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind)
    want = _numpy_steps(mm_h, bias, r1, r2, kind)
    assert got.dtype == want.dtype
    if kind == 3:
        # libm's erff vs scipy's float64 erf rounded: equal except at fp16 rounding boundaries
        diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
        ulp = np.maximum(np.abs(want.astype(np.float64)) * 2.0 ** -10, 2.0 ** -24)
        assert (diff <= ulp).all() and (diff == 0).mean() > 0.99
    else:
        assert np.array_equal(got.view(np.uint16 if got.dtype == np.float16 else np.uint32),
                              want.view(np.uint16 if want.dtype == np.float16 else np.uint32))


@pytest.mark.parametrize("kind", [1, 3])
def test_close_to_the_float64_closed_form(oracle, kind):
    a, w, bias, r1, r2 = _inputs(33, 48, 512, kind)
    got = oracle.c.gemm_fused(a, w, bias, r1 if kind == 1 else None, r2 if kind == 1 else None, kind).astype(np.float64)
    want = oracle.np64.gemm_fused(a, w, bias, r1, r2, kind)
    assert (np.abs(got - want) <= 4e-3 + 4e-3 * np.abs(want)).all()


def test_identities(oracle):
    a, w, bias, r1, r2 = _inputs(9, 40, 64, 3)
    zero = np.zeros_like(r1)
    plain = oracle.c.gemm(a, w, bias)
    # zero residuals leave the biased product; kind 2 is kind 1 widened; kind 0 is the plain entry point
    assert np.array_equal(oracle.c.gemm_fused(a, w, bias, zero, zero, 1).view(np.uint16), plain.view(np.uint16))
    k1 = oracle.c.gemm_fused(a, w, bias, r1, r2, 1)
    assert np.array_equal(oracle.c.gemm_fused(a, w, bias, r1, r2, 2), k1.astype(np.float32))
    assert np.array_equal(oracle.c.gemm_fused(a, w, bias, None, None, 0).view(np.uint16), plain.view(np.uint16))
    # the residuals are not interchangeable with the product in rounding order: (r1 + t) + r2
    big = np.full_like(r1, 1024.0)
    tiny = np.full_like(r1, 0.25)
    t = oracle.c.gemm_fused(a * 0, w, None, big, tiny, 1)          # (1024 + 0) + 0.25 -> 1024 in fp16
    u = oracle.c.gemm_fused(a * 0, w, None, tiny, big, 1)          # (0.25 + 0) + 1024 -> 1024 as well
    assert (t == 1024).all() and (u == 1024).all()
    v = oracle.c.gemm_fused(a * 0, w, None, tiny, tiny, 1)
    assert (v == 0.5).all()


def test_gelu_special_values(oracle):
    # one-hot rows of A select a column of W^T: the product is exactly w, so gelu's input is known
    K = 16
    xs = np.array([0.0, -0.0, 1.0, -1.0, 3.0, -3.0, 6.0, -6.0, 0.5, 2.0 ** -14, 100.0, -100.0, 1.0, 1.0, 1.0, 1.0], np.float16)
    a = np.eye(K, dtype=np.float16)
    w = np.zeros((1, K), np.float16)
    w[0, :] = xs
    got = oracle.c.gemm_fused(a, w, None, None, None, 3).astype(np.float64).ravel()
    x = xs.astype(np.float64)
    want = x * (0.5 + 0.5 * erf(x * 0.70710678118654757))
    assert got[0] == 0 and got[1] == 0
    assert got[10] == 100.0 and got[11] == 0.0                        # saturates to x and to 0
    assert (np.abs(got - want) <= 2e-3 + 2e-3 * np.abs(want)).all()
    assert got[2] + got[3] == pytest.approx(0.0 + (got[2] + got[3]))  # finite
    assert abs((got[2] - got[3]) - 1.0) < 2e-3                        # gelu(x) - gelu(-x) = x

"""Pins the row-reduction part of the CPU oracle: closed forms in float64, torch / scipy CPU
routines, and invariants chosen so that a dropped term, a wrong sign or a wrong axis fails."""
import numpy as np
import pytest
import torch
from scipy.special import softmax as scipy_softmax

ATOL = 1e-2  # the stated tolerance for fp16 outputs of the reductions


def _ln_inputs(n=9, H=2560, seed=3):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((n, H)) * 2 + 0.5).astype(np.float32)
    return x, rng.uniform(0.5, 1.5, H).astype(np.float32), rng.uniform(-1, 1, H).astype(np.float32)


def test_layer_norm_closed_form_and_torch(oracle):
    x, g, b = _ln_inputs()
    got = oracle.c.layer_norm(x, g, b).astype(np.float64)
    assert np.abs(got - oracle.np64.layer_norm(x, g, b)).max() < ATOL
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (x.shape[-1],), torch.from_numpy(g), torch.from_numpy(b), 1e-5)
    assert np.abs(got - ref.numpy()).max() < ATOL


def test_layer_norm_invariants(oracle):
    x, g, b = _ln_inputs(n=5)
    one, zero = np.ones_like(g), np.zeros_like(b)
    y = oracle.c.layer_norm(x, one, zero).astype(np.float64)
    assert np.abs(y.mean(-1)).max() < 1e-3 and np.abs(y.var(-1) - 1).max() < 1e-2
    # affine invariance in x: LN(a*x + c) == LN(x) for a > 0
    y2 = oracle.c.layer_norm((3.0 * x + 7.0).astype(np.float32), one, zero).astype(np.float64)
    assert np.abs(y - y2).max() < ATOL
    # sign: negating x negates the normalised value (catches a dropped mean or |.|)
    y3 = oracle.c.layer_norm(-x, one, zero).astype(np.float64)
    assert np.abs(y + y3).max() < ATOL
    # gamma scales, beta shifts
    y4 = oracle.c.layer_norm(x, 2 * one, zero + 0.25).astype(np.float64)
    assert np.abs(y4 - (2 * y + 0.25)).max() < ATOL
    # a constant row has zero variance: output is beta exactly (eps keeps rsqrt finite)
    c = np.full((1, 2560), 3.25, np.float32)
    assert np.abs(oracle.c.layer_norm(c, one, b).astype(np.float32) - b.astype(np.float16).astype(np.float32)).max() < 2e-3


def test_layer_norm_uses_the_row_length_not_2560(oracle):
    x, g, b = _ln_inputs(n=3, H=4096)
    assert np.abs(oracle.c.layer_norm(x, g, b).astype(np.float64) - oracle.np64.layer_norm(x, g, b)).max() < ATOL


def _rms_inputs(n=7, H=4096, seed=3):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((n, H)).astype(np.float16), rng.uniform(0.5, 1.5, H).astype(np.float16)


def test_rms_norm_closed_form_and_torch(oracle):
    x, w = _rms_inputs()
    got = oracle.c.rms_norm(x, w).astype(np.float64)
    assert np.abs(got - oracle.np64.rms_norm(x, w)).max() < ATOL
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x).float(), (x.shape[-1],), torch.from_numpy(w).float(), 1e-5)
    assert np.abs(got - ref.numpy()).max() < ATOL


def test_rms_norm_invariants(oracle):
    x, w = _rms_inputs(n=4)
    one = np.ones_like(w)
    y = oracle.c.rms_norm(x, one).astype(np.float64)
    assert np.abs(np.sqrt((y * y).mean(-1)) - 1).max() < 2e-3            # unit rms
    y2 = oracle.c.rms_norm((x * np.float16(4)).astype(np.float16), one).astype(np.float64)
    assert np.abs(y - y2).max() < ATOL                                   # scale invariance
    assert np.abs(oracle.c.rms_norm(-x, one).astype(np.float64) + y).max() < 1e-6   # odd in x: no mean subtraction
    # unlike layer norm, a constant row is NOT mapped to zero
    c = np.full((1, 4096), 2.0, np.float16)
    assert np.abs(oracle.c.rms_norm(c, one).astype(np.float64) - 1.0).max() < 1e-3
    # eps matters for a zero row: output is exactly zero, not NaN
    assert not np.isnan(oracle.c.rms_norm(np.zeros((1, 4096), np.float16), one)).any()


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("cols", [1, 2, 3, 7, 8, 31, 257, 1024, 4096])
def test_softmax_closed_form_and_scipy(oracle, dtype, cols):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((13, cols)) * 2).astype(dtype)
    got = oracle.c.softmax(x).astype(np.float64)
    assert np.abs(got - oracle.np64.softmax(x)).max() < ATOL
    assert np.abs(got - scipy_softmax(x.astype(np.float64), axis=-1)).max() < ATOL
    assert np.abs(got.sum(-1) - 1).max() < cols * 2.0 ** -11 + 1e-3


def test_softmax_invariants(oracle):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((6, 300)) * 2).astype(np.float32)
    y = oracle.c.softmax(x).astype(np.float64)
    assert np.abs(oracle.c.softmax(x + np.float32(5)).astype(np.float64) - y).max() < 1e-3     # shift invariance
    assert (oracle.c.softmax(np.array([[3.5]], np.float32)) == np.float16(1.0)).all()            # single column
    assert np.abs(oracle.c.softmax(np.full((2, 8), -2.0, np.float32)).astype(np.float64) - 0.125).max() == 0
    assert np.array_equal(np.argmax(y, -1), np.argmax(x, -1))                                    # monotone, right axis
    # large magnitudes: the max subtraction keeps exp finite
    big = np.array([[1e4, 1e4 - 1, -1e4]], np.float32)
    out = oracle.c.softmax(big).astype(np.float64)
    assert np.isfinite(out).all() and abs(out[0, 0] - 1 / (1 + np.exp(-1))) < 1e-3 and out[0, 2] == 0
    # rows are independent: permuting rows permutes outputs
    assert np.array_equal(oracle.c.softmax(x[::-1].copy()), oracle.c.softmax(x)[::-1])


@pytest.mark.parametrize("cols,t", [(1, 0.7), (5, 1.0), (1000, 0.7), (50280, 0.7), (50280, 1.3)])
def test_softmax_temperature_closed_form_and_scipy(oracle, cols, t):
    rng = np.random.default_rng(cols)
    x = (rng.standard_normal((2, cols)) * 4).astype(np.float32)
    got = oracle.c.softmax_temperature(x, t)
    assert got.dtype == np.float32
    want = scipy_softmax(x.astype(np.float64) / float(np.float32(t)), axis=-1)
    # the sum runs in fp32 in the PrimFunc's order: its rounding (a common factor of each row) grows with the row length
    assert np.abs(got - want).max() < 1e-4 and np.abs(got / want - 1).max() < 1e-3
    assert np.abs(got.astype(np.float64).sum(-1) - 1).max() < 1e-3


def test_softmax_temperature_invariants(oracle):
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((3, 777)) * 3).astype(np.float32)
    # temperature 1 divides by exactly 1: the plain fp32 softmax, whose fp16 rounding is the other oracle function
    one = oracle.c.softmax_temperature(x, 1.0)
    assert np.array_equal(one.astype(np.float16), oracle.c.softmax(x))
    # a division, not a product: t = 0.5 doubles the logits exactly
    assert np.array_equal(oracle.c.softmax_temperature(x, 0.5), oracle.c.softmax_temperature(x * np.float32(2), 1.0))
    # a lower temperature sharpens: the largest probability grows
    assert (oracle.c.softmax_temperature(x, 0.5).max(-1) > one.max(-1)).all()
    assert (oracle.c.softmax_temperature(np.array([[2.5]], np.float32), 0.3) == np.float32(1)).all()
    assert np.array_equal(np.argmax(one, -1), np.argmax(x, -1))


def test_softmax_f32_is_the_temperature_form_with_nothing_divided(oracle):
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((2, 3000)) * 3).astype(np.float32)
    got = oracle.c.softmax_f32(x)
    assert got.dtype == np.float32 and np.array_equal(got.astype(np.float16), oracle.c.softmax(x))
    assert np.abs(got / scipy_softmax(x.astype(np.float64), axis=-1) - 1).max() < 1e-4
    # divide2 then softmax2 is softmax_with_temperature, bit for bit
    assert np.array_equal(oracle.c.softmax_f32(oracle.c.divide(x, 0.7)), oracle.c.softmax_temperature(x, 0.7))


def test_layer_norm_f32_rounds_to_the_fused_form_and_matches_the_closed_form(oracle):
    x, g, b = _ln_inputs()
    got = oracle.c.layer_norm_f32(x, g, b)
    assert got.dtype == np.float32 and np.array_equal(got.astype(np.float16), oracle.c.layer_norm(x, g, b))
    assert np.abs(got - oracle.np64.layer_norm(x, g, b)).max() < 1e-4
    want = torch.layer_norm(torch.from_numpy(x), (x.shape[-1],), torch.from_numpy(g), torch.from_numpy(b), 1e-5).numpy()
    assert np.abs(got - want).max() < 1e-4
    short = x[:, :777].copy()                                                   # 1/H follows the row length
    assert np.abs(oracle.c.layer_norm_f32(short, g[:777].copy(), b[:777].copy()) - oracle.np64.layer_norm(short, g[:777], b[:777])).max() < 1e-4

"""Pins the elementwise part of the CPU oracle (oracle/cpu_ref.c) without the reference:
IEEE-754 closed forms, numpy as the library routine, exhaustive enumeration where feasible."""
import numpy as np
import pytest

ALL_F16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)


def test_widen_all_65536_patterns(oracle):
    h = ALL_F16.view(np.float16)
    got = oracle.c.cast(h, "float32")
    want = h.astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    # NaNs stay NaNs with their payload; the conversion instruction sets the quiet bit of a
    # signalling NaN (IEEE 754 conversion), numpy's software path does not
    quiet = np.uint32(0x00400000)
    assert np.array_equal(got.view(np.uint32)[nan], want.view(np.uint32)[nan] | quiet)


def test_soft_widen_matches_hardware_path(oracle):
    got = np.array([oracle.c.soft_h2f(int(b)) for b in ALL_F16[::7]], dtype=np.float32)
    want = ALL_F16[::7].view(np.float16).astype(np.float32)
    nan = np.isnan(want)  # (a NaN's quiet bit does not survive the float -> Python double return)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.isnan(got[nan]).all()


NARROW_BOUNDARIES = [0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, -65520.0, 1e10, -1e10, np.inf, -np.inf,
                     2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26, 2.0 ** -14, 2.0 ** -14 * (1 - 2 ** -11),
                     1.0 + 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -20, 1.0 + 3 * 2.0 ** -11, 2047.5, 2048.5, 2049.5,
                     6.1e-5, 5.96e-8, 2.98e-8, 2.99e-8]


def test_narrow_boundaries(oracle):
    x = np.array(NARROW_BOUNDARIES, dtype=np.float32)
    got = oracle.c.cast(x, "float16")
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    assert np.isinf(got[2 + 2]) and got[2] == np.float16(65504) and got[3] == np.float16(65504)  # 65520 -> inf
    soft = np.array([oracle.c.soft_f2h(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(soft, want.view(np.uint16))


def test_narrow_random_bit_patterns(oracle):
    rng = np.random.default_rng(11)
    bits = rng.integers(0, 2 ** 32, size=1 << 22, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    got = oracle.c.cast(x, "float16")
    with np.errstate(over="ignore", invalid="ignore"):
        want = x.astype(np.float16)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
    # the integer-only conversion agrees on a sample (python-call bound)
    idx = rng.integers(0, x.size, size=4000)
    soft = np.array([oracle.c.soft_f2h(float(x[i])) if not np.isnan(x[i]) else 0 for i in idx], dtype=np.uint16)
    ok = ~np.isnan(x[idx])
    assert np.array_equal(soft[ok], want.view(np.uint16)[idx][ok])


def test_narrow_scaled_normal_overflows_to_inf(oracle):
    # the benchmark's cast input: normal(0,1) * 100 never overflows, * 1e5 does
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(1 << 16) * 1e5).astype(np.float32)
    got = oracle.c.cast(x, "float16")
    assert np.isinf(got[np.abs(x) >= 65520]).all() and np.isfinite(got[np.abs(x) < 65504]).all()


def test_add_f16_is_one_rounding_of_the_exact_sum(oracle):
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, 1 << 18).astype(np.float16)
    b = rng.uniform(-1, 1, 1 << 18).astype(np.float16)
    got = oracle.c.add(a, b)
    assert np.array_equal(got.view(np.uint16), (a + b).view(np.uint16))
    exact = (a.astype(np.float64) + b.astype(np.float64)).astype(np.float16)  # fp64 holds the sum exactly
    assert np.array_equal(got.view(np.uint16), exact.view(np.uint16))


def test_add_f16_special_values(oracle):
    sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504, -65504, 6e-8, -6e-8, 6.1e-5, 1, -1], dtype=np.float16)
    a, b = np.meshgrid(sp, sp)
    a, b = np.ascontiguousarray(a.ravel()), np.ascontiguousarray(b.ravel())
    got = oracle.c.add(a, b)
    with np.errstate(all="ignore"):
        want = a + b
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
    assert np.isnan(oracle.c.add(np.array([np.inf], np.float16), np.array([-np.inf], np.float16))[0])


def test_add_f16_all_patterns_against_one_operand(oracle):
    a = ALL_F16.view(np.float16)
    for other in (np.float16(1.0), np.float16(-3.140625), np.float16(6e-8), np.float16(60000)):
        b = np.full_like(a, other)
        got = oracle.c.add(a, b)
        with np.errstate(all="ignore"):
            want = a + b
        nan = np.isnan(want)
        assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])


def test_add_i8_wraps_exhaustive(oracle):
    a, b = np.meshgrid(np.arange(-128, 128, dtype=np.int8), np.arange(-128, 128, dtype=np.int8))
    a, b = np.ascontiguousarray(a.ravel()), np.ascontiguousarray(b.ravel())
    got = oracle.c.add(a, b)
    want = ((a.astype(np.int32) + b.astype(np.int32) + 128) % 256 - 128).astype(np.int8)
    assert np.array_equal(got, want)
    assert oracle.c.add(np.array([127], np.int8), np.array([1], np.int8))[0] == -128


def test_add_f32_and_copy(oracle):
    rng = np.random.default_rng(5)
    a, b = rng.standard_normal(10001).astype(np.float32), rng.standard_normal(10001).astype(np.float32)
    assert np.array_equal(oracle.c.add(a, b), a + b)
    h = ALL_F16.view(np.float16)
    assert np.array_equal(oracle.c.copy(h).view(np.uint16), ALL_F16)  # identity on bits, NaNs too


def test_threads_do_not_change_bits(oracle):
    rng = np.random.default_rng(9)
    a = rng.uniform(-1, 1, (37, 4096)).astype(np.float16)
    b = rng.uniform(-1, 1, (37, 4096)).astype(np.float16)
    assert np.array_equal(oracle.c.add(a, b, threads=1).view(np.uint16), oracle.c.add(a, b, threads=4).view(np.uint16))
    assert oracle.c.add(a[:0], b[:0]).size == 0  # empty extent


def test_take_is_numpy_row_indexing(oracle):
    # take (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:1151-1163): T_take[i, :] = A[B[i], :], bit for bit
    rng = np.random.default_rng(31)
    a = rng.integers(0, 2 ** 16, (37, 24), dtype=np.uint16).view(np.float16)      # every bit pattern, NaN payloads included
    ids = np.array([0, 36, 5, 5, 17, 36, 0, 1], np.int32)
    assert np.array_equal(oracle.c.take(a, ids).view(np.uint16), a[ids].view(np.uint16))
    assert oracle.c.take(a, np.zeros(0, np.int32)).shape == (0, 24)


def _rotary_inputs(n, heads, d, rot, max_pos, seed):
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((1, n, heads, d)).astype(np.float16)
    ang = rng.uniform(0, 6.28, (max_pos, rot))
    return a, np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)


def test_rotary_matches_numpy_float16_step_by_step(oracle):
    # rotary_embedding (before_dl.py:1023-1035): B * A + C * (j < 10 ? A[j + 10] * -1 : A[j - 10]) for j < 20, A beyond
    n, heads, d, rot, m = 5, 3, 80, 20, 9
    a, cos, sin = _rotary_inputs(n, heads, d, rot, 16, 1)
    got = oracle.c.rotary(a, cos, sin, m)
    pos = m + np.arange(n) - n
    b, c = cos[pos][:, None, :], sin[pos][:, None, :]                        # [n, 1, rot]
    x = a[0]
    partner = np.concatenate([x[..., 10:20] * np.float16(-1), x[..., 0:10]], axis=-1)      # numpy rounds each fp16 op
    want = x.copy()
    want[..., :rot] = b * x[..., :rot] + c * partner
    assert want.dtype == np.float16 and np.array_equal(got[0].view(np.uint16), want.view(np.uint16))
    # float64 rotation of the pairs (j, j + 10): tolerance, and the pair norms survive when cos^2 + sin^2 = 1
    x64, b64, c64 = x.astype(np.float64), b.astype(np.float64), c.astype(np.float64)
    lo = b64[..., :10] * x64[..., :10] - c64[..., :10] * x64[..., 10:20]
    hi = b64[..., 10:] * x64[..., 10:20] + c64[..., 10:] * x64[..., :10]
    assert np.abs(got[0][..., :10].astype(np.float64) - lo).max() < 4e-3 and np.abs(got[0][..., 10:20].astype(np.float64) - hi).max() < 4e-3
    # a swapped partner or a missing sign fails this: rotating by a quarter turn maps (x, y) to (-y, x)
    q_cos, q_sin = np.zeros((16, rot), np.float16), np.ones((16, rot), np.float16)
    quarter = oracle.c.rotary(a, q_cos, q_sin, m)[0]
    assert np.array_equal(quarter[..., :10], -x[..., 10:20]) and np.array_equal(quarter[..., 10:20], x[..., :10])
    # cos = 1, sin = 0: the identity, bit for bit; the positions are m - n .. m - 1
    ident = oracle.c.rotary(a, np.ones((16, rot), np.float16), np.zeros((16, rot), np.float16), m)
    assert np.array_equal(ident.view(np.uint16), a.view(np.uint16))
    marked = np.ones((16, rot), np.float16)
    marked[m - n] = 2
    assert np.array_equal(oracle.c.rotary(a, marked, np.zeros((16, rot), np.float16), m)[0, 0, :, :rot], x[0, :, :rot] * np.float16(2))


def test_attn_mask_is_the_two_primfuncs_in_sequence(oracle):
    # make_diag_mask_te: Select(i < j, -65504, 65504) on [n, n]; extend_te: j < m - n ? 65504 : A[i, j + n - m] on [n, m]
    for n, m in ((1, 1), (1, 7), (5, 5), (5, 9), (64, 200)):
        diag = np.where(np.arange(n)[:, None] < np.arange(n)[None, :], np.float16(-65504), np.float16(65504)).astype(np.float16)
        ext = np.full((n, m), np.float16(65504), np.float16)
        ext[:, m - n:] = diag
        got = oracle.layout.attn_mask(n, m)
        assert got.dtype == np.float16 and np.array_equal(got, ext)
    assert np.array_equal(oracle.layout.attn_mask(1, 9), np.full((1, 9), 65504, np.float16))      # full: nothing hidden from the last position
    last = oracle.layout.attn_mask(4, 6)
    assert (last[0] == [65504, 65504, 65504, -65504, -65504, -65504]).all() and (last[3] == 65504).all()


def test_swap_axes_follows_the_index_expression(oracle):
    rng = np.random.default_rng(3)
    a = rng.integers(0, 2 ** 16, (1, 5, 3, 8), dtype=np.uint16).view(np.float16)
    t = oracle.layout.swap_axes(a)
    assert t.shape == (1, 3, 5, 8)
    for i1 in range(3):
        for i2 in range(5):
            assert np.array_equal(t[0, i1, i2].view(np.uint16), a[0, i2, i1].view(np.uint16))


def test_split3_follows_the_index_expression(oracle):
    rng = np.random.default_rng(5)
    a = rng.integers(0, 2 ** 16, (1, 4, 32, 240), dtype=np.uint16).view(np.float16)
    outs = oracle.layout.split3(a)
    assert all(o.shape == (1, 4, 32, 80) and o.flags.c_contiguous for o in outs)
    for sec, off in enumerate((0, 80, 160)):                 # T_split_sections_s[.., ax3] = A[.., ax3 + 80 s]
        for ax3 in (0, 1, 79):
            assert np.array_equal(outs[sec][..., ax3].view(np.uint16), a[..., ax3 + off].view(np.uint16))
    # the decode form reads the flat [1, 1, 7680] projection: same bytes, reshaped to heads x 240 first
    flat = a[:, :1].reshape(1, 1, 7680)
    again = oracle.layout.split3(flat.reshape(1, 1, 32, 240))
    assert np.array_equal(again[1].view(np.uint16), outs[1][:, :1].view(np.uint16))


def test_divide_is_numpy_float32_division(oracle):
    rng = np.random.default_rng(6)
    a = np.concatenate([(rng.standard_normal(5000) * 10).astype(np.float32), np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, 3.4e38], np.float32)])
    with np.errstate(over="ignore"):                                                    # 3.4e38 / 1e-30 is meant to overflow
        for b in (0.7, 1.0, -0.3, 3.0, 1e-30):
            got = oracle.c.divide(a, b)
            want = a / np.float32(b)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
            finite = np.isfinite(want) & (np.abs(want) > 1e-30)
            exact = (a.astype(np.float64) / float(np.float32(b))).astype(np.float32)    # one rounding of the exact quotient
            assert np.array_equal(got[finite], exact[finite])
    assert np.array_equal(oracle.c.divide(a, 1.0).view(np.uint32), a.view(np.uint32))

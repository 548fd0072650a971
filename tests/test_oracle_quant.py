"""Pins oracle_decode_q8_f16 / oracle_gemv_q8_f16 / oracle_take_q8_f16 / oracle_gemv_q8_f32 (the q8f16_1 PrimFuncs,
experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py:335-343, :401-426, :428-502) without the reference:
numpy float16 arithmetic on the bytes, byte order, scale groups, closed forms, and the pinned GEMM oracle."""
import numpy as np


def _weights(N, K, seed):
    rng = np.random.default_rng(seed)
    wq = rng.integers(0, 2 ** 32, (N, K // 4), dtype=np.uint32)
    scale = (rng.random((N, K // 32)) * 0.02 + 0.001).astype(np.float16)
    return wq, scale


def test_decode_matches_numpy_float16_on_the_bytes(oracle):
    wq, scale = _weights(5, 96, 1)
    got = oracle.c.decode_q8(wq, scale)
    # the PrimFunc shifts word j / 4 right by 8 * (j % 4): element j is byte j of the row in little-endian memory
    shifts = (8 * (np.arange(96) % 4)).astype(np.uint32)
    by_shift = (wq[:, np.arange(96) // 4] >> shifts) & np.uint32(255)
    assert np.array_equal(by_shift.astype(np.uint8), wq.view(np.uint8).reshape(5, 96))
    want = (by_shift.astype(np.float16) - np.float16(127)) * np.repeat(scale, 32, axis=1)        # numpy rounds each fp16 op
    assert want.dtype == np.float16 and np.array_equal(got.view(np.uint16), want.view(np.uint16))
    f64 = oracle.np64.decode_q8(wq, scale)
    assert (np.abs(got.astype(np.float64) - f64) <= 2.0 ** -11 * np.abs(f64) + 1e-9).all()        # one rounding


def test_decode_special_bytes_order_and_group_boundary(oracle):
    scale = np.array([[0.5, 2.0]], np.float16)
    wq = np.zeros((1, 16), np.uint32)
    wq[0, 0] = 127 | (0 << 8) | (255 << 16) | (128 << 24)      # elements 0..3: bytes 127, 0, 255, 128
    wq[0, 7] = 129 << 24                                       # element 31: last of scale group 0
    wq[0, 8] = 129                                             # element 32: first of scale group 1
    got = oracle.c.decode_q8(wq, scale).astype(np.float64)[0]
    assert list(got[:4]) == [0.0, -63.5, 64.0, 0.5]
    assert got[31] == 1.0 and got[32] == 4.0
    assert (got[4:31] == -63.5).all() and (got[33:] == -254.0).all()                            # byte 0 elsewhere
    # the fp16 product rounds: (255 - 127) * 0.1 (fp16 0.0999755859375) = 12.796875 exactly; * 3 needs rounding
    s = np.array([[np.float16(1 / 3)]], np.float16)
    w = np.full((1, 8), 0x82828282, np.uint32)                 # bytes 130: q = 3
    assert np.array_equal(oracle.c.decode_q8(w, s), np.full((1, 32), np.float16(3) * np.float16(1 / 3), np.float16))


def test_gemv_equals_the_gemm_oracle_on_the_decoded_matrix(oracle):
    rng = np.random.default_rng(3)
    wq, scale = _weights(37, 160, 2)
    x = rng.standard_normal(160).astype(np.float16)
    bias = rng.standard_normal(37).astype(np.float16)
    w = oracle.c.decode_q8(wq, scale)
    for kind in (0, 3):
        for b in (None, bias):
            got = oracle.c.gemv_q8(x, wq, scale, b, kind=kind)
            want = oracle.c.gemm_fused(x[None], w, b, None, None, kind)[0]                      # pinned in test_oracle_fused_gemm.py
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    lit = oracle.c.gemv_q8(x, wq, scale, bias, acc_f16=True)
    assert np.array_equal(lit.view(np.uint16), oracle.c.gemm(x[None], w, bias, acc_f16=True)[0].view(np.uint16))
    f64 = w.astype(np.float64) @ x.astype(np.float64) + bias.astype(np.float64)
    got = oracle.c.gemv_q8(x, wq, scale, bias).astype(np.float64)
    assert (np.abs(got - f64) <= 2e-3 + 2e-3 * np.abs(f64)).all()


def test_gemv_one_hot_x_selects_a_decoded_column(oracle):
    wq, scale = _weights(9, 64, 4)
    w = oracle.c.decode_q8(wq, scale)
    for k in (0, 3, 31, 32, 63):
        x = np.zeros(64, np.float16)
        x[k] = 1
        assert np.array_equal(oracle.c.gemv_q8(x, wq, scale), w[:, k])


def test_take_is_rows_of_the_pinned_dequantiser(oracle):
    # fused_fused_decode1_take1 (before_dl.py:357-369): out[i, :] = decode(...)[ids[i], :]
    wq, scale = _weights(23, 96, 5)
    ids = np.array([0, 22, 7, 7, 1, 22, 0], np.int32)
    got = oracle.c.take_q8(wq, scale, ids)
    assert np.array_equal(got.view(np.uint16), oracle.c.decode_q8(wq, scale)[ids].view(np.uint16))
    assert oracle.c.take_q8(wq, scale, np.zeros(0, np.int32)).shape == (0, 96)


def _weights_f32(N, K, seed):
    rng = np.random.default_rng(seed)
    wq = rng.integers(0, 2 ** 32, (N, K // 4), dtype=np.uint32)
    return wq, (rng.random((N, K // 32)) * 0.02 + 0.001).astype(np.float32)


def test_gemv_f32_scales_matches_numpy_float32_and_the_pinned_fp32_gemv(oracle):
    # fused_fused_decode6_NT_matmul5 (before_dl.py:640-657): W = float32(fp16(byte) - 127) * fp32 scale, then NT_matmul5
    rng = np.random.default_rng(6)
    wq, scale = _weights_f32(29, 160, 7)
    x = rng.standard_normal(160).astype(np.float32)
    q = wq.view(np.uint8).reshape(29, 160).astype(np.float16) - np.float16(127)                  # exact: integers in [-127, 128]
    assert np.array_equal(q.astype(np.float64), wq.view(np.uint8).reshape(29, 160).astype(np.float64) - 127)
    w32 = q.astype(np.float32) * np.repeat(scale, 32, axis=1)                                    # numpy rounds the fp32 product
    assert w32.dtype == np.float32
    got = oracle.c.gemv_q8_f32(x, wq, scale)
    assert np.array_equal(got.view(np.uint32), oracle.c.gemv_f32(x, w32).view(np.uint32))       # pinned in test_oracle_matmul.py
    f64 = (wq.view(np.uint8).reshape(29, 160).astype(np.float64) - 127) * np.repeat(scale.astype(np.float64), 32, axis=1)
    bound = (np.abs(f64) @ np.abs(x.astype(np.float64))) * 160 * 2.0 ** -24
    assert (np.abs(got.astype(np.float64) - f64 @ x.astype(np.float64)) <= bound).all()
    for k in (0, 31, 32, 159):                                                                   # one-hot x: a column of W, exact
        e = np.zeros(160, np.float32)
        e[k] = 1
        assert np.array_equal(oracle.c.gemv_q8_f32(e, wq, scale).view(np.uint32), w32[:, k].view(np.uint32))
    # the product must round: byte 130 (q = 3) times fp32(1/3)
    w = np.full((1, 8), 0x82828282, np.uint32)
    s = np.array([[np.float32(1) / np.float32(3)]], np.float32)
    e = np.zeros(32, np.float32)
    e[5] = 1
    assert oracle.c.gemv_q8_f32(e, w, s)[0] == np.float32(3) * s[0, 0]

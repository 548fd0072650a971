"""Pins the GEMV / GEMM part of the CPU oracle: float64 product, exact special cases,
brute force on tiny ragged shapes, torch CPU matmul, and the literal fp16-accumulate order."""
import numpy as np
import pytest
import torch

RTOL = 1e-2


def _close(got, want, rtol=RTOL, atol=2e-3):
    got, want = got.astype(np.float64), np.asarray(want, np.float64)
    return np.all(np.abs(got - want) <= atol + rtol * np.abs(want))


def _inputs(M, N, K, seed=6):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((M, K)).astype(np.float16), (rng.standard_normal((N, K)) * 0.02).astype(np.float16)


@pytest.mark.parametrize("M,N,K", [(1, 64, 4096), (1, 33, 1000), (5, 7, 3), (16, 48, 256), (3, 130, 520)])
def test_gemm_against_float64_and_torch(oracle, M, N, K):
    a, w = _inputs(M, N, K)
    got = oracle.c.gemm(a, w)
    assert _close(got, oracle.np64.gemm(a, w))
    ref = (torch.from_numpy(a).float() @ torch.from_numpy(w).float().T).numpy()
    assert _close(got, ref)
    # W is [N, K] and is used transposed: a transposed-operand mistake fails on a ragged shape
    assert got.shape == (M, N)


def test_gemm_exact_cases(oracle):
    rng = np.random.default_rng(1)
    # K = 1: each output is one fp16 x fp16 product, exact in fp32, rounded once
    a = rng.standard_normal((4, 1)).astype(np.float16)
    w = rng.standard_normal((6, 1)).astype(np.float16)
    want = (a.astype(np.float32) * w.astype(np.float32).T).astype(np.float16)
    assert np.array_equal(oracle.c.gemm(a, w).view(np.uint16), want.view(np.uint16))
    # identity W returns A bit for bit; a permutation of W's rows permutes C's columns
    a = rng.standard_normal((5, 32)).astype(np.float16)
    eye = np.eye(32, dtype=np.float16)
    assert np.array_equal(oracle.c.gemm(a, eye).view(np.uint16), a.view(np.uint16))
    perm = rng.permutation(32)
    assert np.array_equal(oracle.c.gemm(a, eye[perm].copy()).view(np.uint16), a[:, perm].view(np.uint16))
    # one-hot x selects a column of W^T exactly (GEMV)
    w = (rng.standard_normal((9, 64)) * 0.02).astype(np.float16)
    x = np.zeros((1, 64), np.float16)
    x[0, 17] = 1
    assert np.array_equal(oracle.c.gemm(x, w).view(np.uint16).ravel(), w[:, 17].view(np.uint16))


def test_gemm_bias_is_added_after_rounding(oracle):
    a, w = _inputs(3, 10, 64)
    bias = np.linspace(-1, 1, 10).astype(np.float16)
    base = oracle.c.gemm(a, w)
    want = (base.astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
    assert np.array_equal(oracle.c.gemm(a, w, bias).view(np.uint16), want.view(np.uint16))


def test_gemm_brute_force_python_loops(oracle):
    a, w = _inputs(2, 3, 5, seed=8)
    got32 = oracle.c.gemm_f32out(a, w)
    for i in range(2):
        for j in range(3):
            acc = np.float32(0)
            for k in range(5):
                acc = np.float32(acc + np.float32(a[i, k]) * np.float32(w[j, k]))
            assert got32[i, j] == acc
            assert oracle.c.gemm(a, w)[i, j] == np.float16(acc)


def test_fp16_accumulate_follows_the_primfunc_text(oracle):
    # acc = f16(acc + f16(a*w)), k ascending (before_dl.py:96-113 keeps the sum in an fp16 buffer)
    a, w = _inputs(2, 4, 40, seed=9)
    got = oracle.c.gemm(a, w, acc_f16=True)
    for i in range(2):
        for j in range(4):
            acc = np.float16(0)
            for k in range(40):
                acc = np.float16(acc + np.float16(a[i, k] * w[j, k]))
            assert got[i, j] == acc
    # and it differs from fp32 accumulation on long sums (so the two modes are really distinct)
    a, w = _inputs(1, 64, 4096, seed=10)
    assert not np.array_equal(oracle.c.gemm(a, w, acc_f16=True), oracle.c.gemm(a, w))


def test_fp16_accumulator_rounded_once_per_k_step_of_16(oracle):
    """acc_f16 = 2 restates the reference's scheduled GEMM: an fp16 accumulator fragment updated once per k step of
    16 (experiment/testIR/GEMM/m_n2560_k10240/wmma/16x16x16/i2j4_x7y2_in8.py:19,37).  Pinned without repeating
    the formula: by results that only this grouping gives."""
    # (1) up to 16 terms there is one step: the fp32 sum rounded once, i.e. the fp32-accumulate mode bit for bit
    for K in (1, 7, 16):
        a, w = _inputs(3, 5, K, seed=20 + K)
        assert np.array_equal(oracle.c.gemm(a, w, acc_f16=2).view(np.uint16), oracle.c.gemm(a, w).view(np.uint16))
    # (2) where the accumulator stalls tells the step length: every product is 1/16, so a step of g terms adds g/16,
    # and an fp16 sum stops growing where half its spacing reaches the increment (ties go to the even neighbour):
    # one term at a time at 128, steps of 8 at 1024, of 16 at 2048, of 32 at 4096; fp32 accumulation reaches K/16
    K = 16 * 8192
    a = np.ones((1, K), np.float16)
    w = np.full((1, K), 1 / 16, np.float16)
    assert float(oracle.c.gemm(a, w, acc_f16=2)[0, 0]) == 2048.0
    assert float(oracle.c.gemm(a, w, acc_f16=1)[0, 0]) == 128.0
    assert float(oracle.c.gemm(a, w)[0, 0]) == 8192.0
    # (3) inside a step the sum is not rounded: 2048 + sixteen 1s in one step is 2064 (one at a time each would be lost),
    # and the steps are aligned at multiples of 16 from k = 0: eight 1s at the end of a step and eight at the start of
    # the next are two ties, both lost
    def run(entries, K=48):
        wv = np.zeros((1, K), np.float16)
        for k, v in entries:
            wv[0, k] = v
        return float(oracle.c.gemm(np.ones((1, K), np.float16), wv, acc_f16=2)[0, 0])
    assert run([(0, 2048)] + [(k, 1) for k in range(16, 32)]) == 2064.0
    assert run([(0, 2048)] + [(k, 1) for k in range(24, 32)]) == 2056.0      # eight in one step: 2056 is representable
    assert run([(0, 2048)] + [(k, 1) for k in range(31, 33)]) == 2048.0      # one in each of two steps: each a tie, lost
    assert run([(0, 2048)] + [(k, 1) for k in range(30, 32)]) == 2050.0      # the same two inside one step survive
    # (4) the fused form takes its product from the same sum, and a K that is not a multiple of 16 ends with a short step
    a, w = _inputs(4, 6, 200, seed=31)
    bias = np.linspace(-1, 1, 6).astype(np.float16)
    plain = oracle.c.gemm(a, w, bias, acc_f16=2)
    assert np.array_equal(oracle.c.gemm_fused(a, w, bias, None, None, 0, acc_f16=2).view(np.uint16), plain.view(np.uint16))
    f64 = a.astype(np.float64) @ w.astype(np.float64).T + bias.astype(np.float64)
    assert np.abs(plain.astype(np.float64) - f64).max() < 0.05 * max(1.0, np.abs(f64).max())
    head = oracle.c.gemm(a[:, :192].copy(), w[:, :192].copy(), acc_f16=2).astype(np.float32)
    tail = (a[:, 192:].astype(np.float32)[:, None, :] * w[:, 192:].astype(np.float32)[None, :, :])
    want = head.copy()
    for k in range(8):
        want = want + tail[:, :, k]
    assert np.array_equal(oracle.c.gemm(a, w, acc_f16=2), want.astype(np.float16))


def test_gemv_rf_follows_the_order_of_the_reference_schedule(oracle):
    """oracle.c.gemv_rf restates experiment/testIR/GEMV/m1n2560k10240/IR/5wt.py:11-92.  Each case below has a result
    that one stage's order fixes: 2048 + 1 is a tie in fp16 (spacing 2) and rounds back to 2048, so ones added one at
    a time vanish, ones added to each other first survive."""
    def run(K, entries, x_entries=()):
        w = np.zeros((1, K), np.float16)
        x = np.ones(K, np.float16)
        for k, v in entries:
            w[0, k] = v
        for k, v in x_entries:
            x[k] = v
        return float(oracle.c.gemv_rf(x, w)[0])
    # stage 1, one strided chain (k = j, 256 + j, 512 + j), ascending: (2048 + 1) + 1 = 2048; descending would give 2050
    assert run(768, [(0, 2048), (256, 1), (512, 1)]) == 2048.0
    assert run(768, [(0, 1), (256, 1), (512, 2048)]) == 2050.0
    # stage 2, the 8 chains of one lane, ascending from 0: ones after 2048 vanish; a pairwise fold would keep two of them
    assert run(256, [(0, 2048), (1, 1), (2, 1), (3, 1), (4, 1)]) == 2048.0
    assert run(256, [(0, 1), (1, 1), (2, 1), (3, 1), (4, 2048)]) == 2052.0
    # stage 3, the 32 lanes (lane t owns k = 8t .. 8t+7), shuffle tree with strides 16, 8, 4, 2, 1:
    # lanes 0..3 = 2048, 1, 1, 1: stride 2 gives lane 0 = 2048 + 1 = 2048 and lane 1 = 1 + 1, stride 1 adds them: 2050
    # (a left-to-right sum would give 2048)
    assert run(256, [(0, 2048), (8, 1), (16, 1), (24, 1)]) == 2050.0
    # lanes 0, 16, 17 = 2048, 1, 1: stride 16 comes first, lane 0 = 2048 + 1 = 2048, lane 1 = 0 + 1, then 2048 + 1 = 2048
    # (strides 1, 2, ..., 16 would join lanes 16 and 17 first: 2050)
    assert run(256, [(0, 2048), (128, 1), (136, 1)]) == 2048.0
    # the product is rounded before it is added: (1 + 2^-10)(1 - 2^-11) = 1.000488 rounds to 1, and 2048 + 1 = 2048;
    # a fused multiply-add would see 2049.000488 and give 2050
    assert run(512, [(0, 2048), (256, 1 - 2.0 ** -11)], [(256, 1 + 2.0 ** -10)]) == 2048.0
    # small integers: exact whatever the order; bias added last, in fp16; K that is no multiple of 256
    rng = np.random.default_rng(12)
    xi, wi = rng.integers(-2, 3, 1000).astype(np.float16), rng.integers(-2, 3, (37, 1000)).astype(np.float16)
    bi = rng.integers(-4, 5, 37).astype(np.float16)
    assert np.array_equal(oracle.c.gemv_rf(xi, wi, bi).astype(np.float64), wi.astype(np.float64) @ xi.astype(np.float64) + bi)
    # random data: within fp16 accumulation error of the exact product, and not the fp32-accumulated result
    x, w = (rng.standard_normal(10240) * 0.5).astype(np.float16), (rng.standard_normal((64, 10240)) * 0.05).astype(np.float16)
    got, f64 = oracle.c.gemv_rf(x, w, threads=4).astype(np.float64), w.astype(np.float64) @ x.astype(np.float64)
    assert np.abs(got - f64).max() < 0.05
    assert not np.array_equal(oracle.c.gemv_rf(x, w), oracle.c.gemm(x[None, :], w)[0])
    assert np.array_equal(oracle.c.gemv_rf(x, w, threads=1).view(np.uint16), oracle.c.gemv_rf(x, w, threads=4).view(np.uint16))


def test_threads_do_not_change_bits(oracle):
    a, w = _inputs(7, 33, 100)
    assert np.array_equal(oracle.c.gemm(a, w, threads=1).view(np.uint16), oracle.c.gemm(a, w, threads=4).view(np.uint16))


# ---- fp32 GEMV: NT_matmul5 (before_dl.py:8-19) ----------------------------------------------------------

def test_gemv_f32_closed_forms_and_exact_cases(oracle):
    rng = np.random.default_rng(31)
    x = rng.standard_normal(2560).astype(np.float32)
    w = (rng.standard_normal((97, 2560)) * 0.02).astype(np.float32)
    got = oracle.c.gemv_f32(x, w)
    f64 = w.astype(np.float64) @ x.astype(np.float64)
    bound = (np.abs(w.astype(np.float64)) @ np.abs(x.astype(np.float64))) * 2560 * 2.0 ** -24      # a running fp32 sum of K terms
    assert got.dtype == np.float32 and (np.abs(got - f64) <= bound).all()
    assert (np.abs(got - f64) <= 1e-5 * np.abs(f64) + 1e-5).all()
    # short rows: numpy's float32 dot product has the same few roundings
    assert np.allclose(oracle.c.gemv_f32(x[:8], np.ascontiguousarray(w[:, :8])), w[:, :8] @ x[:8], rtol=1e-6, atol=1e-7)
    # one-hot x returns a column of W exactly; K = 1 is one rounded product; small integers are exact
    for k in (0, 1, 2559):
        e = np.zeros(2560, np.float32)
        e[k] = 1
        assert np.array_equal(oracle.c.gemv_f32(e, w), w[:, k])
    assert np.array_equal(oracle.c.gemv_f32(np.float32([3.1]), np.float32([[0.7], [-2.0]])), np.float32([3.1]) * np.float32([0.7, -2.0]))
    xi = rng.integers(-8, 9, 64).astype(np.float32)
    wi = rng.integers(-8, 9, (5, 64)).astype(np.float32)
    assert np.array_equal(oracle.c.gemv_f32(xi, wi), (wi.astype(np.int64) @ xi.astype(np.int64)).astype(np.float32))
    assert np.array_equal(oracle.c.gemv_f32(x, w, threads=4), got)                               # rows are independent

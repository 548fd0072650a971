"""Pins oracle_attn_scores_f16_f32 (fused_NT_matmul1_divide_maximum_minimum_cast2, before_dl.py:116-160)
without the reference: numpy float16 arithmetic step by step, the float64 closed form, mask cases."""
import numpy as np

SCALE = 0.11179039301310044   # the constant in the PrimFunc: 1 / sqrt(80) rounded as written there


def _inputs(heads, n, m, d, seed):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((heads, n, d)).astype(np.float16)
    k = rng.standard_normal((heads, m, d)).astype(np.float16)
    mask = np.where(np.arange(m)[None, :] <= np.arange(n)[:, None] + (m - n), 65504.0, -65504.0).astype(np.float16)
    return q, k, mask


def test_matches_numpy_float16_step_by_step(oracle):
    q, k, mask = _inputs(3, 9, 13, 80, 1)
    got = oracle.c.attn_scores(q, k, mask, SCALE)
    mm = np.stack([oracle.c.gemm(q[h], k[h]) for h in range(3)])        # pinned in test_oracle_matmul.py
    t = (mm * np.float16(SCALE)).astype(np.float16)
    t = np.maximum(t, np.float16(-65504))
    t = np.minimum(t, mask[None])
    assert got.dtype == np.float32 and np.array_equal(got.view(np.uint32), t.astype(np.float32).view(np.uint32))


def test_close_to_float64_and_mask_semantics(oracle):
    q, k, mask = _inputs(2, 16, 16, 80, 2)
    got = oracle.c.attn_scores(q, k, mask, SCALE).astype(np.float64)
    want = oracle.np64.attn_scores(q, k, mask, SCALE)
    assert (np.abs(got - want) <= 2e-3 + 2e-3 * np.abs(want)).all()
    upper = np.triu(np.ones((16, 16), bool), 1)
    assert (got[:, upper] == -65504.0).all()                             # the causal triangle is masked out
    open_mask = np.full((16, 16), 65504.0, np.float16)
    free = oracle.c.attn_scores(q, k, open_mask, SCALE)
    assert np.array_equal(free[:, ~upper], oracle.c.attn_scores(q, k, mask, SCALE)[:, ~upper])
    shut = oracle.c.attn_scores(q, k, np.full((16, 16), -65504.0, np.float16), SCALE)
    assert (shut == -65504.0).all()
    # heads are independent
    assert np.array_equal(oracle.c.attn_scores(q[1:], k[1:], mask, SCALE)[0], oracle.c.attn_scores(q, k, mask, SCALE)[1])


def test_overflowing_products_are_clamped(oracle):
    q = np.full((1, 2, 8), 200.0, np.float16)
    k = np.ascontiguousarray(np.stack([np.full(8, 200.0, np.float16), np.full(8, -200.0, np.float16)])[None])
    open_mask = np.full((2, 2), 65504.0, np.float16)
    got = oracle.c.attn_scores(q, k, open_mask, 1.0)
    # 8 * 200 * 200 = 320000 overflows fp16 to +-inf; min(+inf, 65504) = 65504, max(-inf, -65504) = -65504
    assert (got[0, :, 0] == 65504.0).all() and (got[0, :, 1] == -65504.0).all()


# ---- P.V: matmul8 / matmul10 (before_dl.py:915-929, :899-912) --------------------------------------------

def _pv_inputs(heads, n, m, d, seed):
    rng = np.random.default_rng(seed)
    p = rng.random((heads, n, m)).astype(np.float32)
    p = (p / np.maximum(p.sum(-1, keepdims=True), 1e-6)).astype(np.float16)       # rows like a softmax's
    v = rng.standard_normal((heads, m, d)).astype(np.float16)
    return p, v


def test_pv_close_to_float64_matmul(oracle):
    p, v = _pv_inputs(3, 7, 29, 80, 11)
    got = oracle.c.attn_pv(p, v).astype(np.float64)
    want = oracle.np64.attn_pv(p, v)
    assert (np.abs(got - want) <= 1e-3 + 1e-3 * np.abs(want)).all()
    # the transposed GEMM oracle (pinned in test_oracle_matmul.py) gives the same bits: out = P . (V^T)^T
    for h in range(3):
        assert np.array_equal(oracle.c.attn_pv(p, v)[h].view(np.uint16),
                              oracle.c.gemm(p[h], np.ascontiguousarray(v[h].T)).view(np.uint16))


def test_pv_selectors_pick_rows_of_v_exactly(oracle):
    _, v = _pv_inputs(2, 1, 12, 16, 12)
    eye = np.ascontiguousarray(np.broadcast_to(np.eye(12, dtype=np.float16), (2, 12, 12)))
    assert np.array_equal(oracle.c.attn_pv(eye, v).view(np.uint16), v.view(np.uint16))   # a transposed operand would fail
    pick = np.zeros((2, 3, 12), np.float16)
    pick[:, 0, 5] = pick[:, 1, 0] = pick[:, 2, 11] = 1
    assert np.array_equal(oracle.c.attn_pv(pick, v), v[:, [5, 0, 11], :])
    # heads are independent; n = 1 (matmul10) is a row of the n > 1 case
    p, v = _pv_inputs(4, 5, 9, 8, 13)
    full = oracle.c.attn_pv(p, v)
    assert np.array_equal(oracle.c.attn_pv(p[2:3], v[2:3])[0], full[2])
    assert np.array_equal(oracle.c.attn_pv(np.ascontiguousarray(p[:, 3:4]), v)[:, 0], full[:, 3])


def test_pv_means_linearity_and_empty_sum(oracle):
    rng = np.random.default_rng(14)
    v = rng.integers(-8, 9, (2, 16, 24)).astype(np.float16)                       # exactly representable sums
    mean_row = np.full((2, 1, 16), 1.0 / 16, np.float16)
    assert np.array_equal(oracle.c.attn_pv(mean_row, v)[:, 0].astype(np.float64), v.astype(np.float64).mean(1))
    a = rng.integers(0, 4, (2, 3, 16)).astype(np.float16)
    b = rng.integers(0, 4, (2, 3, 16)).astype(np.float16)
    assert np.array_equal(oracle.c.attn_pv(a + b, v).astype(np.float32),
                          oracle.c.attn_pv(a, v).astype(np.float32) + oracle.c.attn_pv(b, v).astype(np.float32))
    empty = oracle.c.attn_pv(np.zeros((2, 3, 0), np.float16), np.zeros((2, 0, 8), np.float16))
    assert empty.shape == (2, 3, 8) and (empty == 0).all()


def test_pv_fp16_running_sum_is_the_literal_reading(oracle):
    # 2048 + 1 is not representable in fp16: the literal fp16 accumulator stalls, the fp32 one does not
    p = np.ones((1, 1, 2100), np.float16)
    v = np.ones((1, 2100, 8), np.float16)
    assert (oracle.c.attn_pv(p, v, acc_f16=True) == 2048).all()
    assert (oracle.c.attn_pv(p, v) == np.float16(2100)).all()

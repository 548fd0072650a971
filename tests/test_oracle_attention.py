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

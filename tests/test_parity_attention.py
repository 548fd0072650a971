"""GPU parity of the attention-scores kernel (fused_NT_matmul1_divide_maximum_minimum_cast2) through the C
ABI against the CPU oracle: scale, clamp and mask act on fp16 values, so apart from an fp16 ulp of the product
(fp32 summation order) the result is bit-identical."""
import numpy as np
import pytest
import torch

from dtas_amd import _lib, ops
from gpu_util import Guarded, cfg, dev

pytestmark = pytest.mark.gpu
SCALE = 0.11179039301310044


def _inputs(heads, n, m, d, seed):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((heads, n, d)).astype(np.float16)
    k = rng.standard_normal((heads, m, d)).astype(np.float16)
    mask = np.where(np.arange(m)[None, :] <= np.arange(n)[:, None] + (m - n), 65504.0, -65504.0).astype(np.float16)
    return q, k, mask


def _check(got, q, k, mask, oracle):
    want = oracle.c.attn_scores(q, k, mask, SCALE, threads=8)
    f64 = oracle.np64.attn_scores(q, k, mask, SCALE)
    assert np.isfinite(got).all()
    assert (np.abs(got.astype(np.float64) - f64) <= 2e-3 + 1e-2 * np.abs(f64)).all()
    assert (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 1e-3 + 2.0 ** -9 * np.abs(want)).all()
    assert (got == want).mean() > 0.98
    assert np.array_equal(got == -65504.0, want == -65504.0)            # the masked set is exact


@pytest.mark.parametrize("n,m", [(1, 1), (1, 77), (5, 5), (64, 64), (130, 200), (257, 513), (1024, 1024)])
def test_scores_builtin_config(oracle, n, m):
    q, k, mask = _inputs(32, n, m, 80, n + m)
    out = Guarded((1, 32, n, m), torch.float32)
    ops.attn_scores(dev(q).view(1, 32, n, 80), dev(k).view(1, 32, m, 80), dev(mask).view(1, 1, n, m), out.t, SCALE)
    _check(out.check().reshape(32, n, m), q, k, mask, oracle)


@pytest.mark.parametrize("tile,block,stages", [((64, 64), 256, 2), ((64, 64), 256, 3), ((128, 128), 256, 2), ((128, 64), 256, 2),
                                               ((64, 128), 256, 2), ((256, 128), 256, 2), ((256, 256), 512, 2), ((256, 256), 256, 2)])
@pytest.mark.parametrize("heads,n,m,d", [(3, 70, 131, 80), (2, 300, 260, 64), (1, 33, 7, 8)])
def test_scores_every_tile(oracle, tile, block, stages, heads, n, m, d):
    q, k, mask = _inputs(heads, n, m, d, n + m + d)
    out = Guarded((heads, n, m), torch.float32)
    ops.attn_scores(dev(q), dev(k), dev(mask), out.t, SCALE,
                    cfg(variant=_lib.GEMM_MFMA, block=block, vec=8, unroll=stages, tile=[tile[0], tile[1], 64]))
    _check(out.check(), q, k, mask, oracle)


def test_scores_errors():
    q, k, mask = _inputs(2, 8, 8, 80, 1)
    out = torch.empty(2, 8, 8, dtype=torch.float32, device="cuda")
    with pytest.raises(_lib.DtasError, match="not split"):
        ops.attn_scores(dev(q), dev(k), dev(mask), out, SCALE, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=2, tile=[64, 64, 64], split_k=2))
    q7 = np.zeros((2, 8, 12), np.float16)
    with pytest.raises(_lib.DtasError, match="multiple of 8"):
        ops.attn_scores(dev(q7), dev(q7), dev(mask), out, SCALE)
    assert _lib.lib().dtas_attn_scores_f16_f32(None, None, None, None, 0, 0, 0, 80, SCALE, None, None) == 0   # empty: no-op


def test_scores_through_the_primfunc_descriptor(oracle):
    from dtas_amd import primfuncs as pf
    from dtas_amd.codegen.runtime_packer import bind_extents, call_primfunc

    func = pf.fused_NT_matmul_divide_maximum_minimum_cast(32, 80)
    q, k, mask = _inputs(32, 40, 56, 80, 9)
    out = torch.empty(1, 32, 40, 56, dtype=torch.float32, device="cuda")
    tensors = (dev(q).view(1, 32, 40, 80), dev(k).view(1, 32, 56, 80), dev(mask).view(1, 1, 40, 56), out)
    assert bind_extents(func, tensors) == {"n": 40, "m": 56}
    call_primfunc(func, tensors)
    torch.cuda.synchronize()
    _check(out.cpu().numpy().reshape(32, 40, 56), q, k, mask, oracle)

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


@pytest.mark.parametrize("heads,n,m,d", [(3, 70, 131, 8), (2, 129, 65, 64), (5, 300, 260, 128), (2, 100, 90, 136), (1, 1, 3, 72),
                                         (40, 520, 512, 80), (3, 1300, 1700, 80), (2, 2049, 1030, 80), (40, 520, 512, 96), (9, 700, 2048, 80),
                                         (12, 1300, 1712, 96)])
def test_scores_builtin_other_head_dims(oracle, heads, n, m, d):
    # d <= 128 is served by the kernel that walks tiles (one or two k tiles), beyond that by the general one;
    # 40 heads x 5 x 8 tiles = 1600 tiles: more than one tile per workgroup; from 2 M scores per head on an XCD keeps a
    # span of tiles and walks the heads: 11 x 27 and 17 x 17 tiles do not divide by the 8 XCDs (spans of unequal length);
    # d = 80 and 96 with rows of whole 64-byte sectors (m % 16 == 0) take the two-deep pipeline (tails of 16 / 32 elements)
    q, k, mask = _inputs(heads, n, m, d, n + m + d)
    out = Guarded((heads, n, m), torch.float32)
    ops.attn_scores(dev(q), dev(k), dev(mask), out.t, SCALE)
    _check(out.check(), q, k, mask, oracle)


@pytest.mark.parametrize("tile,block,stages", [((64, 64), 256, 2), ((64, 64), 256, 3), ((128, 128), 256, 2), ((128, 64), 256, 2),
                                               ((64, 128), 256, 2), ((256, 128), 256, 2), ((256, 256), 512, 2), ((256, 256), 256, 2)])
@pytest.mark.parametrize("heads,n,m,d", [(3, 70, 131, 80), (2, 300, 260, 64), (1, 33, 7, 8)])
def test_scores_every_tile(oracle, tile, block, stages, heads, n, m, d):
    q, k, mask = _inputs(heads, n, m, d, n + m + d)
    out = Guarded((heads, n, m), torch.float32)
    ops.attn_scores(dev(q), dev(k), dev(mask), out.t, SCALE,
                    cfg(variant=_lib.GEMM_MFMA, block=block, vec=8, unroll=stages, tile=[tile[0], tile[1], 64]))
    _check(out.check(), q, k, mask, oracle)


@pytest.mark.parametrize("rows", [1, 2, 4, 8])
@pytest.mark.parametrize("heads,n,m,d,keys", [(32, 1, 2048, 80, 0), (3, 1, 515, 80, 102), (2, 3, 77, 64, 0), (2, 8, 1000, 128, 128), (1, 5, 1, 16, 0),
                                              (2, 2, 300, 136, 60), (1, 9, 4100, 8, 1024), (1, 2, 260, 1024, 8)])
def test_scores_row_kernel(oracle, rows, heads, n, m, d, keys):
    # a workgroup of 1024 threads sweeps a run of the head's keys for 1, 2, 4 or 8 query rows (d / 8 = 1 .. 128 threads
    # per key; keys per workgroup given or chosen; more query rows than a workgroup takes: further workgroups)
    q, k, mask = _inputs(heads, n, m, d, rows + n + m + d)
    out = Guarded((heads, n, m), torch.float32)
    ops.attn_scores(dev(q), dev(k), dev(mask), out.t, SCALE, cfg(variant=_lib.GEMM_SKINNY, block=1024, vec=8, tile=[rows, 8, keys]))
    _check(out.check(), q, k, mask, oracle)


def test_scores_row_kernel_is_the_choice_for_one_and_two_rows_and_refuses_what_it_cannot_hold(oracle):
    for n, m in ((1, 2048), (2, 700), (3, 3100), (4, 3072)):
        q, k, mask = _inputs(32, n, m, 80, n + m)
        out = Guarded((32, n, m), torch.float32)
        ops.attn_scores(dev(q), dev(k), dev(mask), out.t, SCALE)
        _check(out.check(), q, k, mask, oracle)
    q, k, mask = _inputs(2, 2, 64, 80, 1)
    out = Guarded((2, 2, 64), torch.float32)
    for bad in (dict(block=256, tile=[1, 8, 0]), dict(block=1024, tile=[3, 8, 0]), dict(block=1024, tile=[2, 8, 50]), dict(block=1024, tile=[2, 16, 0])):
        with pytest.raises(_lib.DtasError):
            ops.attn_scores(dev(q), dev(k), dev(mask), out.t, SCALE, cfg(variant=_lib.GEMM_SKINNY, vec=8, **bad))


def test_scores_errors():
    q, k, mask = _inputs(2, 8, 8, 80, 1)
    out = torch.empty(2, 8, 8, dtype=torch.float32, device="cuda")
    with pytest.raises(_lib.DtasError, match="not split"):
        ops.attn_scores(dev(q), dev(k), dev(mask), out, SCALE, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=2, tile=[64, 64, 64], split_k=2))
    q7 = np.zeros((2, 8, 12), np.float16)
    with pytest.raises(_lib.DtasError, match="multiple of 8"):
        ops.attn_scores(dev(q7), dev(q7), dev(mask), out, SCALE)
    assert _lib.lib().dtas_attn_scores_f16_f32(None, None, None, None, 0, 0, 0, 80, SCALE, None, None) == 0   # empty: no-op


def test_scores_with_an_empty_head_dimension():
    # d = 0: every product is an empty sum, so out = min(max(0, -65504), mask); one query row reaches the built-in
    # choice that takes the row kernel for d >= 8 (its launch shape divides by d / 8)
    for n, m in ((1, 40), (3, 4096), (70, 33)):
        rng = np.random.default_rng(n)
        mask = np.where(rng.random((n, m)) < 0.5, 65504.0, -65504.0).astype(np.float16)
        dummy = torch.zeros(8, dtype=torch.float16, device="cuda")
        out = torch.full((2, n, m), 7.0, dtype=torch.float32, device="cuda")
        mask_d = dev(mask)
        rc = _lib.lib().dtas_attn_scores_f16_f32(dummy.data_ptr(), dummy.data_ptr(), mask_d.data_ptr(), out.data_ptr(), 2, n, m, 0,
                                                 SCALE, None, None)
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        want = np.minimum(np.float32(0), mask.astype(np.float32))
        assert np.array_equal(out.cpu().numpy(), np.broadcast_to(want, (2, n, m)))


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


# ---- P.V: matmul8 / matmul10 (before_dl.py:915-929, :899-912) --------------------------------------------

def _pv_inputs(heads, n, m, d, seed):
    rng = np.random.default_rng(seed)
    p = rng.random((heads, n, m)).astype(np.float32)
    p = (p / np.maximum(p.sum(-1, keepdims=True), 1e-6)).astype(np.float16)       # rows like a softmax's
    v = rng.standard_normal((heads, m, d)).astype(np.float16)
    return p, v


def _check_pv(got, p, v, oracle):
    want = oracle.c.attn_pv(p, v, threads=8)
    f64 = oracle.np64.attn_pv(p, v)
    assert np.isfinite(got).all()
    assert (np.abs(got.astype(np.float64) - f64) <= 1e-3 + 1e-2 * np.abs(f64)).all()     # rtol 1e-2 against float64
    assert (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 1e-4 + 2.0 ** -9 * np.abs(want)).all()
    if got.size:
        assert (got == want).mean() > 0.97      # the rest: one fp16 ulp from the fp32 summation order


@pytest.mark.parametrize("n,m", [(1, 1), (1, 77), (1, 2048), (3, 300), (8, 129), (9, 64), (9, 77), (64, 64), (130, 200),
                                 (257, 520), (1024, 1024),
                                 # the fitted choice of tile and key split up to one 128-row tile per CU: 64x64 whole and in parts,
                                 # 64x128 in 2 / 4 / 8 parts, 128x128 in 2 parts
                                 (128, 128), (64, 1024), (256, 1024), (256, 4096), (128, 4100), (16, 8192), (384, 4096), (192, 2049),
                                 # 256-row tiles would make one round and a thin second one: 64-row tiles (1.125 rounds), 128-row (1.5)
                                 (2304, 512), (3072, 256)])
def test_pv_builtin_config(oracle, n, m):
    p, v = _pv_inputs(32, n, m, 80, 3 * n + m)
    out = Guarded((1, 32, n, 80), torch.float16)
    ops.attn_pv(dev(p).view(1, 32, n, m), dev(v).view(1, 32, m, 80), out.t)
    _check_pv(out.check().reshape(32, n, 80), p, v, oracle)


@pytest.mark.parametrize("heads,n,m,d", [(40, 1, 2048, 128), (64, 1, 2048, 128), (40, 8, 2048, 128), (16, 8, 8192, 128), (40, 2, 8192, 128),
                                         (32, 4, 4096, 128), (32, 2, 8192, 128), (64, 12, 1024, 128), (40, 1, 520, 128), (40, 1, 1001, 96)])
def test_pv_few_rows_with_other_head_counts_and_dimensions(oracle, heads, n, m, d):
    # the choice between the row kernels and the tiles goes with heads x head dimension: one row on the tiles with their
    # keys in parts (40 and 64 heads of 128), the tiles instead of the row kernel or of the sweep in key runs, and the
    # cases that stay on those
    p, v = _pv_inputs(heads, n, m, d, heads + n + m)
    out = Guarded((1, heads, n, d), torch.float16)
    ops.attn_pv(dev(p).view(1, heads, n, m), dev(v).view(1, heads, m, d), out.t)
    _check_pv(out.check().reshape(heads, n, d), p, v, oracle)


@pytest.mark.parametrize("tile,stages", [((64, 64), 2), ((64, 128), 2), ((64, 128), 3), ((128, 64), 2), ((128, 128), 2), ((128, 128), 3), ((256, 128), 3)])
@pytest.mark.parametrize("heads,n,m,d", [(2, 1, 264, 128), (3, 70, 136, 80), (2, 300, 264, 64), (1, 33, 8, 8), (2, 50, 72, 136), (1, 129, 1032, 128),
                                         (2, 260, 64, 80), (2, 20, 128, 80), (1, 515, 192, 80)])
def test_pv_every_tile(oracle, tile, stages, heads, n, m, d):
    # m = 8 .. 1032: one k tile, two, three (every prologue / drain case of the two- and three-stage pipelines), many
    p, v = _pv_inputs(heads, n, m, d, n + m + d)
    out = Guarded((heads, n, d), torch.float16)
    ops.attn_pv(dev(p), dev(v), out.t, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=stages, tile=[tile[0], tile[1], 64]))
    _check_pv(out.check(), p, v, oracle)


@pytest.mark.parametrize("tile,stages,split", [((64, 128), 2, 2), ((64, 128), 2, 16), ((64, 64), 2, 3), ((128, 128), 3, 4), ((256, 128), 3, 2)])
@pytest.mark.parametrize("heads,n,m,d", [(32, 16, 2048, 80), (3, 70, 1032, 80), (2, 5, 64, 64), (1, 130, 8192, 128)])
def test_pv_split_over_workgroups(oracle, tile, stages, split, heads, n, m, d):
    """Few query rows against many keys: the workgroups of a (head, tile) split m and meet in the workspace; the
    partials are added in split order, so two runs give the same bits, and the counters re-arm themselves."""
    p, v = _pv_inputs(heads, n, m, d, n + m + d + split)
    row = cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=stages, tile=[tile[0], tile[1], 64], split_k=split)
    first = None
    for _ in range(2):
        out = Guarded((heads, n, d), torch.float16)
        ops.attn_pv(dev(p), dev(v), out.t, row)
        got = out.check()
        _check_pv(got, p, v, oracle)
        assert first is None or np.array_equal(first, got)
        first = got


@pytest.mark.parametrize("tile,stages", [((64, 128), 3), ((128, 128), 2), ((128, 128), 3), ((256, 128), 3), ((64, 64), 2)])
@pytest.mark.parametrize("heads,n,m,d", [(5, 300, 2048, 80), (3, 130, 2049, 80), (2, 70, 4096, 128), (3, 260, 2056, 80), (7, 64, 2048, 64)])
def test_pv_with_rows_of_p_a_multiple_of_4_kib_apart(oracle, tile, stages, heads, n, m, d):
    """Key counts whose rows of P lie (nearly) a multiple of 4 KiB apart: every workgroup starts its walk over the keys
    at a k tile of its own and wraps around (the last, partial k tile and the m % 8 tail then come mid-walk).  The
    order is a function of the tile, so two runs give the same bits."""
    p, v = _pv_inputs(heads, n, m, d, n + m + d)
    row = cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=stages, tile=[tile[0], tile[1], 64])
    first = None
    for _ in range(2):
        out = Guarded((heads, n, d), torch.float16)
        ops.attn_pv(dev(p), dev(v), out.t, row)
        got = out.check()
        _check_pv(got, p, v, oracle)
        assert first is None or np.array_equal(first, got)
        first = got


@pytest.mark.parametrize("rows", [1, 2, 4, 8])
@pytest.mark.parametrize("heads,n,m,d", [(32, 1, 515, 80), (32, 1, 4096, 80), (3, 3, 64, 8), (2, 11, 1000, 128), (1, 8, 1, 16),
                                         (2, 5, 300, 264)])
def test_pv_row_kernel(oracle, rows, heads, n, m, d):
    p, v = _pv_inputs(heads, n, m, d, n + m + d + rows)
    out = Guarded((heads, n, d), torch.float16)
    ops.attn_pv(dev(p), dev(v), out.t, cfg(variant=_lib.GEMM_SKINNY, block=256, vec=8, unroll=1, tile=[rows, 8, 0]))
    _check_pv(out.check(), p, v, oracle)


@pytest.mark.parametrize("heads,n,m,d", [(32, 1, 515, 80), (32, 4, 2048, 80), (3, 3, 64, 8), (2, 8, 1000, 128), (1, 5, 1, 16), (2, 2, 77, 136),
                                         (2, 3, 9000, 64), (1, 7, 300, 1024)])
def test_pv_whole_row_kernel(oracle, heads, n, m, d):
    # one workgroup of 1024 threads per (head, query row): the head's V read as one contiguous run of 16-byte pieces,
    # d / 8 of them per key (1 .. 128: every thread count per key, idle threads at the end of the workgroup included);
    # or several workgroups per (head, row), each with an equal share of a key's pieces (tile[2] columns), 256 .. 1024 threads
    p, v = _pv_inputs(heads, n, m, d, heads + n + m + d)
    rng = np.random.default_rng(m)
    pi = rng.integers(0, 3, size=(heads, n, m)).astype(np.float16)
    vi = rng.integers(-3, 4, size=(heads, m, d)).astype(np.float16)
    want_i = np.einsum("hnm,hmd->hnd", pi.astype(np.float64), vi.astype(np.float64))
    shares = [(1024, 0, 1), (1024, d, 1), (1024, d, 2), (1024, 0, 8), (512, d, 64)]
    shares += [(block, d // parts, split) for block, parts, split in ((1024, 2, 1), (512, 2, 4), (256, d // 8, 1)) if (d // 8) % parts == 0]
    for block, cols, split in shares:  # (split: the workgroups of a (head, row) share the keys and meet in the workspace)
        if (cols or d) > block:
            continue  # (a thread per column of the workgroup's share)
        c = cfg(variant=_lib.GEMM_SKINNY, block=block, vec=8, tile=[1, 8, cols], split_k=split)
        out = Guarded((heads, n, d), torch.float16)
        ops.attn_pv(dev(p), dev(v), out.t, c)
        _check_pv(out.check(), p, v, oracle)
        ops.attn_pv(dev(pi), dev(vi), out.t, c)
        assert np.array_equal(out.check().astype(np.float64), want_i)
    out = Guarded((heads, n, d), torch.float16)
    for bad in (dict(block=1024, tile=[2, 8, 0]), dict(block=1024, tile=[1, 8, 12]), dict(block=128, tile=[1, 8, d]), dict(block=1024, tile=[1, 8, 2 * d]), dict(block=256, tile=[1, 8, d], split_k=128)):
        with pytest.raises(_lib.DtasError):
            ops.attn_pv(dev(p), dev(v), out.t, cfg(variant=_lib.GEMM_SKINNY, vec=8, **bad))


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 8, 12])
@pytest.mark.parametrize("m", [77, 512, 1024, 3072, 4096, 4097])
def test_pv_few_rows_builtin_choice(oracle, n, m):
    # 2 .. 12 query rows: two- or four-row workgroups of the row kernel, one workgroup per row sweeping the head's V
    # (3 .. 8 rows, up to ~3000 keys), or 64-row MFMA tiles with the keys split (any key count: P is read where it lies)
    p, v = _pv_inputs(32, n, m, 80, n + m)
    out = Guarded((32, n, 80), torch.float16)
    ops.attn_pv(dev(p), dev(v), out.t)
    _check_pv(out.check(), p, v, oracle)


def test_pv_selector_rows_are_exact_and_edge_cases(oracle):
    # P = identity picks the rows of V: any operand mix-up (a transposed V, a shifted k) shows as wrong bits
    rng = np.random.default_rng(5)
    v = rng.standard_normal((4, 200, 80)).astype(np.float16)
    eye = np.ascontiguousarray(np.broadcast_to(np.eye(200, dtype=np.float16), (4, 200, 200)))
    out = Guarded((4, 200, 80), torch.float16)
    ops.attn_pv(dev(eye), dev(v), out.t)
    assert np.array_equal(out.check().view(np.uint16), v.view(np.uint16))
    # element-access fallback: m % 8 != 0, d % 8 != 0, an odd V pointer
    for (n, m, d) in [(40, 77, 80), (12, 16, 12)]:
        p, v = _pv_inputs(2, n, m, d, n + m)
        out = Guarded((2, n, d), torch.float16)
        ops.attn_pv(dev(p), dev(v), out.t)
        _check_pv(out.check(), p, v, oracle)
    p, v = _pv_inputs(2, 40, 80, 80, 6)
    vbuf = torch.empty(2 * 80 * 80 + 1, dtype=torch.float16, device="cuda")
    vbuf[1:].copy_(dev(v).flatten())
    out = Guarded((2, 40, 80), torch.float16)
    ops.attn_pv(dev(p), vbuf[1:].view(2, 80, 80), out.t)
    _check_pv(out.check(), p, v, oracle)
    # m == 0: an empty sum is zeros; n == 0: a no-op
    out = Guarded((2, 5, 80), torch.float16)
    ops.attn_pv(torch.empty(2, 5, 0, dtype=torch.float16, device="cuda"), torch.empty(2, 0, 80, dtype=torch.float16, device="cuda"), out.t)
    assert (out.check() == 0).all()
    assert _lib.lib().dtas_attn_pv_f16(None, None, None, 32, 0, 16, 80, None, None) == 0


@pytest.mark.parametrize("n,m", [(13, 1025), (64, 77), (130, 1027), (300, 1028), (257, 513), (1024, 1032), (515, 7)])
def test_scores_and_pv_with_key_counts_off_the_vector_width(oracle, n, m):
    # rows of m floats / halves start anywhere: the scores keep their vector stores (at the rows' alignment), P.V
    # fetches the 16-byte pieces of P's rows where they lie and adds the last m % 8 keys in its epilogue
    heads, d = 4, 80
    q, k, mask = _inputs(heads, n, m, d, n + m)
    out = Guarded((heads, n, m), torch.float32)
    ops.attn_scores(dev(q), dev(k), dev(mask), out.t, SCALE)
    _check(out.check(), q, k, mask, oracle)
    p, v = _pv_inputs(heads, n, m, d, n * m)
    o = Guarded((heads, n, d), torch.float16)
    ops.attn_pv(dev(p), dev(v), o.t)
    _check_pv(o.check(), p, v, oracle)
    # an explicit tile on the same shapes, and a split over the keys
    for c in (cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=2, tile=[64, 128, 64]),
              cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=3, tile=[128, 128, 64], split_k=2 if m >= 256 else 1)):
        o = Guarded((heads, n, d), torch.float16)
        ops.attn_pv(dev(p), dev(v), o.t, c)
        _check_pv(o.check(), p, v, oracle)


@pytest.mark.parametrize("n,m", [(70, 1025), (130, 71), (33, 15)])
def test_pv_row_is_untouched_by_its_neighbours_with_key_counts_off_the_vector_width(oracle, n, m):
    # the 16-byte piece that would straddle the end of a row of P is never fetched: a row of Inf next to a finite row
    # leaves the finite row's result as it is (and exact, on small integers)
    heads, d = 3, 80
    rng = np.random.default_rng(n + m)
    p = rng.integers(0, 3, size=(heads, n, m)).astype(np.float16)
    v = rng.integers(-3, 4, size=(heads, m, d)).astype(np.float16)
    want = np.einsum("hnm,hmd->hnd", p.astype(np.float64), v.astype(np.float64))
    p[:, 1::2, :] = np.inf
    o = Guarded((heads, n, d), torch.float16)
    ops.attn_pv(dev(p), dev(v), o.t)
    got = o.check()
    assert np.array_equal(got[:, 0::2].astype(np.float64), want[:, 0::2])


def test_pv_with_a_p_that_is_not_16_byte_aligned(oracle):
    heads, n, m, d = 2, 70, 136, 80
    p, v = _pv_inputs(heads, n, m, d, 5)
    buf = torch.empty(heads * n * m + 1, dtype=torch.float16, device="cuda")
    buf[1:] = dev(p).reshape(-1)
    o = Guarded((heads, n, d), torch.float16)
    ops.attn_pv(buf[1:].view(heads, n, m), dev(v), o.t)
    _check_pv(o.check(), p, v, oracle)


def test_pv_errors():
    p, v = _pv_inputs(2, 16, 16, 80, 1)
    out = torch.empty(2, 16, 80, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match=r"split_k must be in \[1, 16\]"):
        ops.attn_pv(dev(p), dev(v), out, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=2, tile=[64, 64, 64], split_k=17))
    with pytest.raises(_lib.DtasError, match="three LDS stages come with"):
        ops.attn_pv(dev(p), dev(v), out, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=4, tile=[64, 64, 64]))
    with pytest.raises(_lib.DtasError, match="three LDS stages come with"):
        ops.attn_pv(dev(p), dev(v), out, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=3, tile=[64, 64, 64]))
    with pytest.raises(_lib.DtasError, match="no transposing"):
        ops.attn_pv(dev(p), dev(v), out, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=2, tile=[256, 128, 64]))
    with pytest.raises(_lib.DtasError, match="1, 2, 4 or 8"):
        ops.attn_pv(dev(p), dev(v), out, cfg(variant=_lib.GEMM_SKINNY, block=256, vec=8, unroll=1, tile=[3, 8, 0]))
    with pytest.raises(_lib.DtasError, match="does not split"):
        ops.attn_pv(dev(p), dev(v), out, cfg(variant=_lib.GEMM_SKINNY, block=256, vec=8, unroll=1, tile=[1, 8, 0], split_k=2))
    pd = dev(p)
    with pytest.raises(_lib.DtasError, match="overlaps"):
        check_rc = _lib.lib().dtas_attn_pv_f16(pd.data_ptr(), dev(v).data_ptr(), pd.data_ptr(), 2, 16, 16, 80, None, None)
        _lib.check(check_rc, "dtas_attn_pv_f16")


def test_pv_through_the_primfunc_descriptors(oracle):
    from dtas_amd import primfuncs as pf
    from dtas_amd.codegen.runtime_packer import bind_extents, call_primfunc

    for decode, n in ((False, 40), (True, 1)):
        func = pf.matmul_pv(32, 80, decode=decode)
        p, v = _pv_inputs(32, n, 56, 80, 9 + n)
        out = torch.empty(1, 32, n, 80, dtype=torch.float16, device="cuda")
        tensors = (dev(p).view(1, 32, n, 56), dev(v).view(1, 32, 56, 80), out)
        assert bind_extents(func, tensors) == ({"m": 56} if decode else {"n": 40, "m": 56})
        call_primfunc(func, tensors)
        torch.cuda.synchronize()
        _check_pv(out.cpu().numpy().reshape(32, n, 80), p, v, oracle)


def test_attention_full_size_properties(oracle):
    """n = m = 2048, 32 heads of 80 (268 M scores): properties that need no oracle pass over the whole output,
    plus sampled rows against the oracle."""
    heads, n, d = 32, 2048, 80
    g = torch.Generator(device="cuda").manual_seed(7)
    q = torch.randn(heads, n, d, device="cuda", generator=g).half()
    k = torch.randn(heads, n, d, device="cuda", generator=g).half()
    causal = torch.ones(n, n, device="cuda").tril_().bool()
    mask = torch.where(causal, torch.tensor(65504.0, device="cuda"), torch.tensor(-65504.0, device="cuda")).half()
    sc = torch.empty(heads, n, n, dtype=torch.float32, device="cuda")
    ops.attn_scores(q, k, mask, sc, SCALE)
    torch.cuda.synchronize()
    assert bool((sc[:, ~causal] == -65504.0).all())                          # the masked set is exact
    assert bool(torch.isfinite(sc).all()) and bool((sc[:, causal] > -65504.0).all())
    assert bool((sc.half().float() == sc).all())                             # every score is an fp16 value widened
    open_mask = torch.full((n, n), 65504.0, dtype=torch.float16, device="cuda")
    sc2 = torch.empty_like(sc)
    ops.attn_scores(q, k, open_mask, sc2, SCALE)
    assert bool((sc2[:, causal] == sc[:, causal]).all())                      # the mask only takes a minimum
    ops.attn_scores(k, q, open_mask, sc, SCALE)                              # (Q K^T)^T = K Q^T, bit for bit
    assert bool((sc.transpose(1, 2) == sc2).all())
    rows = [0, 1, 777, 2047]
    qn, kn = q.cpu().numpy(), k.cpu().numpy()
    want = oracle.c.attn_scores(np.ascontiguousarray(qn[:, rows]), kn, np.full((len(rows), n), 65504.0, np.float16), SCALE, threads=8)
    got = sc2[:, rows].cpu().numpy()
    assert (np.abs(got - want) <= 1e-3 + 2.0 ** -9 * np.abs(want)).all() and (got == want).mean() > 0.98
    del sc, sc2

    # P.V: a permutation matrix as P returns the permuted rows of V exactly; rows that sum to one return
    # values inside V's range; sampled rows against the oracle
    v = torch.randn(heads, n, d, device="cuda", generator=g).half()
    perm = torch.randperm(n, device="cuda", generator=g)
    p = torch.zeros(heads, n, n, dtype=torch.float16, device="cuda")
    p[:, torch.arange(n, device="cuda"), perm] = 1
    o = torch.empty(heads, n, d, dtype=torch.float16, device="cuda")
    ops.attn_pv(p, v, o)
    assert bool((o == v[:, perm]).all())
    p = torch.softmax(torch.randn(heads, n, n, device="cuda", generator=g), -1).half()
    ops.attn_pv(p, v, o)
    torch.cuda.synchronize()
    assert bool((o.float().abs().amax(1) <= v.float().abs().amax(1) * 1.01).all())
    pn, vn = p.cpu().numpy(), v.cpu().numpy()
    want = oracle.c.attn_pv(np.ascontiguousarray(pn[:, rows]), vn, threads=8).astype(np.float64)
    got = o[:, rows].cpu().numpy().astype(np.float64)
    assert (np.abs(got - want) <= 1e-4 + 2.0 ** -9 * np.abs(want)).all()


@pytest.mark.parametrize("n", [1, 2, 4, 8])
def test_decode_attention_against_the_prefill_kernels_and_properties(oracle, n):
    """A handful of query rows against 8192 keys, 32 heads of 80 (the decode step and short continuations): the row
    kernels return what the same rows return as part of a long prompt (same arithmetic per score; P.V within the fp32
    summation order), a one-hot P returns a row of V exactly, and sampled heads match the oracle."""
    heads, m, d = 32, 8192, 80
    g = torch.Generator(device="cuda").manual_seed(11 + n)
    q = torch.randn(heads, n, d, device="cuda", generator=g).half()
    k = torch.randn(heads, m, d, device="cuda", generator=g).half()
    v = torch.randn(heads, m, d, device="cuda", generator=g).half()
    mask = torch.full((n, m), 65504.0, dtype=torch.float16, device="cuda")
    mask[:, m - 5:] = -65504.0
    sc = torch.empty(heads, n, m, dtype=torch.float32, device="cuda")
    ops.attn_scores(q, k, mask, sc, SCALE)
    # the same rows as the last rows of a 128-row block go through the MFMA tiles
    qq = torch.zeros(heads, 128, d, dtype=torch.float16, device="cuda")
    qq[:, 128 - n:] = q
    mm = torch.full((128, m), 65504.0, dtype=torch.float16, device="cuda")
    mm[128 - n:] = mask
    big = torch.empty(heads, 128, m, dtype=torch.float32, device="cuda")
    ops.attn_scores(qq, k, mm, big, SCALE)
    torch.cuda.synchronize()
    same = (big[:, 128 - n:] == sc).float().mean().item()
    assert same > 0.999 and bool(((big[:, 128 - n:] - sc).abs() <= 2.0 ** -9 * sc.abs() + 1e-3).all())
    assert bool((sc[:, :, m - 5:] == -65504.0).all()) and bool((sc.half().float() == sc).all())
    want = oracle.c.attn_scores(q[:2].cpu().numpy(), k[:2].cpu().numpy(), mask.cpu().numpy(), SCALE, threads=8)
    got = sc[:2].cpu().numpy()
    assert (np.abs(got - want) <= 1e-3 + 2.0 ** -9 * np.abs(want)).all() and (got == want).mean() > 0.98
    # P.V: one-hot rows pick rows of V; softmaxed rows against the oracle
    pick = torch.randint(0, m, (heads, n), device="cuda", generator=g)
    p = torch.zeros(heads, n, m, dtype=torch.float16, device="cuda")
    p.scatter_(2, pick.unsqueeze(-1), 1.0)
    o = torch.empty(heads, n, d, dtype=torch.float16, device="cuda")
    ops.attn_pv(p, v, o)
    assert bool((o == torch.gather(v, 1, pick.unsqueeze(-1).expand(-1, -1, d))).all())
    p = torch.softmax(sc, -1).half()
    ops.attn_pv(p, v, o)
    torch.cuda.synchronize()
    want = oracle.c.attn_pv(p[:2].cpu().numpy(), v[:2].cpu().numpy(), threads=8).astype(np.float64)
    got = o[:2].cpu().numpy().astype(np.float64)
    assert (np.abs(got - want) <= 1e-4 + 2.0 ** -9 * np.abs(want)).all()

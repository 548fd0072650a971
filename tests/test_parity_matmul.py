"""GPU parity, decode GEMV and dynamic-M GEMM through the C ABI: against the fp32-accumulating CPU
oracle and the float64 product (rtol 1e-2), exact special cases, every tile variant on ragged
shapes.  At the large benchmark sizes the oracle is run on sampled rows of A (rows are independent)."""
import numpy as np
import pytest
import torch

from dtas_amd import _lib, ops
from gpu_util import Guarded, assert_bits_equal, cfg, dev

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 2e-3


def _check(got, oracle_out, f64):
    got = got.astype(np.float64)
    assert np.isfinite(got).all()
    assert (np.abs(got - f64) <= ATOL + RTOL * np.abs(f64)).all()
    # against the oracle (same fp32 arithmetic, another summation order): about one fp16 ulp
    want = oracle_out.astype(np.float64)
    assert (np.abs(got - want) <= 1e-3 + 2.0 ** -9 * np.abs(want)).all()


def _inputs(M, N, K, seed):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((M, K)).astype(np.float16), (rng.standard_normal((N, K)) * 0.02).astype(np.float16)


GEMV_SHAPES = [(4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096),
               # short rows (2 wavefronts on 2 or 4 rows, 4 on 2) and the other branches of the built-in choice
               (5120, 1024), (13824, 1024), (8192, 2048), (3000, 520), (7680, 2560), (2560, 10240), (300, 72), (20000, 512), (12288, 264)]


@pytest.mark.parametrize("N,K", GEMV_SHAPES)
def test_gemv_benchmark_config(oracle, N, K):
    x, w = _inputs(1, N, K, 5)
    out = Guarded((1, N), torch.float16)
    ops.gemv(dev(x), dev(w), None, out.t)
    _check(out.check(), oracle.c.gemm(x, w, threads=8), oracle.np64.gemm(x, w))


@pytest.mark.parametrize("rows", [1, 2, 4, 8])
@pytest.mark.parametrize("block", [64, 256, 512])
@pytest.mark.parametrize("N,K", [(2560, 10240), (1001, 2560), (7, 8), (130, 520)])
def test_gemv_every_variant_and_bias(oracle, rows, block, N, K):
    x, w = _inputs(1, N, K, N + K)
    bias = np.random.default_rng(1).uniform(-1, 1, N).astype(np.float16)
    out = Guarded((1, 1, N), torch.float16)
    ops.gemv(dev(x), dev(w), dev(bias), out.t, cfg(variant=_lib.GEMV_SPLITK, block=block, vec=8, unroll=2, tile=[rows, 0, 0]))
    _check(out.check().reshape(1, N), oracle.c.gemm(x, w, bias), oracle.np64.gemm(x, w, bias))


@pytest.mark.parametrize("N,K", [(2560, 10240), (4096, 4096), (33, 1003), (7, 8), (1001, 2560), (64, 256), (5, 250)])
def test_gemv_fp16_accumulate_in_the_reference_schedules_order(oracle, N, K):
    # variant RF16: every sum in fp16 in the order of the reference's scheduled kernel -> the same bits as its CPU restatement
    rng = np.random.default_rng(N + K)
    x = (rng.standard_normal(K) * 0.5).astype(np.float16)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    bias = rng.uniform(-1, 1, N).astype(np.float16)
    c = cfg(variant=_lib.GEMV_RF16, block=256, vec=8, tile=[8, 0, 0])
    for b in (bias, None):
        out = Guarded((N,), torch.float16)
        ops.gemv(dev(x), dev(w), None if b is None else dev(b), out.t, c)
        assert_bits_equal(out.check(), oracle.c.gemv_rf(x, w, b, threads=8))
    assert list(_lib.describe_launch(_lib.OP_GEMV_F16, 1, N, K, c).launch_args)[:4] == [-(-N // 8), 1, 1, 256]
    # the fused epilogues act on the fp16 sum as they do on the rounded fp32 one
    r1, r2 = rng.standard_normal(N).astype(np.float16), rng.standard_normal(N).astype(np.float16)
    out = Guarded((N,), torch.float16)
    ops.gemv(dev(x), dev(w), dev(bias), out.t, c, epilogue=1, res1=dev(r1), res2=dev(r2))
    mm = oracle.c.gemv_rf(x, w, bias, threads=8)
    assert_bits_equal(out.check(), ((r1 + mm).astype(np.float16) + r2).astype(np.float16))


def test_gemv_fp16_accumulate_order_cases_and_errors(oracle):
    # the hand-built cases that pin each stage's order in the oracle, through the kernel: 2048 + 1 ties back to 2048
    def run(K, entries, x_entries=()):
        w, x = np.zeros((3, K), np.float16), np.ones(K, np.float16)
        for k, v in entries:
            w[1, k] = v
        for k, v in x_entries:
            x[k] = v
        out = Guarded((3,), torch.float16)
        ops.gemv(dev(x), dev(w), None, out.t, cfg(variant=_lib.GEMV_RF16, block=256, vec=8, tile=[8, 0, 0]))
        got = out.check()
        assert_bits_equal(got, oracle.c.gemv_rf(x, w))
        return float(got[1])
    assert run(768, [(0, 2048), (256, 1), (512, 1)]) == 2048.0                      # a chain, ascending
    assert run(256, [(0, 2048), (1, 1), (2, 1), (3, 1), (4, 1)]) == 2048.0          # a lane's 8 chains, ascending
    assert run(256, [(0, 2048), (8, 1), (16, 1), (24, 1)]) == 2050.0                # the tree: strides 2 then 1
    assert run(256, [(0, 2048), (128, 1), (136, 1)]) == 2048.0                      # ... after stride 16
    assert run(512, [(0, 2048), (256, 1 - 2.0 ** -11)], [(256, 1 + 2.0 ** -10)]) == 2048.0   # product rounded before the add
    with pytest.raises(_lib.DtasError, match="256 threads"):
        _lib.describe_launch(_lib.OP_GEMV_F16, 1, 64, 64, cfg(variant=_lib.GEMV_RF16, block=128, vec=8, tile=[8, 0, 0]))


def test_gemv_exact_and_ragged(oracle):
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((96, 64)) * 0.02).astype(np.float16)
    x = np.zeros((1, 64), np.float16)
    x[0, 17] = 1
    out = Guarded((1, 96), torch.float16)
    ops.gemv(dev(x), dev(w), None, out.t)
    assert_bits_equal(out.check().ravel(), w[:, 17].copy())       # one-hot x selects a column of W exactly
    # K not a multiple of 8: element-access kernel
    x, w = _inputs(1, 33, 1003, 3)
    out = Guarded((1, 33), torch.float16)
    ops.gemv(dev(x), dev(w), None, out.t)
    _check(out.check(), oracle.c.gemm(x, w), oracle.np64.gemm(x, w))
    out = Guarded((1, 33), torch.float16)   # an explicit vector config steps down to element accesses
    ops.gemv(dev(x), dev(w), None, out.t, cfg(variant=_lib.GEMV_SPLITK, block=256, vec=8, unroll=2, tile=[4, 0, 0]))
    _check(out.check(), oracle.c.gemm(x, w), oracle.np64.gemm(x, w))


NK = [(4096, 4096), (11008, 4096), (4096, 11008)]


@pytest.mark.parametrize("N,K", NK)
@pytest.mark.parametrize("M", [1, 16, 64, 256])
def test_gemm_benchmark_config_small_m(oracle, M, N, K):
    a, w = _inputs(M, N, K, 6)
    out = Guarded((M, N), torch.float16)
    ops.gemm(dev(a), dev(w), None, out.t)
    _check(out.check(), oracle.c.gemm(a, w, threads=8), oracle.np64.gemm(a, w))


@pytest.mark.parametrize("N,K", NK)
@pytest.mark.parametrize("M", [1024, 2048, 4096, 8192])
def test_gemm_benchmark_config_large_m_sampled_rows(oracle, M, N, K):
    g = torch.Generator(device="cuda").manual_seed(6)
    a = torch.randn(M, K, device="cuda", generator=g).half()
    w = (torch.randn(N, K, device="cuda", generator=g) * 0.02).half()
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ops.gemm(a, w, None, out)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())                           # every element was written
    rows = np.unique(np.concatenate([[0, 1, 31, 32, 127, 128, 255, 256, M - 1], np.random.default_rng(M).integers(0, M, 7)]))
    idx = torch.from_numpy(rows).cuda()
    a_s, w_h = a[idx].cpu().numpy(), w.cpu().numpy()
    _check(out[idx].cpu().numpy(), oracle.c.gemm(a_s, w_h, threads=8), oracle.np64.gemm(a_s, w_h))
    # linearity over all rows: (sum_i C[i, :]) == (sum_i A[i, :]) . W^T, accumulated in fp64 on the device
    lhs = out.double().sum(0)
    rhs = a.double().sum(0) @ w.double().T
    assert float((lhs - rhs).abs().max()) < 1e-3 * M ** 0.5 + 0.5     # fp16 rounding of M outputs per column


def _threads(bm, bn):
    return 512 if (bm, bn) == (256, 256) else 256


@pytest.mark.parametrize("M,N,K", [(5, 7, 8), (300, 260, 200), (257, 513, 264), (512, 512, 64), (256, 256, 1024), (700, 300, 4104)])
@pytest.mark.parametrize("split", [1, 3])
def test_gemm_256x256_with_four_wavefronts(oracle, M, N, K, split):
    # block = 256 selects the variant with one wavefront per SIMD and 128x128 wavefront tiles
    a, w = _inputs(M, N, K, M + N + K)
    bias = np.random.default_rng(1).uniform(-1, 1, N).astype(np.float16)
    out = Guarded((M, N), torch.float16)
    c = cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, tile=[256, 256, 64], split_k=split)
    ops.gemm(dev(a), dev(w), dev(bias), out.t, c)
    _check(out.check(), oracle.c.gemm(a, w, bias, threads=8), oracle.np64.gemm(a, w, bias))
    assert list(_lib.describe_launch(_lib.OP_GEMM_F16, M, N, K, c).launch_args)[3:5] == [256, 5 * 256 * 128]


TILES = [(256, 256), (256, 128), (128, 256), (128, 128), (64, 128), (128, 64), (64, 64)]


@pytest.mark.parametrize("bm,bn", TILES)
@pytest.mark.parametrize("M,N,K", [(5, 7, 8), (33, 65, 72), (300, 260, 200), (257, 513, 264), (512, 512, 64), (64, 64, 1024)])
def test_gemm_every_mfma_tile_on_ragged_shapes(oracle, bm, bn, M, N, K):
    a, w = _inputs(M, N, K, M + N + K)
    bias = np.random.default_rng(1).uniform(-1, 1, N).astype(np.float16)
    out = Guarded((1, M, N), torch.float16)
    ops.gemm(dev(a), dev(w), dev(bias), out.t, cfg(variant=_lib.GEMM_MFMA, block=_threads(bm, bn), vec=8, tile=[bm, bn, 64]))
    _check(out.check().reshape(M, N), oracle.c.gemm(a, w, bias, threads=8), oracle.np64.gemm(a, w, bias))


@pytest.mark.parametrize("rows,block", [(16, 512), (16, 64), (32, 256), (48, 512), (64, 512), (80, 128)])
@pytest.mark.parametrize("N,K", [(64, 64), (100, 520), (4096, 1000 * 8), (33, 40)])
def test_gemm_every_skinny_tile(oracle, rows, block, N, K):
    for M in (rows, rows - 3, 1):
        a, w = _inputs(M, N, K, M + N + K)
        out = Guarded((M, N), torch.float16)
        ops.gemm(dev(a), dev(w), None, out.t, cfg(variant=_lib.GEMM_SKINNY, block=block, vec=8, unroll=4, tile=[rows, 16, 32]))
        _check(out.check(), oracle.c.gemm(a, w, threads=8), oracle.np64.gemm(a, w))


STREAM_TILES = [(16, 64, 512), (16, 64, 1024), (16, 128, 512), (32, 64, 512), (32, 128, 512), (64, 64, 512)]


@pytest.mark.parametrize("rows,cols,kslice", STREAM_TILES)
@pytest.mark.parametrize("N,K", [(64, 64), (100, 520), (1000, 2560), (4096, 4096), (33, 40), (2560, 8 * 1000)])
def test_gemm_every_streaming_tile(oracle, rows, cols, kslice, N, K):
    # the W-streaming kernel: one K slice (K <= the slice) up to 16 of them, ragged N, K and M, with and without bias
    for M in (rows, rows - 3, 1):
        a, w = _inputs(M, N, K, M + N + K)
        bias = np.random.default_rng(2).uniform(-1, 1, N).astype(np.float16) if M != 1 else None
        out = Guarded((M, N), torch.float16)
        c = cfg(variant=_lib.GEMM_STREAM, block=4 * cols, vec=8, unroll=1, tile=[rows, cols, kslice])
        ops.gemm(dev(a), dev(w), None if bias is None else dev(bias), out.t, c)
        _check(out.check(), oracle.c.gemm(a, w, bias, threads=8), oracle.np64.gemm(a, w, bias))
        info = _lib.describe_launch(_lib.OP_GEMM_F16, M, N, K, c)
        assert list(info.launch_args)[:5] == [-(-N // cols) * -(-K // kslice), 1, 1, 4 * cols, (rows + cols) * kslice * 2]


@pytest.mark.parametrize("cols", [16, 64])
@pytest.mark.parametrize("N,K", [(64, 64), (100, 520), (1000, 2560), (7680, 2560), (33, 40), (300, 256 * 9 + 8), (11008, 4096)])
def test_gemm_looping_streaming_tiles(oracle, cols, N, K):
    # the looping form (tile[2] = 256: the whole of K per workgroup through a ring of four LDS stages): fewer segments
    # than stages, exactly as many, many, a ragged last one; ragged N and M; with and without bias
    for M in (16, 13, 1):
        a, w = _inputs(M, N, K, M + N + K + cols)
        bias = np.random.default_rng(3).uniform(-1, 1, N).astype(np.float16) if M != 1 else None
        out = Guarded((M, N), torch.float16)
        c = cfg(variant=_lib.GEMM_STREAM, block=4 * cols, vec=8, unroll=1, tile=[16, cols, 256])
        ops.gemm(dev(a), dev(w), None if bias is None else dev(bias), out.t, c)
        _check(out.check(), oracle.c.gemm(a, w, bias, threads=8), oracle.np64.gemm(a, w, bias))
        info = _lib.describe_launch(_lib.OP_GEMM_F16, M, N, K, c)
        assert list(info.launch_args)[:5] == [-(-N // cols), 1, 1, 4 * cols, 4 * (16 + cols) * 512]


def test_gemm_looping_streaming_tile_is_the_choice_for_many_rows_of_w_exact_and_refuses_what_it_cannot_hold(oracle):
    # what cfg = NULL runs for M <= 16 against 4096 < N <= 16384 rows of W with K <= 4096
    for N, K, tile, block in ((7680, 2560, [16, 16, 256], 64), (8192, 4096, [16, 16, 256], 64), (11008, 4096, [16, 64, 256], 256),
                              (10240, 2560, [16, 64, 256], 256)):
        got = _lib.select_bucket(_lib.OP_GEMM_F16, 16, N, K).config
        assert (got.variant, list(got.tile), got.block) == (_lib.GEMM_STREAM, tile, block), (N, K)
    for N, K in ((4096, 4096), (4096, 11008), (32000, 4096), (11008, 8192)):
        got = _lib.select_bucket(_lib.OP_GEMM_F16, 16, N, K).config
        assert not (got.variant == _lib.GEMM_STREAM and got.tile[2] == 256), (N, K)
    assert _lib.select_bucket(_lib.OP_GEMM_F16, 17, 11008, 4096).config.variant == _lib.GEMM_MFMA
    # small integers: every sum is exact in fp32 and fp16, whatever the order
    rng = np.random.default_rng(7)
    ai, wi = rng.integers(-2, 3, (13, 2048)).astype(np.float16), rng.integers(-2, 3, (200, 2048)).astype(np.float16)
    for cols in (16, 64):
        out = Guarded((13, 200), torch.float16)
        ops.gemm(dev(ai), dev(wi), None, out.t, cfg(variant=_lib.GEMM_STREAM, block=4 * cols, vec=8, unroll=1, tile=[16, cols, 256]))
        assert np.array_equal(out.check().astype(np.float64), ai.astype(np.float64) @ wi.astype(np.float64).T)
    big = dev(np.zeros((17, 64), np.float16))
    with pytest.raises(_lib.DtasError, match="cannot hold M=17"):
        ops.gemm(big, dev(np.zeros((8, 64), np.float16)), None, torch.empty(17, 8, dtype=torch.float16, device="cuda"),
                 cfg(variant=_lib.GEMM_STREAM, block=256, vec=8, unroll=1, tile=[16, 64, 256]))
    for tile, block in (([32, 64, 256], 256), ([16, 32, 256], 128), ([16, 64, 256], 512)):
        with pytest.raises(_lib.DtasError, match="streaming"):
            _lib.describe_launch(_lib.OP_GEMM_F16, 8, 64, 64, cfg(variant=_lib.GEMM_STREAM, block=block, vec=8, unroll=1, tile=tile))


@pytest.mark.parametrize("kind", [1, 2, 3])
@pytest.mark.parametrize("cols", [16, 64])
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 7, 8), (16, 130, 1096), (13, 2560, 2560)])
def test_gemm_fused_epilogues_looping_streaming_tile(oracle, kind, cols, M, N, K):
    a, w, bias, r1, r2 = _fused_inputs(M, N, K, M + N + K + kind)
    res = (dev(r1), dev(r2)) if kind in (1, 2) else (None, None)
    out = Guarded((M, N), torch.float32 if kind == 2 else torch.float16)
    c = cfg(variant=_lib.GEMM_STREAM, block=4 * cols, vec=8, unroll=1, tile=[16, cols, 256])
    ops.gemm(dev(a), dev(w), dev(bias), out.t, c, epilogue=kind, res1=res[0], res2=res[1])
    want = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind, threads=8)
    _check_fused(out.check(), want, oracle.np64.gemm_fused(a, w, bias, r1, r2, kind), kind, r1, r2)


def test_gemm_streaming_tile_is_reproducible_exact_and_refuses_what_it_cannot_hold(oracle):
    M, N, K = 16, 4096, 4096
    a, w = _inputs(M, N, K, 5)
    assert _lib.select_bucket(_lib.OP_GEMM_F16, M, N, K).config.variant == _lib.GEMM_STREAM   # what cfg = NULL runs here
    runs = []
    for _ in range(3):
        out = Guarded((M, N), torch.float16)
        ops.gemm(dev(a), dev(w), None, out.t)
        runs.append(out.check())
    assert all(np.array_equal(r.view(np.uint16), runs[0].view(np.uint16)) for r in runs)   # slices are added in slice order
    _check(runs[0], oracle.c.gemm(a, w, threads=8), oracle.np64.gemm(a, w))
    # small integers: every sum is exact in fp32 and fp16, whatever the order
    rng = np.random.default_rng(6)
    ai, wi = rng.integers(-2, 3, (13, 2048)).astype(np.float16), rng.integers(-2, 3, (200, 2048)).astype(np.float16)
    out = Guarded((13, 200), torch.float16)
    ops.gemm(dev(ai), dev(wi), None, out.t, cfg(variant=_lib.GEMM_STREAM, block=256, vec=8, unroll=1, tile=[16, 64, 512]))
    assert np.array_equal(out.check().astype(np.float64), ai.astype(np.float64) @ wi.astype(np.float64).T)
    big = dev(np.zeros((17, 64), np.float16))
    with pytest.raises(_lib.DtasError, match="cannot hold M=17"):
        ops.gemm(big, dev(np.zeros((8, 64), np.float16)), None, torch.empty(17, 8, dtype=torch.float16, device="cuda"),
                 cfg(variant=_lib.GEMM_STREAM, block=256, vec=8, unroll=1, tile=[16, 64, 512]))
    for tile, block in (([64, 128, 512], 512), ([16, 64, 2048], 256), ([48, 64, 512], 256), ([16, 64, 512], 512)):
        with pytest.raises(_lib.DtasError, match="streaming"):
            _lib.describe_launch(_lib.OP_GEMM_F16, 8, 64, 64, cfg(variant=_lib.GEMM_STREAM, block=block, vec=8, unroll=1, tile=tile))


@pytest.mark.parametrize("bm,bn", [(256, 128), (128, 256), (192, 256), (192, 128)])
@pytest.mark.parametrize("split", [1, 2, 3])
@pytest.mark.parametrize("M,N,K", [(5, 7, 8), (300, 260, 200), (257, 513, 1096), (512, 512, 64), (256, 256, 4096), (700, 300, 4104),
                                   (193, 257, 72), (960, 520, 264)])
def test_gemm_rectangular_tiles_with_eight_wavefronts(oracle, bm, bn, split, M, N, K):
    # block = 512 on 256x128 / 128x256 / 192x256 / 192x128: 64x64, 96x64 or 48x64 per wavefront on the ring loop of the
    # 256x256 kernel (the ring's units are the larger side's rows of a k tile)
    a, w = _inputs(M, N, K, M + N + K)
    bias = np.random.default_rng(1).uniform(-1, 1, N).astype(np.float16)
    out = Guarded((M, N), torch.float16)
    c = cfg(variant=_lib.GEMM_MFMA, block=512, vec=8, unroll=2, tile=[bm, bn, 64], split_k=split)
    ops.gemm(dev(a), dev(w), dev(bias), out.t, c)
    _check(out.check(), oracle.c.gemm(a, w, bias, threads=8), oracle.np64.gemm(a, w, bias))
    assert list(_lib.describe_launch(_lib.OP_GEMM_F16, M, N, K, c).launch_args)[3:5] == [512, 5 * max(bm, bn) * 128]


def test_gemm_tiles_of_192_rows_come_with_eight_wavefronts_and_two_stages():
    for bad, msg in ((dict(block=256), "512 threads"), (dict(unroll=3), "at most 2 LDS stages"), (dict(tile=[256, 192, 64]), "no MFMA kernel")):
        c = dict(variant=_lib.GEMM_MFMA, block=512, vec=8, unroll=2, tile=[192, 256, 64])
        c.update(bad)
        with pytest.raises(_lib.DtasError, match=msg):
            _lib.describe_launch(_lib.OP_GEMM_F16, 512, 512, 512, cfg(**c))


@pytest.mark.parametrize("mv,r", [(2, 1), (2, 2), (2, 4), (4, 1), (4, 2), (4, 4)])
@pytest.mark.parametrize("block", [64, 128, 256])
@pytest.mark.parametrize("N,K", [(64, 64), (101, 520), (4096, 4096), (33, 8 * 64 * 5 + 8)])
def test_gemm_row_kernel_every_variant(oracle, mv, r, block, N, K):
    # W streamed in whole rows against up to four rows of A: every M the tile holds, ragged N, K with a tail
    for M in range(1, mv + 1):
        a, w = _inputs(M, N, K, M + N + K)
        bias = np.random.default_rng(M).uniform(-1, 1, N).astype(np.float16)
        out = Guarded((M, N), torch.float16)
        ops.gemm(dev(a), dev(w), dev(bias), out.t, cfg(variant=_lib.GEMM_ROWS, block=block, vec=8, tile=[mv, r, 8]))
        _check(out.check(), oracle.c.gemm(a, w, bias, threads=8), oracle.np64.gemm(a, w, bias))


@pytest.mark.parametrize("M", [3, 4])
def test_gemm_three_and_four_rows_against_few_rows_of_w_take_the_row_kernel(oracle, M):
    # built-in: the row kernel up to 2560 rows of W (or 4096 x 4096), the tiles beyond; every epilogue
    for kind, N, K in ((0, 2560, 2560), (1, 2560, 10240), (2, 4096, 4096), (3, 1000, 520), (0, 7680, 2560)):
        a, w, bias, r1, r2 = _fused_inputs(M, N, K, 50 + kind + M)
        res = (dev(r1), dev(r2)) if kind in (1, 2) else (None, None)
        out = Guarded((1, M, N), torch.float32 if kind == 2 else torch.float16)
        ops.gemm(dev(a), dev(w), dev(bias), out.t, None, epilogue=kind, res1=res[0], res2=res[1])
        want = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind, threads=8)
        _check_fused(out.check().reshape(M, N), want, oracle.np64.gemm_fused(a, w, bias, r1, r2, kind), kind, r1, r2)


def test_gemm_two_rows_take_the_row_kernel_with_every_epilogue_and_errors(oracle):
    for kind, N, K in ((0, 4096, 4096), (1, 2560, 2560), (2, 2560, 2560), (3, 10240, 2560)):
        a, w, bias, r1, r2 = _fused_inputs(2, N, K, 40 + kind)
        res = (dev(r1), dev(r2)) if kind in (1, 2) else (None, None)
        out = Guarded((1, 2, N), torch.float32 if kind == 2 else torch.float16)
        ops.gemm(dev(a), dev(w), dev(bias), out.t, None, epilogue=kind, res1=res[0], res2=res[1])
        want = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind, threads=8)
        _check_fused(out.check().reshape(2, N), want, oracle.np64.gemm_fused(a, w, bias, r1, r2, kind), kind, r1, r2)
    a, w = _inputs(2, 96, 64, 3)
    x = np.zeros((2, 64), np.float16)
    x[0, 5], x[1, 63] = 1, 1
    out = Guarded((2, 96), torch.float16)
    ops.gemm(dev(x), dev(w), None, out.t)
    got = out.check()
    assert_bits_equal(got[0], w[:, 5].copy())          # one-hot rows of A select columns of W exactly
    assert_bits_equal(got[1], w[:, 63].copy())
    out = torch.empty(5, 96, dtype=torch.float16, device="cuda")
    a5, _ = _inputs(5, 96, 64, 4)
    with pytest.raises(_lib.DtasError, match="cannot hold M=5"):
        ops.gemm(dev(a5), dev(w), None, out, cfg(variant=_lib.GEMM_ROWS, block=64, vec=8, tile=[4, 2, 8]))
    with pytest.raises(_lib.DtasError, match="row kernel takes tile"):
        ops.gemm(dev(a), dev(w), None, out[:2], cfg(variant=_lib.GEMM_ROWS, block=64, vec=8, tile=[8, 2, 8]))
    with pytest.raises(_lib.DtasError, match="64, 128 or 256 threads"):
        ops.gemm(dev(a), dev(w), None, out[:2], cfg(variant=_lib.GEMM_ROWS, block=512, vec=8, tile=[2, 2, 8]))


def test_gemm_exact_cases(oracle):
    rng = np.random.default_rng(7)
    a = rng.standard_normal((300, 256)).astype(np.float16)
    eye = np.eye(256, dtype=np.float16)
    perm = rng.permutation(256)
    for tile in ([256, 256, 64], [64, 64, 64], [128, 256, 64]):
        out = Guarded(a.shape, torch.float16)
        ops.gemm(dev(a), dev(eye[perm].copy()), None, out.t, cfg(variant=_lib.GEMM_MFMA, block=_threads(*tile[:2]), vec=8, tile=tile))
        assert_bits_equal(out.check(), a[:, perm].copy())             # a permutation matrix permutes columns exactly
    # an asymmetric case pins which operand is transposed and the accumulator layout
    a = np.zeros((70, 64), np.float16)
    w = np.zeros((90, 64), np.float16)
    a[np.arange(70), np.arange(70) % 64] = np.arange(1, 71)
    w[np.arange(90), (np.arange(90) * 7) % 64] = 1
    out = Guarded((70, 90), torch.float16)
    ops.gemm(dev(a), dev(w), None, out.t)
    assert_bits_equal(out.check(), oracle.c.gemm(a, w))


def test_gemm_k_not_multiple_of_8_and_errors(oracle):
    a, w = _inputs(9, 20, 77, 9)
    out = Guarded((9, 20), torch.float16)
    ops.gemm(dev(a), dev(w), None, out.t)                            # element-access kernel
    _check(out.check(), oracle.c.gemm(a, w), oracle.np64.gemm(a, w))
    big, wb = _inputs(40, 20, 80, 9)
    with pytest.raises(_lib.DtasError, match="cannot hold"):
        ops.gemm(dev(big), dev(wb), None, torch.empty(40, 20, dtype=torch.float16, device="cuda"),
                 cfg(variant=_lib.GEMM_SKINNY, block=512, vec=8, tile=[16, 16, 32]))
    out = Guarded((9, 20), torch.float16)   # an explicit MFMA config steps down to element accesses
    ops.gemm(dev(a), dev(w), None, out.t, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, tile=[64, 64, 64]))
    _check(out.check(), oracle.c.gemm(a, w), oracle.np64.gemm(a, w))


# ---- the reference's scheduled GEMM arithmetic: an fp16 accumulator rounded once per k step of 16
# (experiment/testIR/GEMM/m_n2560_k10240/wmma/16x16x16/i2j4_x7y2_in8.py:19,37) -------------------------------------
ACC16 = dict(variant=_lib.GEMM_MFMA_ACC16, block=256, vec=8, unroll=1, tile=[64, 64, 16], split_k=1)


def _check_acc16(got, want, f64):
    """Against oracle.c.gemm(acc_f16=2): the same roundings step by step; inside a step the matrix core adds its 16
    exact products in an order of its own, so a sum that lands on a rounding boundary may fall to the other side --
    one fp16 ulp there, which later steps carry along."""
    g, w = got.astype(np.float64), want.astype(np.float64)
    assert np.isfinite(g).all()
    scale = max(1.0, float(np.abs(f64).max()))
    assert (np.abs(g - w) <= 4 * 2.0 ** -10 * np.maximum(np.abs(w), 0.25 * scale)).all(), float(np.abs(g - w).max())
    assert (got == want).mean() > 0.9, float((got == want).mean())
    # an fp16 running sum loses what fp32 accumulation keeps: the bound against float64 grows with sqrt(K / 16) roundings
    assert np.abs(g - f64).max() <= 0.02 * scale + 1e-2


@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 7, 8), (33, 65, 72), (70, 130, 136), (300, 260, 200), (64, 2560, 2560), (256, 512, 10240)])
def test_gemm_fp16_accumulator_per_k_step_of_16(oracle, M, N, K):
    a, w = _inputs(M, N, K, 40 + M)
    bias = np.random.default_rng(M).uniform(-1, 1, N).astype(np.float16)
    out = Guarded((M, N), torch.float16)
    ops.gemm(dev(a), dev(w), dev(bias), out.t, cfg(**ACC16))
    _check_acc16(out.check(), oracle.c.gemm(a, w, bias, acc_f16=2, threads=8), oracle.np64.gemm(a, w, bias))


def test_gemm_fp16_accumulator_exact_cases_element_accesses_epilogues_and_errors(oracle):
    def run(a, w, **kw):
        out = Guarded((a.shape[0], w.shape[0]), torch.float16)
        ops.gemm(dev(a), dev(w), None, out.t, cfg(**{**ACC16, **kw}))
        return out.check()
    # where the accumulator stalls tells the step: products of 1/16, a step adds 1.0 and an fp16 sum stops at 2048
    # (fp32 accumulation reaches 8192, one product at a time 128)
    K = 16 * 8192
    a = np.ones((3, K), np.float16)
    w = np.full((2, K), 1 / 16, np.float16)
    assert (run(a, w) == 2048.0).all()
    fp32 = Guarded((3, 2), torch.float16)
    ops.gemm(dev(a), dev(w), None, fp32.t, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, tile=[64, 64, 64]))
    assert (fp32.check() == 8192.0).all()
    # inside a step nothing is rounded (2048 + 2 ones = 2050), across steps each tie is lost; steps start at k = 0, 16, ...
    def one(entries, K=48):
        wv = np.zeros((1, K), np.float16)
        for k, v in entries:
            wv[0, k] = v
        return float(run(np.ones((1, K), np.float16), wv)[0, 0])
    assert one([(0, 2048), (30, 1), (31, 1)]) == 2050.0
    assert one([(0, 2048), (31, 1), (32, 1)]) == 2048.0
    assert one([(0, 2048)] + [(k, 1) for k in range(16, 32)]) == 2064.0
    # small integers: every sum is exact, so the result is the oracle's bit for bit (a transposed operand or a
    # misplaced accumulator register fails here), on a shape that leaves tiles and the last step ragged
    rng = np.random.default_rng(3)
    ai = rng.integers(-3, 4, (70, 136)).astype(np.float16)
    wi = rng.integers(-3, 4, (90, 136)).astype(np.float16)
    assert_bits_equal(run(ai, wi), oracle.c.gemm(ai, wi, acc_f16=2))
    # K % 8 != 0 (and odd pointers): element accesses, same arithmetic
    a7, w7 = _inputs(9, 20, 77, 9)
    _check_acc16(run(a7, w7), oracle.c.gemm(a7, w7, acc_f16=2), oracle.np64.gemm(a7, w7))
    assert_bits_equal(run(ai[:, :77].copy(), wi[:, :77].copy()), oracle.c.gemm(ai[:, :77].copy(), wi[:, :77].copy(), acc_f16=2))
    # the fused epilogues act on the fp16 sum as everywhere else
    a2, w2 = _inputs(37, 96, 264, 11)
    bias = rng.uniform(-1, 1, 96).astype(np.float16)
    r1, r2 = rng.standard_normal((37, 96)).astype(np.float16), rng.standard_normal((37, 96)).astype(np.float16)
    for kind in (1, 2, 3):
        out = Guarded((37, 96), torch.float32 if kind == 2 else torch.float16)
        ops.gemm(dev(a2), dev(w2), dev(bias), out.t, cfg(**ACC16), epilogue=kind, res1=dev(r1) if kind < 3 else None,
                 res2=dev(r2) if kind < 3 else None)
        want = oracle.c.gemm_fused(a2, w2, bias, r1 if kind < 3 else None, r2 if kind < 3 else None, kind, acc_f16=2)
        g, wv = out.check().astype(np.float64), want.astype(np.float64)
        assert (np.abs(g - wv) <= 4 * 2.0 ** -10 * np.maximum(np.abs(wv), 1.0)).all()
    # what the mode cannot be combined with
    o = torch.empty(9, 20, dtype=torch.float16, device="cuda")
    for bad, msg in ((dict(split_k=2), "cannot be split"), (dict(tile=[128, 128, 16]), "64x64x16"), (dict(block=512), "256 threads")):
        with pytest.raises(_lib.DtasError, match=msg):
            ops.gemm(dev(a7[:, :72].copy()), dev(w7[:, :72].copy()), None, o, cfg(**{**ACC16, **bad}))
    # the Python config object reaches the same kernel
    from dtas_amd.common.config import MFMAConfig
    c = MFMAConfig()
    c.acc_f16 = True
    abi = c.to_abi()
    assert (abi.variant, abi.block, list(abi.tile)) == (_lib.GEMM_MFMA_ACC16, 256, [64, 64, 16])
    assert MFMAConfig().from_dict(c.to_dict()).acc_f16


SPLIT_TILES = [(256, 256), (128, 128), (128, 64), (64, 64)]


@pytest.mark.parametrize("bm,bn", SPLIT_TILES)
@pytest.mark.parametrize("split", [2, 3, 4, 7])
@pytest.mark.parametrize("M,N,K", [(5, 7, 8), (70, 130, 136), (300, 260, 1096), (64, 512, 4096)])
def test_gemm_split_k_on_ragged_shapes(oracle, bm, bn, split, M, N, K):
    # K = 8 and 136 leave some of the K partitions without a single k tile; 1096 splits unevenly
    a, w = _inputs(M, N, K, M + N + K + split)
    bias = np.random.default_rng(1).uniform(-1, 1, N).astype(np.float16)
    out = Guarded((M, N), torch.float16)
    c = cfg(variant=_lib.GEMM_MFMA, block=_threads(bm, bn), vec=8, tile=[bm, bn, 64], split_k=split)
    ops.gemm(dev(a), dev(w), dev(bias), out.t, c)
    _check(out.check(), oracle.c.gemm(a, w, bias, threads=8), oracle.np64.gemm(a, w, bias))
    info = _lib.describe_launch(_lib.OP_GEMM_F16, M, N, K, c)
    assert info.launch_args[0] == -(-M // bm) * -(-N // bn) * split


def test_gemm_split_k_is_reproducible_and_rearms_its_counters(oracle):
    # the partial tiles are summed in partition order whichever workgroup arrives last, so repeated
    # launches give identical bits; launches of other shapes in between share the same counters
    shapes = [(64, 4096, 4096, 4, (64, 64)), (200, 1000, 2048, 3, (128, 128)), (512, 512, 8192, 2, (256, 256))]
    first = {}
    for rep in range(3):
        for (M, N, K, split, (bm, bn)) in shapes:
            a, w = _inputs(M, N, K, M + K)
            out = Guarded((M, N), torch.float16)
            ops.gemm(dev(a), dev(w), None, out.t, cfg(variant=_lib.GEMM_MFMA, block=_threads(bm, bn), vec=8, tile=[bm, bn, 64], split_k=split))
            got = out.check()
            if rep == 0:
                first[(M, N, K)] = got
                _check(got, oracle.c.gemm(a, w, threads=8), oracle.np64.gemm(a, w))
            else:
                assert_bits_equal(got, first[(M, N, K)])


def test_gemm_split_k_many_launches_back_to_back():
    # no synchronisation between launches: each reads the counters the previous one re-armed
    M, N, K = 96, 2048, 4096
    g = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randn(M, K, device="cuda", generator=g).half()
    w = (torch.randn(N, K, device="cuda", generator=g) * 0.02).half()
    c = cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, tile=[64, 64, 64], split_k=4)
    outs = [torch.empty(M, N, dtype=torch.float16, device="cuda") for _ in range(50)]
    for o in outs:
        ops.gemm(a, w, None, o, c)
    torch.cuda.synchronize()
    ref = a.float() @ w.float().T
    for o in outs:
        assert torch.equal(o, outs[0])
    assert float((outs[0].float() - ref).abs().max()) < 2e-2


@pytest.mark.parametrize("c", [dict(variant=3, block=256, vec=8, unroll=1, tile=[32, 64, 512]),
                               dict(variant=3, block=256, vec=8, unroll=1, tile=[16, 64, 512]),
                               dict(variant=0, block=256, vec=8, unroll=4, tile=[64, 64, 64], split_k=4)])
def test_gemm_split_k_hands_over_fresh_partials(c):
    # launches alternate between two problems in one workspace: a partial sum read before its writer's stores have
    # landed would be the other problem's (small partials and a short hand-over are where that shows)
    M, N, K = 32 if c["tile"][0] >= 32 else 16, 4096, 4096
    g = torch.Generator(device="cuda").manual_seed(11)
    a = [torch.randn(M, K, device="cuda", generator=g).half() for _ in range(2)]
    w = [(torch.randn(N, K, device="cuda", generator=g) * 0.02).half() for _ in range(2)]
    outs = [torch.empty(M, N, dtype=torch.float16, device="cuda") for _ in range(120)]
    for i, o in enumerate(outs):
        ops.gemm(a[i % 2], w[i % 2], None, o, cfg(**c))
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        assert torch.equal(o, outs[i % 2]), i
    for i in range(2):
        assert float((outs[i].float() - a[i].float() @ w[i].float().T).abs().max()) < 2e-2


def test_gemm_split_k_on_two_streams_at_once():
    # each stream has its own partial tiles and arrival counters: launches that split K may overlap.
    # Two streams of the default priority take turns launching different problems without any
    # synchronisation in between; every result must equal the bits of the same launch made alone.
    g = torch.Generator(device="cuda").manual_seed(11)
    probs = []
    for (M, N, K) in ((64, 4096, 4096), (48, 2048, 8192)):
        a = torch.randn(M, K, device="cuda", generator=g).half()
        w = (torch.randn(N, K, device="cuda", generator=g) * 0.02).half()
        alone = torch.empty(M, N, dtype=torch.float16, device="cuda")
        ops.gemm(a, w, None, alone)                     # the built-in row: 64x64 tiles, K split over workgroups
        assert _lib.select_bucket(_lib.OP_GEMM_F16, M, N, K).config.split_k > 1
        probs.append((a, w, alone))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[torch.empty_like(probs[i][2]) for _ in range(40)] for i in range(2)]
    for rep in range(40):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                ops.gemm(probs[i][0], probs[i][1], None, outs[i][rep])
    torch.cuda.synchronize()
    for i in range(2):
        for o in outs[i]:
            assert torch.equal(o, probs[i][2])


@pytest.mark.parametrize("M,N,K", [(300, 1000, 4096), (1536, 4096, 2048), (1100, 5000, 1024), (8192 + 256, 4096, 512)])
def test_gemm_256_tile_splits_only_its_last_round(oracle, M, N, K):
    # split_k = 0 on the 8-wavefront tile: whole rounds of the chip one workgroup per tile, the tiles of the
    # partly filled last round shared by several; the launch description tells how many
    a, w = _inputs(M, N, K, M + N)
    bias = np.random.default_rng(5).uniform(-1, 1, N).astype(np.float16)
    c = cfg(variant=_lib.GEMM_MFMA, block=512, vec=8, unroll=2, tile=[256, 256, 64], split_k=0)
    tiles, ktiles = -(-M // 256) * -(-N // 256), -(-K // 64)
    info = _lib.describe_launch(_lib.OP_GEMM_F16, M, N, K, c)
    rem = tiles % 256
    assert rem > 0
    split, rest = divmod(info.launch_args[0] - (tiles - rem), rem)
    assert rest == 0 and 1 <= split <= 4 and rem * split <= 256 and (split == 1 or ktiles // split >= 8)
    out = Guarded((M, N), torch.float16)
    ops.gemm(dev(a), dev(w), dev(bias), out.t, c)
    got = out.check()
    _check(got, oracle.c.gemm(a, w, bias, threads=8), oracle.np64.gemm(a, w, bias))
    again = Guarded((M, N), torch.float16)
    ops.gemm(dev(a), dev(w), dev(bias), again.t, c)
    assert_bits_equal(again.check(), got)


def test_gemm_split_k_errors():
    a, w = _inputs(64, 64, 64, 1)
    with pytest.raises(_lib.DtasError, match="split_k"):
        ops.gemm(dev(a), dev(w), None, torch.empty(64, 64, dtype=torch.float16, device="cuda"),
                 cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, tile=[64, 64, 64], split_k=17))


def _fused_inputs(M, N, K, seed):
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((N, K)) * 0.03).astype(np.float16)
    bias = rng.uniform(-1, 1, N).astype(np.float16)
    r1 = rng.standard_normal((M, N)).astype(np.float16)
    r2 = rng.standard_normal((M, N)).astype(np.float16)
    return a, w, bias, r1, r2


def _check_fused(got, want_oracle, want_f64, kind, r1=None, r2=None):
    got = got.astype(np.float64)
    assert np.isfinite(got).all()
    # the fp16 rounding after every step acts at the magnitude of the intermediates: where the residuals
    # cancel, the result is small but carries their rounding
    scale = np.abs(want_f64)
    if kind in (1, 2):
        scale = np.maximum(scale, np.maximum(np.abs(r1.astype(np.float64)), np.abs(r2.astype(np.float64))))
    assert (np.abs(got - want_f64) <= 4e-3 + RTOL * scale).all()
    # against the oracle: the product may differ by an fp16 ulp (fp32 summation order), and each later
    # fp16 rounding step can carry that over; gelu also sits on another erf implementation
    want = want_oracle.astype(np.float64)
    assert (np.abs(got - want) <= 2e-3 + 2.0 ** -8 * scale).all()
    assert (got == want).mean() > 0.9


FUSED_CONFIGS = [None,
                 dict(variant=0, block=512, vec=8, tile=[256, 256, 64]),
                 dict(variant=0, block=256, vec=8, tile=[256, 256, 64]),
                 dict(variant=0, block=256, vec=8, unroll=3, tile=[256, 128, 64]),
                 dict(variant=0, block=256, vec=8, unroll=4, tile=[64, 64, 64], split_k=3),
                 dict(variant=1, block=512, vec=8, unroll=4, tile=[80, 16, 32]),
                 dict(variant=0, block=512, vec=8, unroll=2, tile=[256, 128, 64], split_k=2),
                 dict(variant=0, block=512, vec=8, unroll=2, tile=[192, 256, 64]),
                 dict(variant=0, block=512, vec=8, unroll=2, tile=[192, 128, 64], split_k=2)]


@pytest.mark.parametrize("kind", [1, 2, 3])
@pytest.mark.parametrize("tile,split", [((192, 256), 1), ((192, 256), 2), ((192, 128), 1), ((192, 128), 3)])
def test_gemm_fused_epilogues_on_tiles_of_192_rows(oracle, kind, tile, split):
    M, N, K = 400, 520, 264      # three tile rows, the last one ragged
    a, w, bias, r1, r2 = _fused_inputs(M, N, K, M + N + K + kind)
    res = (dev(r1), dev(r2)) if kind in (1, 2) else (None, None)
    out = Guarded((M, N), torch.float32 if kind == 2 else torch.float16)
    c = cfg(variant=0, block=512, vec=8, unroll=2, tile=[tile[0], tile[1], 64], split_k=split)
    ops.gemm(dev(a), dev(w), dev(bias), out.t, c, epilogue=kind, res1=res[0], res2=res[1])
    want = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind, threads=8)
    _check_fused(out.check(), want, oracle.np64.gemm_fused(a, w, bias, r1, r2, kind), kind, r1, r2)


@pytest.mark.parametrize("kind", [1, 2, 3])
@pytest.mark.parametrize("which", range(len(FUSED_CONFIGS)))
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 7, 8), (70, 130, 136), (77, 2560, 520)])
def test_gemm_fused_epilogues(oracle, kind, which, M, N, K):
    # fused_NT_matmul2_add1_add3_add3(_cast) and fused_NT_matmul3_add2_gelu through every kernel family
    a, w, bias, r1, r2 = _fused_inputs(M, N, K, M + N + K + kind)
    res = (dev(r1), dev(r2)) if kind in (1, 2) else (None, None)
    out = Guarded((M, N), torch.float32 if kind == 2 else torch.float16)
    c = None if FUSED_CONFIGS[which] is None else cfg(**FUSED_CONFIGS[which])
    ops.gemm(dev(a), dev(w), dev(bias), out.t, c, epilogue=kind, res1=res[0], res2=res[1])
    want = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind, threads=8)
    _check_fused(out.check(), want, oracle.np64.gemm_fused(a, w, bias, r1, r2, kind), kind, r1, r2)


@pytest.mark.parametrize("kind", [1, 2, 3])
@pytest.mark.parametrize("rows,cols,kslice", [(16, 64, 1024), (32, 128, 512), (64, 64, 512)])
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 7, 8), (16, 130, 1096), (13, 2560, 2560)])
def test_gemm_fused_epilogues_streaming_tile(oracle, kind, rows, cols, kslice, M, N, K):
    a, w, bias, r1, r2 = _fused_inputs(M, N, K, M + N + K + kind)
    res = (dev(r1), dev(r2)) if kind in (1, 2) else (None, None)
    out = Guarded((M, N), torch.float32 if kind == 2 else torch.float16)
    c = cfg(variant=_lib.GEMM_STREAM, block=4 * cols, vec=8, unroll=1, tile=[rows, cols, kslice])
    ops.gemm(dev(a), dev(w), dev(bias), out.t, c, epilogue=kind, res1=res[0], res2=res[1])
    want = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind, threads=8)
    _check_fused(out.check(), want, oracle.np64.gemm_fused(a, w, bias, r1, r2, kind), kind, r1, r2)


@pytest.mark.parametrize("kind,N,K", [(1, 2560, 2560), (2, 2560, 2560), (3, 10240, 2560)])
def test_gemm_fused_at_the_models_shapes(oracle, kind, N, K):
    M = 300
    a, w, bias, r1, r2 = _fused_inputs(M, N, K, kind)
    res = (dev(r1), dev(r2)) if kind in (1, 2) else (None, None)
    out = Guarded((1, M, N), torch.float32 if kind == 2 else torch.float16)
    ops.gemm(dev(a), dev(w), dev(bias), out.t, None, epilogue=kind, res1=res[0], res2=res[1])
    want = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind, threads=8)
    _check_fused(out.check().reshape(M, N), want, oracle.np64.gemm_fused(a, w, bias, r1, r2, kind), kind, r1, r2)


@pytest.mark.parametrize("kind", [0, 1, 2, 3])
@pytest.mark.parametrize("rows,block", [(None, None), (1, 64), (2, 256), (4, 512), (8, 256)])
@pytest.mark.parametrize("N,K", [(2560, 2560), (10240, 2560), (1001, 520), (7, 8), (33, 1003)])
def test_gemv_fused_epilogues(oracle, kind, rows, block, N, K):
    # the decode forms fused_NT_matmul8_add5_add7_add7(_cast5) and fused_NT_matmul9_add6_gelu1 on every GEMV
    # variant (K = 1003: the element-access kernel)
    a, w, bias, r1, r2 = _fused_inputs(1, N, K, N + K + kind)
    res = (dev(r1), dev(r2)) if kind in (1, 2) else (None, None)
    out = Guarded((1, 1, N), torch.float32 if kind == 2 else torch.float16)
    c = None if rows is None else cfg(variant=_lib.GEMV_SPLITK, block=block, vec=8, unroll=2, tile=[rows, 0, 0])
    ops.gemv(dev(a), dev(w), dev(bias), out.t, c, epilogue=kind, res1=res[0], res2=res[1])
    want = oracle.c.gemm_fused(a, w, bias, r1 if kind in (1, 2) else None, r2 if kind in (1, 2) else None, kind)
    _check_fused(out.check().reshape(1, N), want, oracle.np64.gemm_fused(a, w, bias, r1, r2, kind), kind, r1, r2)


def test_gemv_fused_is_what_one_row_of_the_gemm_entry_runs_and_errors(oracle):
    a, w, bias, r1, r2 = _fused_inputs(1, 2560, 2560, 11)
    via_gemv = Guarded((1, 2560), torch.float16)
    ops.gemv(dev(a), dev(w), dev(bias), via_gemv.t, None, epilogue=1, res1=dev(r1), res2=dev(r2))
    via_gemm = Guarded((1, 2560), torch.float16)
    ops.gemm(dev(a), dev(w), dev(bias), via_gemm.t, None, epilogue=1, res1=dev(r1), res2=dev(r2))
    assert_bits_equal(via_gemv.check(), via_gemm.check())
    # without a bias the epilogue still applies
    out = Guarded((1, 2560), torch.float16)
    ops.gemv(dev(a), dev(w), None, out.t, None, epilogue=3)
    want = oracle.c.gemm_fused(a, w, None, None, None, 3)
    _check_fused(out.check(), want, oracle.np64.gemm_fused(a, w, None, r1, r2, 3), 3)
    y = torch.empty(2560, dtype=torch.float16, device="cuda")
    L = _lib.lib()
    with pytest.raises(_lib.DtasError, match="residual"):
        _lib.check(L.dtas_gemv_f16_fused(dev(a).data_ptr(), dev(w).data_ptr(), None, None, None, y.data_ptr(), 2560, 2560,
                                         _lib.EPI_BIAS_ADD2, None, None), "fused")
    with pytest.raises(_lib.DtasError, match="residual"):
        _lib.check(L.dtas_gemv_f16_fused(dev(a).data_ptr(), dev(w).data_ptr(), None, dev(r1).data_ptr(), None, y.data_ptr(),
                                         2560, 2560, _lib.EPI_BIAS_GELU, None, None), "fused")
    with pytest.raises(_lib.DtasError, match="epilogue"):
        _lib.check(L.dtas_gemv_f16_fused(dev(a).data_ptr(), dev(w).data_ptr(), None, None, None, y.data_ptr(), 2560, 2560,
                                         7, None, None), "fused")
    with pytest.raises(_lib.DtasError, match="overlaps"):
        _lib.check(L.dtas_gemv_f16_fused(dev(a).data_ptr(), dev(w).data_ptr(), None, y.data_ptr(), dev(r2).data_ptr(),
                                         y.data_ptr(), 2560, 2560, _lib.EPI_BIAS_ADD2, None, None), "fused")
    with pytest.raises(ValueError, match="fp32 y"):
        ops.gemv(dev(a), dev(w), None, y, None, epilogue=_lib.EPI_BIAS_ADD2_CAST_F32, res1=dev(r1), res2=dev(r2))


def test_gemm_fused_argument_errors():
    a, w, bias, r1, r2 = _fused_inputs(8, 16, 16, 1)
    out = torch.empty(8, 16, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match="residual"):
        _lib.check(_lib.lib().dtas_gemm_f16_fused(dev(a).data_ptr(), dev(w).data_ptr(), None, None, None, out.data_ptr(),
                                                  8, 16, 16, _lib.EPI_BIAS_ADD2, None, None), "fused")
    with pytest.raises(_lib.DtasError, match="epilogue"):
        _lib.check(_lib.lib().dtas_gemm_f16_fused(dev(a).data_ptr(), dev(w).data_ptr(), None, None, None, out.data_ptr(),
                                                  8, 16, 16, 9, None, None), "fused")
    with pytest.raises(ValueError, match="fp32 C"):
        ops.gemm(dev(a), dev(w), None, out, None, epilogue=_lib.EPI_BIAS_ADD2_CAST_F32, res1=dev(r1), res2=dev(r2))


def test_gelu_over_every_fp16_preactivation(oracle):
    """A product that is exactly x (one 1 in W) for every finite fp16 x: the epilogue's erf is a polynomial
    fitted for fp16 inputs and outputs, the oracle's is libm's; the rounded results may differ in a handful
    of the 63 488 values, by one fp16 ulp."""
    bits = np.concatenate([np.arange(0, 0x7c00, dtype=np.uint16), np.arange(0x8000, 0xfc00, dtype=np.uint16)])
    a = np.zeros((bits.size, 8), np.float16)
    a[:, 0] = bits.view(np.float16)
    w = np.zeros((8, 8), np.float16)
    w[:, 0] = 1                                                       # every column of C repeats x
    want = oracle.c.gemm_fused(a, w, None, None, None, 3, threads=8)
    for conf in (None, dict(variant=0, block=256, vec=8, unroll=2, tile=[64, 64, 64])):
        out = Guarded((bits.size, 8), torch.float16)
        ops.gemm(dev(a), dev(w), None, out.t, cfg(**conf) if conf else None, epilogue=_lib.EPI_BIAS_GELU)
        got = out.check()
        assert np.isfinite(got).all()
        diff = got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32)
        assert np.abs(diff).max() <= 1
        assert (diff[:, 0] != 0).sum() <= 16, (diff[:, 0] != 0).sum()
    # the decode path (q8 GEMV) and the skinny kernel share the same steps


@pytest.mark.parametrize("N,K", [(50280, 2560), (4096, 4096), (101, 36), (7, 4)])
def test_gemv_f32(oracle, N, K):
    """NT_matmul5: fp32 in, fp32 out.  The kernel's summation order differs from the oracle's running sum, so both
    are held to the float64 product within the bound a K-term fp32 sum carries."""
    rng = np.random.default_rng(N + K)
    x = rng.standard_normal(K).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    out = Guarded((1, 1, N), torch.float32)
    ops.gemv_f32(dev(x).view(1, 1, K), dev(w), out.t)
    got = out.check().reshape(N).astype(np.float64)
    f64 = w.astype(np.float64) @ x.astype(np.float64)
    mag = np.abs(w.astype(np.float64)) @ np.abs(x.astype(np.float64))
    assert (np.abs(got - f64) <= mag * 64 * 2.0 ** -24 + 1e-30).all()          # far inside rtol 1e-2
    want = oracle.c.gemv_f32(x, w, threads=8).astype(np.float64)
    assert (np.abs(got - want) <= mag * K * 2.0 ** -24 + 1e-30).all()


def test_gemv_f32_variants_exact_cases_and_errors(oracle):
    rng = np.random.default_rng(77)
    N, K = 203, 1028
    w = rng.integers(-8, 9, (N, K)).astype(np.float32)                        # sums of small integers are exact in fp32
    x = rng.integers(-8, 9, K).astype(np.float32)
    want = (w.astype(np.int64) @ x.astype(np.int64)).astype(np.float32)
    for rows in (1, 2, 4, 8):
        for block in (64, 256, 512):
            out = Guarded((N,), torch.float32)
            ops.gemv_f32(dev(x), dev(w), out.t, cfg(variant=_lib.GEMV_SPLITK, block=block, vec=4, unroll=2, tile=[rows, 0, 0]))
            assert np.array_equal(out.check(), want)
    out = Guarded((N,), torch.float32)
    ops.gemv_f32(dev(x), dev(w), out.t, cfg(variant=_lib.GEMV_SPLITK, block=256, vec=1, unroll=1, tile=[1, 0, 0]))
    assert np.array_equal(out.check(), want)
    # K % 4 != 0 and an odd x pointer take the element path
    w3, x3 = np.ascontiguousarray(w[:, :1027]), np.ascontiguousarray(x[:1027])
    out = Guarded((N,), torch.float32)
    ops.gemv_f32(dev(x3), dev(w3), out.t)
    assert np.array_equal(out.check(), (w3.astype(np.int64) @ x3.astype(np.int64)).astype(np.float32))
    xb = torch.empty(K + 1, dtype=torch.float32, device="cuda")
    xb[1:].copy_(dev(x))
    out = Guarded((N,), torch.float32)
    ops.gemv_f32(xb[1:], dev(w), out.t)
    assert np.array_equal(out.check(), want)
    with pytest.raises(_lib.DtasError, match="vector width"):
        ops.gemv_f32(dev(x), dev(w), out.t, cfg(variant=_lib.GEMV_SPLITK, block=256, vec=2, unroll=1, tile=[1, 0, 0]))
    assert _lib.lib().dtas_gemv_f32(None, None, None, 0, 8, None, None) == 0

"""GPU parity of the q8f16_1 kernels (dequantiser and dequantising GEMV,
experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py:335-343, :401-426, :428-502) through the C ABI against the
CPU oracle: the dequantised weights are bit-exact (integer bytes, one fp16 product); the GEMV is held to rtol 1e-2
against float64 and to an fp16 ulp or two of the oracle (fp32 summation order)."""
import numpy as np
import pytest
import torch

from dtas_amd import _lib, ops
from gpu_util import Guarded, cfg, dev

pytestmark = pytest.mark.gpu


def _weights(N, K, seed):
    rng = np.random.default_rng(seed)
    wq = rng.integers(0, 2 ** 32, (N, K // 4), dtype=np.uint32)
    scale = (rng.random((N, K // 32)) * 0.02 + 0.001).astype(np.float16)
    return wq, scale


def _words(wq):
    return torch.from_numpy(wq.view(np.int32)).cuda()


@pytest.mark.parametrize("N,K", [(1, 32), (3, 96), (2560, 2560), (7680, 2560), (50, 10240)])
def test_decode_is_bit_exact(oracle, N, K):
    wq, scale = _weights(N, K, N + K)
    out = Guarded((N, K), torch.float16)
    ops.decode_q8(_words(wq), dev(scale), out.t)
    assert np.array_equal(out.check().view(np.uint16), oracle.c.decode_q8(wq, scale, threads=8).view(np.uint16))


def test_decode_every_byte_value_scalar_path_and_errors(oracle):
    # all 256 byte values against scales that make the fp16 product round, overflow and go subnormal
    wq = np.tile(np.arange(256, dtype=np.uint8), 4).reshape(4, 256).view(np.uint32)
    scale = np.array([[1 / 3, 0.1, 7.0, 1e-3, 1.0, 6e-8, 0.5, 600.0]] * 4, np.float16)   # 600 * (255 - 127) overflows
    want = oracle.c.decode_q8(np.ascontiguousarray(wq), scale)
    for vec in (8, 1):
        out = Guarded((4, 256), torch.float16)
        ops.decode_q8(_words(np.ascontiguousarray(wq)), dev(scale), out.t, cfg(variant=_lib.ELT_VECTOR, block=256, vec=vec))
        got = out.check()
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    assert np.isinf(want).any() and (want == 0).any()
    # an output that is only 2-byte aligned takes the element path
    buf = torch.empty(4 * 256 + 1, dtype=torch.float16, device="cuda")
    ops.decode_q8(_words(np.ascontiguousarray(wq)), dev(scale), buf[1:].view(4, 256))
    torch.cuda.synchronize()
    assert np.array_equal(buf[1:].cpu().numpy().reshape(4, 256).view(np.uint16), want.view(np.uint16))
    with pytest.raises(ValueError, match="groups of 32"):
        ops.decode_q8(torch.zeros(2, 4, dtype=torch.int32, device="cuda"), torch.zeros(2, 1, dtype=torch.float16, device="cuda"),
                      torch.zeros(2, 16, dtype=torch.float16, device="cuda"))
    L = _lib.lib()
    assert L.dtas_decode_q8_f16(None, None, None, 4, 48, None, None) == -1 and b"multiple of the scale group" in L.dtas_last_error()
    assert L.dtas_decode_q8_f16(None, None, None, 0, 64, None, None) == 0


def _check_gemv(got, x, wq, scale, bias, kind, oracle):
    want = oracle.c.gemv_q8(x, wq, scale, bias, kind=kind, threads=8)
    w64 = oracle.c.decode_q8(wq, scale, threads=8).astype(np.float64)
    f64 = w64 @ x.astype(np.float64) + (bias.astype(np.float64) if bias is not None else 0.0)
    if kind == _lib.EPI_BIAS_GELU:
        from scipy.special import erf
        f64 = f64 * (0.5 + 0.5 * erf(f64 * 0.70710678118654757))
    mag = np.abs(w64) @ np.abs(x.astype(np.float64)) * 2.0 ** -11 + 2e-3       # what rounding the sum to fp16 can move
    assert np.isfinite(got).all()
    assert (np.abs(got.astype(np.float64) - f64) <= 1e-2 * np.abs(f64) + mag).all()
    assert (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 2.0 ** -9 * np.abs(want) + 2e-3).all()
    assert (got == want).mean() > 0.9


@pytest.mark.parametrize("N,K", [(7680, 2560), (2560, 10240), (10240, 2560), (50280, 2560), (33, 64), (5, 32),
                                 (13824, 1024), (16400, 512), (12300, 2048), (5120, 1024), (4096, 8192), (20000, 768)])
@pytest.mark.parametrize("kind", [_lib.EPI_BIAS, _lib.EPI_BIAS_GELU])
def test_gemv_builtin_config(oracle, N, K, kind):
    rng = np.random.default_rng(N + K + kind)
    wq, scale = _weights(N, K, N * 3 + K)
    x = rng.standard_normal(K).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    out = Guarded((1, 1, N), torch.float16)
    ops.gemv_q8(dev(x).view(1, 1, K), _words(wq), dev(scale), dev(bias), out.t, None, kind)
    _check_gemv(out.check().reshape(N), x, wq, scale, bias, kind, oracle)


@pytest.mark.parametrize("rows", [1, 2, 4, 8])
@pytest.mark.parametrize("block", [64, 256, 512])
def test_gemv_every_row_count_and_block(oracle, rows, block):
    rng = np.random.default_rng(rows + block)
    N, K = 101, 1056                       # N not a multiple of the rows per workgroup; K/16 = 66 chunks over up to 512 lanes
    wq, scale = _weights(N, K, rows * 7 + block)
    x = rng.standard_normal(K).astype(np.float16)
    out = Guarded((N,), torch.float16)
    ops.gemv_q8(dev(x), _words(wq), dev(scale), None, out.t, cfg(variant=_lib.GEMV_SPLITK, block=block, vec=8, unroll=2, tile=[rows, 0, 0]))
    _check_gemv(out.check(), x, wq, scale, None, _lib.EPI_BIAS, oracle)


def test_gemv_exact_cases_scalar_path_and_errors(oracle):
    # a one-hot x picks a column of the dequantised matrix, bit for bit
    wq, scale = _weights(64, 128, 5)
    w = oracle.c.decode_q8(wq, scale)
    for k in (0, 3, 31, 32, 127):
        x = np.zeros(128, np.float16)
        x[k] = 1
        out = Guarded((64,), torch.float16)
        ops.gemv_q8(dev(x), _words(wq), dev(scale), None, out.t)
        assert np.array_equal(out.check().view(np.uint16), w[:, k].view(np.uint16))
    # odd x pointer -> element path
    rng = np.random.default_rng(6)
    x = rng.standard_normal(128).astype(np.float16)
    xbuf = torch.empty(129, dtype=torch.float16, device="cuda")
    xbuf[1:].copy_(dev(x))
    out = Guarded((64,), torch.float16)
    ops.gemv_q8(xbuf[1:], _words(wq), dev(scale), None, out.t)
    _check_gemv(out.check(), x, wq, scale, None, _lib.EPI_BIAS, oracle)
    y = torch.empty(64, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match="epilogue must be"):
        ops.gemv_q8(dev(x), _words(wq), dev(scale), None, y, None, _lib.EPI_BIAS_ADD2)
    assert _lib.lib().dtas_gemv_q8_f16(None, None, None, None, None, 0, 64, 0, None, None) == 0


def test_q8_through_the_primfunc_descriptors_and_engine(oracle):
    from dtas_amd import primfuncs as pf
    from dtas_amd.arch import MI355X
    from dtas_amd.engine.tuner import Engine

    rng = np.random.default_rng(8)
    N, K = 7680, 2560
    wq, scale = _weights(N, K, 9)
    x = rng.standard_normal(K).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    mod = pf.module(pf.fused_decode_NT_matmul_add(N, K), pf.fused_decode(N, K), pf.matmul_pv(32, 80, decode=True))
    rt = Engine(topk=2, parallel_build=False).tune_module(mod, MI355X())
    assert rt.entry_for("fused_fused_decode2_fused_NT_matmul_add") is None      # the library's own choice
    y = torch.empty(1, 1, N, dtype=torch.float16, device="cuda")
    rt["fused_fused_decode2_fused_NT_matmul_add"](_words(wq), dev(scale), dev(x).view(1, 1, K), dev(bias), y)
    W = torch.empty(N, K, dtype=torch.float16, device="cuda")
    rt["fused_decode3"](_words(wq), dev(scale), W)
    torch.cuda.synchronize()
    _check_gemv(y.cpu().numpy().reshape(N), x, wq, scale, bias, _lib.EPI_BIAS, oracle)
    assert np.array_equal(W.cpu().numpy().view(np.uint16), oracle.c.decode_q8(wq, scale, threads=8).view(np.uint16))


def test_q8_full_size_properties(oracle):
    """The embedding-sized matrix (50280 x 2560) and the benchmark's largest GEMV (32000 x 4096): dequantising
    twice gives the same bits, the GEMV is linear in x for exactly representable data, and a one-hot x returns a
    column of the dequantised matrix."""
    for N, K in ((50280, 2560), (32000, 4096)):
        g = torch.Generator(device="cuda").manual_seed(N)
        words = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 4), dtype=torch.int32, device="cuda", generator=g)
        scale = (torch.rand(N, K // 32, device="cuda", generator=g) * 0.02 + 0.001).half()
        W = torch.empty(N, K, dtype=torch.float16, device="cuda")
        ops.decode_q8(words, scale, W)
        torch.cuda.synchronize()
        # against torch's own arithmetic on the bytes (little endian), every element
        by = words.view(torch.uint8).view(N, K).to(torch.float16) - 127
        assert bool((W == by * scale.repeat_interleave(32, dim=1)).all())
        del by
        y = torch.empty(N, dtype=torch.float16, device="cuda")
        for kcol in (0, 31, 32, K - 1):
            x = torch.zeros(K, dtype=torch.float16, device="cuda")
            x[kcol] = 1
            ops.gemv_q8(x, words, scale, None, y)
            assert bool((y == W[:, kcol]).all())
        # sampled rows of a dense GEMV against the oracle
        x = torch.randn(K, device="cuda", generator=g).half()
        ops.gemv_q8(x, words, scale, None, y)
        rows = [0, 1, N // 2, N - 1]
        wq = words[rows].cpu().numpy().view(np.uint32)
        want = oracle.c.gemv_q8(x.cpu().numpy(), np.ascontiguousarray(wq), np.ascontiguousarray(scale[rows].cpu().numpy())).astype(np.float64)
        got = y[rows].cpu().numpy().astype(np.float64)
        assert (np.abs(got - want) <= 2e-3 + 2.0 ** -8 * np.abs(want)).all()


def test_q8_dynamic_n_primfuncs_through_the_module(oracle):
    """fused_fused_decode2_fused_NT_matmul6_add4 / ..decode4.._gelu1 (n dynamic): dequantise, then the fp16 GEMM;
    n = 1 goes to the dequantising GEMV.  Against the oracle's GEMM on the oracle's dequantised matrix."""
    from dtas_amd import primfuncs as pf
    from dtas_amd.arch import MI355X
    from dtas_amd.engine.tuner import Engine

    rng = np.random.default_rng(21)
    N, K = 640, 512
    wq, scale = _weights(N, K, 22)
    bias = rng.standard_normal(N).astype(np.float16)
    w = oracle.c.decode_q8(wq, scale)
    mod = pf.module(pf.fused_decode_NT_matmul_add_dyn(N, K), pf.fused_decode_NT_matmul_add_dyn(N, K, gelu=True))
    rt = Engine(topk=2, parallel_build=False).tune_module(mod, MI355X())
    for name, kind in (("fused_fused_decode2_fused_NT_matmul6_add4", 0), ("fused_fused_decode4_fused_NT_matmul9_add6_gelu1", 3)):
        for n in (1, 7, 200):
            a = rng.standard_normal((1, n, K)).astype(np.float16)
            out = torch.empty(1, n, N, dtype=torch.float16, device="cuda")
            rt[name](_words(wq), dev(scale), dev(a), dev(bias), out)
            torch.cuda.synchronize()
            want = oracle.c.gemm_fused(a[0], w, bias, None, None, kind, threads=8).astype(np.float64)
            got = out.cpu().numpy()[0].astype(np.float64)
            assert (np.abs(got - want) <= 4e-3 + 2.0 ** -8 * np.abs(want)).all(), (name, n)


def _check_gemm_q8(got, a, wq, scale, bias, r1, r2, kind, oracle):
    w = oracle.c.decode_q8(wq, scale, threads=8)
    want = oracle.c.gemm_fused(a, w, bias, r1, r2, kind, threads=8).astype(np.float64)
    w64 = w.astype(np.float64)
    f64 = a.astype(np.float64) @ w64.T + (bias.astype(np.float64) if bias is not None else 0.0)
    if kind in (1, 2):
        f64 = r1.astype(np.float64) + f64 + r2.astype(np.float64)
    elif kind == 3:
        from scipy.special import erf
        f64 = f64 * (0.5 + 0.5 * erf(f64 * 0.70710678118654757))
    mag = np.abs(a.astype(np.float64)) @ np.abs(w64).T
    if kind in (1, 2):
        mag = mag + np.abs(r1.astype(np.float64)) + np.abs(r2.astype(np.float64))
    got = got.astype(np.float64)
    assert np.isfinite(got).all()
    assert (np.abs(got - f64) <= 1e-2 * np.abs(f64) + mag * 2.0 ** -9 + 4e-3).all()
    assert (np.abs(got - want) <= 2.0 ** -8 * np.maximum(np.abs(want), mag * 2.0 ** -3) + 4e-3).all()
    assert (got == want).mean() > 0.9


Q8_GEMM_CONFIGS = [None,
                   dict(variant=0, block=256, vec=8, unroll=3, tile=[256, 128, 64]),
                   dict(variant=0, block=256, vec=8, unroll=3, tile=[128, 128, 64]),
                   dict(variant=0, block=256, vec=8, unroll=2, tile=[64, 64, 64]),
                   # K split over workgroups: the parts meet in the split-K workspace as the fp16 GEMM's do
                   dict(variant=0, block=256, vec=8, unroll=3, tile=[256, 128, 64], split_k=2),
                   dict(variant=0, block=256, vec=8, unroll=3, tile=[128, 128, 64], split_k=3),
                   dict(variant=0, block=256, vec=8, unroll=2, tile=[64, 64, 64], split_k=8),
                   # the three-stage tiles of the fitted built-in choice
                   dict(variant=0, block=256, vec=8, unroll=3, tile=[64, 64, 64]),
                   dict(variant=0, block=256, vec=8, unroll=3, tile=[128, 64, 64], split_k=2),
                   dict(variant=0, block=256, vec=8, unroll=3, tile=[64, 128, 64]),
                   dict(variant=0, block=256, vec=8, unroll=3, tile=[64, 64, 64], split_k=6)]


@pytest.mark.parametrize("which", range(len(Q8_GEMM_CONFIGS)))
@pytest.mark.parametrize("M,N,K", [(2, 40, 32), (77, 200, 96), (130, 257, 160), (300, 384, 1056), (520, 130, 64)])
@pytest.mark.parametrize("kind", [0, 1, 3])
def test_gemm_q8_every_tile_on_ragged_shapes(oracle, which, M, N, K, kind):
    # K = 32 .. 1056: half a k tile, one and a half, two and a half, many (every prologue / drain case)
    rng = np.random.default_rng(M + N + K + kind)
    wq, scale = _weights(N, K, M * 3 + N)
    a = rng.standard_normal((M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    r1 = rng.standard_normal((M, N)).astype(np.float16) if kind == 1 else None
    r2 = rng.standard_normal((M, N)).astype(np.float16) if kind == 1 else None
    out = Guarded((M, N), torch.float16)
    conf = Q8_GEMM_CONFIGS[which]
    ops.gemm_q8(dev(a), _words(wq), dev(scale), dev(bias), out.t, cfg(**conf) if conf else None, kind,
                dev(r1) if r1 is not None else None, dev(r2) if r2 is not None else None)
    _check_gemm_q8(out.check(), a, wq, scale, bias, r1, r2, kind, oracle)


@pytest.mark.parametrize("M", [1, 16, 32, 64, 96, 128, 192, 256, 384, 512, 2048])
@pytest.mark.parametrize("N,K,kind", [(7680, 2560, 0), (10240, 2560, 3), (2560, 10240, 0), (2560, 2560, 1)])
def test_gemm_q8_at_the_models_shapes(oracle, M, N, K, kind):
    rng = np.random.default_rng(M + N + kind)
    wq, scale = _weights(N, K, N + K)
    a = rng.standard_normal((M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    r1 = rng.standard_normal((M, N)).astype(np.float16) if kind == 1 else None
    r2 = rng.standard_normal((M, N)).astype(np.float16) if kind == 1 else None
    out = Guarded((1, M, N), torch.float16)
    ops.gemm_q8(dev(a).view(1, M, K), _words(wq), dev(scale), dev(bias), out.t, None, kind,
                dev(r1) if kind == 1 else None, dev(r2) if kind == 1 else None)
    rows = np.unique(np.concatenate([np.arange(min(M, 8)), [M // 2, M - 1]]))       # sampled rows against the oracle
    _check_gemm_q8(out.check().reshape(M, N)[rows], np.ascontiguousarray(a[rows]), wq, scale, bias,
                   None if r1 is None else np.ascontiguousarray(r1[rows]), None if r2 is None else np.ascontiguousarray(r2[rows]), kind, oracle)


@pytest.mark.parametrize("M", [33, 48, 64])
@pytest.mark.parametrize("N,K", [(2048, 4096), (4096, 2048), (3072, 3072), (4096, 2560), (4096, 4096)])
def test_gemm_q8_33_to_64_rows_either_side_of_one_round_of_the_streaming_form(oracle, M, N, K):
    # 64 columns x 512 of K per workgroup: the first two shapes are one round of the chip (the W-streaming kernel),
    # the others more (the tiles with K in parts)
    rng = np.random.default_rng(M + N + K)
    wq, scale = _weights(N, K, N + K + 1)
    a = rng.standard_normal((M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    out = Guarded((1, M, N), torch.float16)
    ops.gemm_q8(dev(a).view(1, M, K), _words(wq), dev(scale), dev(bias), out.t)
    rows = np.unique(np.concatenate([np.arange(8), [M // 2, M - 1]]))
    _check_gemm_q8(out.check().reshape(M, N)[rows], np.ascontiguousarray(a[rows]), wq, scale, bias, None, None, 0, oracle)


Q8_STREAM_TILES = [(16, 64, 512), (16, 64, 1024), (32, 64, 512), (64, 64, 512)]


@pytest.mark.parametrize("kind", [0, 1, 2, 3])
@pytest.mark.parametrize("rows,cols,kslice", Q8_STREAM_TILES)
@pytest.mark.parametrize("M,N,K", [(1, 64, 256), (5, 7, 512), (16, 130, 768), (13, 200, 1280), (16, 2560, 2560), (9, 333, 4096)])
def test_gemm_q8_streaming_tiles(oracle, kind, rows, cols, kslice, M, N, K):
    M = M if M < 16 else rows                                  # a full tile of rows where the case asks for one
    # the W-streaming kernel on bytes: K of one slice, a slice and a half, several; ragged N; every epilogue
    rng = np.random.default_rng(M + N + K + kind)
    wq, scale = _weights(N, K, M * 5 + N)
    a = rng.standard_normal((M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    r1 = rng.standard_normal((M, N)).astype(np.float16) if kind in (1, 2) else None
    r2 = rng.standard_normal((M, N)).astype(np.float16) if kind in (1, 2) else None
    out = Guarded((M, N), torch.float32 if kind == 2 else torch.float16)
    c = cfg(variant=_lib.GEMM_STREAM, block=256, vec=8, unroll=1, tile=[rows, cols, kslice])
    ops.gemm_q8(dev(a), _words(wq), dev(scale), dev(bias), out.t, c, kind,
                dev(r1) if r1 is not None else None, dev(r2) if r2 is not None else None)
    _check_gemm_q8(out.check(), a, wq, scale, bias, r1, r2, kind, oracle)


def test_gemm_q8_streaming_is_the_choice_for_few_rows_exact_and_reproducible(oracle):
    # one-hot rows of A return decoded columns of W bit for bit, through the route cfg = NULL takes for M <= 16
    wq, scale = _weights(200, 1280, 3)
    w = oracle.c.decode_q8(wq, scale)
    ks = (0, 7, 31, 32, 511, 512, 1279)
    a = np.zeros((len(ks), 1280), np.float16)
    for i, k in enumerate(ks):
        a[i, k] = 1
    out = Guarded((len(ks), 200), torch.float16)
    ops.gemm_q8(dev(a), _words(wq), dev(scale), None, out.t)
    assert np.array_equal(out.check().view(np.uint16), np.ascontiguousarray(w[:, list(ks)].T).view(np.uint16))
    # K slices are added in slice order whoever arrives last: three launches agree bit for bit
    rng = np.random.default_rng(8)
    wq, scale = _weights(2560, 2560, 9)
    a = rng.standard_normal((16, 2560)).astype(np.float16)
    runs = []
    for _ in range(3):
        out = Guarded((16, 2560), torch.float16)
        ops.gemm_q8(dev(a), _words(wq), dev(scale), None, out.t)
        runs.append(out.check())
    assert all(np.array_equal(r.view(np.uint16), runs[0].view(np.uint16)) for r in runs)
    _check_gemm_q8(runs[0], a, wq, scale, None, None, None, 0, oracle)
    # K off 256: the tiles take over
    wq, scale = _weights(96, 160, 5)
    a = rng.standard_normal((4, 160)).astype(np.float16)
    out = Guarded((4, 96), torch.float16)
    ops.gemm_q8(dev(a), _words(wq), dev(scale), None, out.t)
    _check_gemm_q8(out.check(), a, wq, scale, None, None, None, 0, oracle)
    c = torch.empty(4, 96, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match="K % 256"):
        ops.gemm_q8(dev(a), _words(wq), dev(scale), None, c, cfg(variant=_lib.GEMM_STREAM, block=256, vec=8, unroll=1, tile=[16, 64, 512]))
    with pytest.raises(_lib.DtasError, match="cannot hold M=17"):
        ops.gemm_q8(dev(np.zeros((17, 256), np.float16)), _words(_weights(8, 256, 1)[0]), dev(_weights(8, 256, 1)[1]), None,
                    torch.empty(17, 8, dtype=torch.float16, device="cuda"), cfg(variant=_lib.GEMM_STREAM, block=256, vec=8, unroll=1, tile=[16, 64, 512]))
    with pytest.raises(_lib.DtasError, match="16x64x512, 16x64x1024, 32x64x512 and 64x64x512"):
        ops.gemm_q8(dev(a), _words(wq), dev(scale), None, c, cfg(variant=_lib.GEMM_STREAM, block=512, vec=8, unroll=1, tile=[16, 128, 512]))


def test_gemm_q8_exact_cases_fallback_and_errors(oracle):
    # A = rows of the identity returns columns... of W^T: C[i, :] = decoded W[:, k_i], bit for bit
    wq, scale = _weights(96, 128, 3)
    w = oracle.c.decode_q8(wq, scale)
    a = np.zeros((5, 128), np.float16)
    for i, k in enumerate((0, 7, 31, 32, 127)):
        a[i, k] = 1
    out = Guarded((5, 96), torch.float16)
    ops.gemm_q8(dev(a), _words(wq), dev(scale), None, out.t)
    assert np.array_equal(out.check().view(np.uint16), np.ascontiguousarray(w[:, [0, 7, 31, 32, 127]].T).view(np.uint16))
    # an odd A pointer takes the element path
    rng = np.random.default_rng(4)
    a = rng.standard_normal((9, 128)).astype(np.float16)
    abuf = torch.empty(9 * 128 + 1, dtype=torch.float16, device="cuda")
    abuf[1:].copy_(dev(a).flatten())
    out = Guarded((9, 96), torch.float16)
    ops.gemm_q8(abuf[1:].view(9, 128), _words(wq), dev(scale), None, out.t)
    _check_gemm_q8(out.check(), a, wq, scale, None, None, None, 0, oracle)
    c = torch.empty(9, 96, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match="8-bit weights come with tiles"):
        ops.gemm_q8(dev(a), _words(wq), dev(scale), None, c, cfg(variant=0, block=256, vec=8, unroll=2, tile=[128, 128, 64]))
    with pytest.raises(_lib.DtasError, match=r"split_k must be in \[1, 16\]"):
        ops.gemm_q8(dev(a), _words(wq), dev(scale), None, c, cfg(variant=0, block=256, vec=8, unroll=2, tile=[64, 64, 64], split_k=17))
    # K split over workgroups gives the same bits whoever arrives last, launch after launch
    big = rng.standard_normal((70, 1056)).astype(np.float16)
    wq2, scale2 = _weights(130, 1056, 5)
    first = None
    for _ in range(5):
        out = Guarded((70, 130), torch.float16)
        ops.gemm_q8(dev(big), _words(wq2), dev(scale2), None, out.t, cfg(variant=0, block=256, vec=8, unroll=2, tile=[64, 64, 64], split_k=4))
        got = out.check()
        first = got if first is None else first
        assert np.array_equal(got.view(np.uint16), first.view(np.uint16))
    with pytest.raises(_lib.DtasError, match="needs both residuals"):
        ops.gemm_q8(dev(a), _words(wq), dev(scale), None, c, None, _lib.EPI_BIAS_ADD2)
    assert _lib.lib().dtas_gemm_q8_f16_fused(None, None, None, None, None, None, None, 0, 96, 128, 0, None, None) == 0


# ---- the embedding gather and the fp32-scale vocabulary projection (before_dl.py:346-369, :640-657) ----------

@pytest.mark.parametrize("V,K,n", [(50280, 2560, 1), (50280, 2560, 300), (50280, 2560, 4096), (7, 32, 19), (100, 96, 1),
                                   (100, 96, 45), (20, 4128, 5), (9, 2048, 3), (11, 2016, 70)])
def test_take_is_bit_exact(oracle, V, K, n):
    wq, scale = _weights(V, K, V + n)
    ids = np.random.default_rng(n).integers(0, V, n).astype(np.int32)
    ids[0], ids[-1] = V - 1, 0
    out = Guarded((n, K), torch.float16)
    ops.take_q8(_words(wq), dev(scale), dev(ids), out.t)
    want = oracle.c.take_q8(wq, scale, ids, threads=8).view(np.uint16)
    assert np.array_equal(out.check().view(np.uint16), want)
    out = Guarded((n, K), torch.float16)          # a grid cap: the grid-stride kernel
    ops.take_q8(_words(wq), dev(scale), dev(ids), out.t, cfg(variant=_lib.ELT_VECTOR, block=256, vec=8, grid_cap=3))
    assert np.array_equal(out.check().view(np.uint16), want)


def test_take_clips_ids_scalar_path_and_errors(oracle):
    wq, scale = _weights(10, 64, 3)
    ids = np.array([-5, 0, 9, 10, 2 ** 31 - 1, -2 ** 31], np.int32)
    want = oracle.c.take_q8(wq, scale, np.clip(ids, 0, 9).astype(np.int32))
    for vec in (8, 1):
        out = Guarded((6, 64), torch.float16)
        ops.take_q8(_words(wq), dev(scale), dev(ids), out.t, cfg(variant=_lib.ELT_VECTOR, block=256, vec=vec))
        assert np.array_equal(out.check().view(np.uint16), want.view(np.uint16))
    buf = torch.empty(6 * 64 + 1, dtype=torch.float16, device="cuda")            # 2-byte aligned output: element path
    ops.take_q8(_words(wq), dev(scale), dev(ids), buf[1:].view(6, 64))
    torch.cuda.synchronize()
    assert np.array_equal(buf[1:].cpu().numpy().reshape(6, 64).view(np.uint16), want.view(np.uint16))
    L = _lib.lib()
    assert L.dtas_take_q8_f16(None, None, None, None, 0, 10, 64, None, None) == 0
    assert L.dtas_take_q8_f16(None, None, None, None, 3, 10, 64, None, None) == -1 and b"NULL" in L.dtas_last_error()
    assert L.dtas_take_q8_f16(None, None, None, None, 3, 0, 64, None, None) == -1 and b"empty table" in L.dtas_last_error()
    assert L.dtas_take_q8_f16(None, None, None, None, -1, 10, 64, None, None) == -1
    with pytest.raises(ValueError, match="int32 ids"):
        ops.take_q8(_words(wq), dev(scale), torch.zeros(6, dtype=torch.int64, device="cuda"), torch.empty(6, 64, dtype=torch.float16, device="cuda"))


def _weights_f32(N, K, seed):
    rng = np.random.default_rng(seed)
    wq = rng.integers(0, 2 ** 32, (N, K // 4), dtype=np.uint32)
    return wq, (rng.random((N, K // 32)) * 0.02 + 0.001).astype(np.float32)


def _check_gemv_f32(got, x, wq, scale, oracle):
    N, K = wq.shape[0], wq.shape[1] * 4
    want = oracle.c.gemv_q8_f32(x, wq, scale, threads=8)
    w64 = (wq.view(np.uint8).reshape(N, K).astype(np.float64) - 127) * np.repeat(scale.astype(np.float64), 32, axis=1)
    f64 = w64 @ x.astype(np.float64)
    mag = np.abs(w64) @ np.abs(x.astype(np.float64))
    assert np.isfinite(got).all()
    assert (np.abs(got.astype(np.float64) - f64) <= 1e-2 * np.abs(f64) + 1e-5 * mag).all()          # rtol 1e-2 where the sum does not cancel
    assert (np.abs(got.astype(np.float64) - f64) <= (K + 2) * 2.0 ** -24 * mag).all()                # fp32 summation, any order
    assert (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 2 * (K + 2) * 2.0 ** -24 * mag).all()


@pytest.mark.parametrize("N,K", [(50280, 2560), (2560, 10240), (33, 64), (5, 32), (50257, 768), (32000, 2048), (300, 1024), (32000, 4096)])
def test_gemv_f32_scales_builtin_config(oracle, N, K):
    wq, scale = _weights_f32(N, K, N + K)
    x = np.random.default_rng(1).standard_normal(K).astype(np.float32)
    out = Guarded((1, 1, N), torch.float32)
    ops.gemv_q8_f32(dev(x), _words(wq), dev(scale), out.t)
    _check_gemv_f32(out.check().reshape(N), x, wq, scale, oracle)


@pytest.mark.parametrize("rows", [1, 2, 4, 8])
@pytest.mark.parametrize("block", [64, 256, 512])
def test_gemv_f32_scales_every_row_count_and_block(oracle, rows, block):
    N, K = 1001, 2560
    wq, scale = _weights_f32(N, K, rows + block)
    x = np.random.default_rng(2).standard_normal(K).astype(np.float32)
    out = Guarded((N,), torch.float32)
    ops.gemv_q8_f32(dev(x), _words(wq), dev(scale), out.t, cfg(variant=_lib.GEMV_SPLITK, block=block, vec=8, unroll=2, tile=[rows, 0, 0]))
    _check_gemv_f32(out.check(), x, wq, scale, oracle)


def test_gemv_f32_scales_exact_cases_scalar_path_and_errors(oracle):
    wq, scale = _weights_f32(40, 96, 5)
    w32 = (wq.view(np.uint8).reshape(40, 96).astype(np.float32) - np.float32(127)) * np.repeat(scale, 32, axis=1)
    for k in (0, 31, 32, 95):                       # one-hot x returns a column of W: the rounded fp32 product, exactly
        e = np.zeros(96, np.float32)
        e[k] = 1
        for c in (None, cfg(variant=_lib.GEMV_SPLITK, block=256, vec=1, unroll=2, tile=[1, 0, 0])):
            out = Guarded((40,), torch.float32)
            ops.gemv_q8_f32(dev(e), _words(wq), dev(scale), out.t, c)
            assert np.array_equal(out.check().view(np.uint32), w32[:, k].view(np.uint32))
    x = np.random.default_rng(3).standard_normal(96).astype(np.float32)
    buf = torch.empty(97, dtype=torch.float32, device="cuda")                       # x only 4-byte aligned: element path
    buf[1:] = dev(x)
    out = Guarded((40,), torch.float32)
    ops.gemv_q8_f32(buf[1:], _words(wq), dev(scale), out.t)
    _check_gemv_f32(out.check(), x, wq, scale, oracle)
    L = _lib.lib()
    assert L.dtas_gemv_q8_f32(None, None, None, None, 0, 64, None, None) == 0
    assert L.dtas_gemv_q8_f32(None, None, None, None, 4, 48, None, None) == -1 and b"multiple of the scale group" in L.dtas_last_error()
    assert L.dtas_gemv_q8_f32(None, None, None, None, 4, 64, None, None) == -1 and b"NULL" in L.dtas_last_error()
    with pytest.raises(ValueError, match="float32 scales"):
        ops.gemv_q8_f32(dev(x), _words(wq), dev(scale.astype(np.float16)), torch.empty(40, dtype=torch.float32, device="cuda"))


def test_take_and_vocabulary_projection_through_the_primfunc_descriptors(oracle):
    from dtas_amd import primfuncs as pf
    from dtas_amd.arch import MI355X
    from dtas_amd.common.analisys import FuncInfo, FuncKind
    from dtas_amd.engine.tuner import Engine

    V, K = 50280, 2560
    funcs = [pf.fused_decode_take(V, K), pf.fused_decode_take(V, K, decode=True), pf.fused_decode_NT_matmul_f32(V, K)]
    assert [f.name for f in funcs] == ["fused_fused_decode1_take1", "fused_fused_decode1_take", "fused_fused_decode6_NT_matmul5"]
    assert FuncInfo(funcs[0]).kind == FuncKind.kFunc_Elementwise and FuncInfo(funcs[2]).kind == FuncKind.kFunc_GEMV
    rt = Engine(topk=2, parallel_build=False).tune_module(pf.module(*funcs, upper_bound={"n": 1024}), MI355X())
    wq, scale = _weights(V, K, 12)
    ids = np.random.default_rng(4).integers(0, V, 77).astype(np.int32)
    out = torch.empty(77, K, dtype=torch.float16, device="cuda")
    rt["fused_fused_decode1_take1"](_words(wq), dev(scale), dev(ids), out)
    one = torch.empty(1, K, dtype=torch.float16, device="cuda")
    rt["fused_fused_decode1_take"](_words(wq), dev(scale), dev(ids[:1]), one)
    s32 = scale.astype(np.float32)
    x = np.random.default_rng(5).standard_normal(K).astype(np.float32)
    y = torch.empty(1, 1, V, dtype=torch.float32, device="cuda")
    rt["fused_fused_decode6_NT_matmul5"](_words(wq), dev(s32), dev(x).view(1, 1, K), y)
    torch.cuda.synchronize()
    want = oracle.c.take_q8(wq, scale, ids, threads=8)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))
    assert np.array_equal(one.cpu().numpy().view(np.uint16), want[:1].view(np.uint16))
    _check_gemv_f32(y.cpu().numpy().reshape(V), x, wq, s32, oracle)

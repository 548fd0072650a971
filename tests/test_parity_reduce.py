"""GPU parity, RMSNorm / LayerNorm / softmax through the C ABI against the CPU oracle and the
float64 closed forms; tolerance atol 1e-2 (fp16 outputs, fp32 accumulation in another order)."""
import numpy as np
import pytest
import torch

from dtas_amd import _lib, ops
from gpu_util import Guarded, cfg, dev

pytestmark = pytest.mark.gpu

ATOL = 1e-2          # the benchmark's stated tolerance
ATOL_ORACLE = 1e-3   # against the fp32 oracle the only differences are summation order and exp /
RTOL_ORACLE = 2.0 ** -10  # rsqrt ulps: at most one fp16 ulp of the result (plus a small absolute term)


def _check(got, oracle_out, f64):
    got = got.astype(np.float64)
    assert np.isfinite(got).all()
    assert np.abs(got - f64).max() < ATOL
    want = oracle_out.astype(np.float64)
    assert (np.abs(got - want) <= ATOL_ORACLE + RTOL_ORACLE * np.abs(want)).all()


@pytest.mark.parametrize("n", [1, 2, 3, 7, 16, 128, 257, 513, 1024, 4096, 4097, 8192, 8193, 20000])
def test_rms_norm_benchmark_config(oracle, n):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((n, 4096)).astype(np.float16)
    w = rng.uniform(0.5, 1.5, 4096).astype(np.float16)
    out = Guarded(x.shape, torch.float16)
    ops.rms_norm(dev(x), dev(w), out.t)
    _check(out.check(), oracle.c.rms_norm(x, w, threads=8), oracle.np64.rms_norm(x, w))


@pytest.mark.parametrize("H", [8, 64, 2560, 8192, 16384, 100, 4100, 12001])
def test_rms_norm_other_row_lengths(oracle, H):
    rng = np.random.default_rng(H)
    x = rng.standard_normal((5, H)).astype(np.float16)
    w = rng.uniform(0.5, 1.5, H).astype(np.float16)
    out = Guarded(x.shape, torch.float16)
    ops.rms_norm(dev(x), dev(w), out.t)
    _check(out.check(), oracle.c.rms_norm(x, w), oracle.np64.rms_norm(x, w))


# one n per branch of the built-in choice (rows per CU: up to 4, 4 .. 8, 8, 8 .. 12, 12 .. 16, 16 .. 24, beyond)
REGIME_N = [1000, 1500, 2048, 3000, 4090, 6001, 8200]


@pytest.mark.parametrize("n", REGIME_N)
@pytest.mark.parametrize("H", [2560, 5120, 6144, 8192, 16384])
def test_rms_norm_builtin_over_row_lengths_and_counts(oracle, n, H):
    rng = np.random.default_rng(n + H)
    x = rng.standard_normal((n, H), dtype=np.float32).astype(np.float16)
    w = rng.uniform(0.5, 1.5, H).astype(np.float16)
    out = Guarded(x.shape, torch.float16)
    ops.rms_norm(dev(x), dev(w), out.t)
    got = out.check()
    rows = np.unique(np.concatenate([[0, 1, 2, 3, n - 4, n - 3, n - 2, n - 1], rng.integers(0, n, 120)]))
    _check(got[rows], oracle.c.rms_norm(x[rows], w), oracle.np64.rms_norm(x[rows], w))
    # every row, against the closed form of its own output: sum (out / w)^2 = H * sum x^2 / (sum x^2 + H eps)
    ss = (x.astype(np.float64) ** 2).sum(-1)
    assert np.abs(((got.astype(np.float64) / w.astype(np.float64)) ** 2).sum(-1) / (H * ss / (ss + H * 1e-5)) - 1).max() < 5e-3


@pytest.mark.parametrize("n", REGIME_N)
@pytest.mark.parametrize("H", [4096, 5120, 6144, 8192, 16384])
def test_layer_norm_builtin_over_row_lengths_and_counts(oracle, n, H):
    rng = np.random.default_rng(n + H + 1)
    x = (rng.standard_normal((n, H), dtype=np.float32) * 2 + 0.5)
    g = rng.uniform(0.5, 1.5, H).astype(np.float32)
    b = rng.uniform(-1, 1, H).astype(np.float32)
    out = Guarded(x.shape, torch.float16)
    ops.layer_norm(dev(x), dev(g), dev(b), out.t)
    got = out.check()
    rows = np.unique(np.concatenate([[0, 1, 2, 3, n - 4, n - 3, n - 2, n - 1], rng.integers(0, n, 120)]))
    _check(got[rows], oracle.c.layer_norm(x[rows], g, b), oracle.np64.layer_norm(x[rows], g, b))
    # every row: the normalised values ((out - beta) / gamma) have mean 0 and variance 1
    z = (got.astype(np.float64) - b) / g
    assert np.abs(z.mean(-1)).max() < 5e-3 and np.abs(z.var(-1) - 1).max() < 1e-2


RED_VARIANTS = [(_lib.RED_WAVE_ROW, b) for b in (64, 128, 256, 512)] + \
               [(_lib.RED_BLOCK_ROW, b) for b in (64, 256, 512, 1024)] + [(_lib.RED_STREAM_ROW, b) for b in (64, 256, 1024)]


@pytest.mark.parametrize("variant,block", RED_VARIANTS)
@pytest.mark.parametrize("n,H", [(1, 4096), (9, 4096), (130, 2560), (6, 8192)])
def test_rms_norm_every_variant(oracle, variant, block, n, H):
    rng = np.random.default_rng(n + H)
    x = rng.standard_normal((n, H)).astype(np.float16)
    w = rng.uniform(0.5, 1.5, H).astype(np.float16)
    out = Guarded(x.shape, torch.float16)
    vec = 1 if variant == _lib.RED_STREAM_ROW else 8
    ops.rms_norm(dev(x), dev(w), out.t, cfg=cfg(variant=variant, block=block, vec=vec))
    _check(out.check(), oracle.c.rms_norm(x, w), oracle.np64.rms_norm(x, w))


def test_rms_norm_grid_cap_and_invariants(oracle):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((1000, 4096)).astype(np.float16)
    w = np.ones(4096, np.float16)
    for variant in (_lib.RED_WAVE_ROW, _lib.RED_BLOCK_ROW):
        out = Guarded(x.shape, torch.float16)
        ops.rms_norm(dev(x), dev(w), out.t, cfg=cfg(variant=variant, block=256, vec=8, grid_cap=13))
        got = out.check()
        _check(got, oracle.c.rms_norm(x, w, threads=8), oracle.np64.rms_norm(x, w))
        assert np.abs(np.sqrt((got.astype(np.float64) ** 2).mean(-1)) - 1).max() < 2e-3   # unit rms with w = 1


@pytest.mark.parametrize("n", [1, 3, 100, 257, 1024, 4096, 4097, 8192, 8193, 20000])
def test_layer_norm_reference_signature(oracle, n):
    rng = np.random.default_rng(13)
    x = (rng.standard_normal((1, n, 2560)) * 2 + 0.5).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 2560).astype(np.float32)
    b = rng.uniform(-1, 1, 2560).astype(np.float32)
    out = Guarded(x.shape, torch.float16)
    ops.layer_norm(dev(x), dev(g), dev(b), out.t)
    _check(out.check(), oracle.c.layer_norm(x, g, b, threads=8), oracle.np64.layer_norm(x, g, b))


@pytest.mark.parametrize("variant,block", RED_VARIANTS)
def test_layer_norm_every_variant(oracle, variant, block):
    rng = np.random.default_rng(14)
    x = (rng.standard_normal((11, 2560)) * 2 + 0.5).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 2560).astype(np.float32)
    b = rng.uniform(-1, 1, 2560).astype(np.float32)
    out = Guarded(x.shape, torch.float16)
    vec = 1 if variant == _lib.RED_STREAM_ROW else 4
    ops.layer_norm(dev(x), dev(g), dev(b), out.t, cfg=cfg(variant=variant, block=block, vec=vec))
    _check(out.check(), oracle.c.layer_norm(x, g, b), oracle.np64.layer_norm(x, g, b))


def test_layer_norm_odd_row_length(oracle):
    rng = np.random.default_rng(15)
    x = rng.standard_normal((4, 1001)).astype(np.float32)
    g, b = rng.uniform(0.5, 1.5, 1001).astype(np.float32), rng.uniform(-1, 1, 1001).astype(np.float32)
    out = Guarded(x.shape, torch.float16)
    ops.layer_norm(dev(x), dev(g), dev(b), out.t)
    _check(out.check(), oracle.c.layer_norm(x, g, b), oracle.np64.layer_norm(x, g, b))


@pytest.mark.parametrize("n", [1, 2, 3, 7, 8, 16, 31, 64, 128, 257, 512, 1024])
def test_softmax_f16_benchmark_config(oracle, n):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((32 * n, n)) * 2).astype(np.float16)
    out = Guarded(x.shape, torch.float16)
    ops.softmax(dev(x), out.t)
    got = out.check()
    _check(got, oracle.c.softmax(x, threads=8), oracle.np64.softmax(x))
    assert np.abs(got.astype(np.float64).sum(-1) - 1).max() < n * 2.0 ** -11 + 1e-3


@pytest.mark.parametrize("n", [2048, 4096, 8192])
def test_softmax_f16_large_rows_sampled(oracle, n):
    # [32n, n] is 1 GiB at n = 4096 and 4 GiB at 8192, the far end of the dynamic range: run all of it, compare
    # sampled rows with the oracle, row sums for all
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.empty(32 * n, n, dtype=torch.float16, device="cuda")
    for r0 in range(0, 32 * n, 32768):     # in slabs: the fp32 draw of the whole tensor would be 8 GiB at n = 8192
        x[r0:r0 + 32768] = (torch.randn(min(32768, 32 * n - r0), n, device="cuda", generator=g) * 2).half()
    out = torch.empty_like(x)
    ops.softmax(x, out)
    torch.cuda.synchronize()
    rows = np.unique(np.concatenate([[0, 1, 32 * n - 1], np.random.default_rng(n).integers(0, 32 * n, 61)]))
    xs = x[torch.from_numpy(rows).cuda()].cpu().numpy()
    got = out[torch.from_numpy(rows).cuda()].cpu().numpy()
    _check(got, oracle.c.softmax(xs), oracle.np64.softmax(xs))
    sums = torch.cat([out[r0:r0 + 32768].float().sum(-1) for r0 in range(0, 32 * n, 32768)])
    assert float((sums - 1).abs().max()) < n * 2.0 ** -11 + 1e-3
    assert bool((out.argmax(-1) == x.argmax(-1)).float().mean() > 0.999)  # ties in fp16 aside


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (600, 4096), (700, 12288), (520, 5002), (530, 16384), (96, 40000)])
def test_softmax_f16_rows_not_tied_to_the_row_length(oracle, rows, cols):
    # chunked attention: every branch of the built-in choice (a wavefront per row at exactly 8 vectors per lane
    # and few rows, four wavefronts per row up to 2048 vectors, wider workgroups and the streaming form beyond)
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 2).astype(np.float16)
    out = Guarded(x.shape, torch.float16)
    ops.softmax(dev(x), out.t)
    _check(out.check(), oracle.c.softmax(x, threads=8), oracle.np64.softmax(x))


@pytest.mark.parametrize("rows,cols", [(12800, 400), (1000, 1000), (32 * 5, 4096), (7, 8192), (3, 3000), (5, 20000),
                                       (4096, 2048), (600, 2048), (600, 6144), (520, 5001), (300, 8192), (130, 16384)])
def test_softmax_f32_reference_signature(oracle, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((1, rows, cols)) * 2).astype(np.float32)
    out = Guarded(x.shape, torch.float16)
    ops.softmax(dev(x), out.t)
    _check(out.check(), oracle.c.softmax(x, threads=8), oracle.np64.softmax(x))


@pytest.mark.parametrize("variant,block", RED_VARIANTS)
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_softmax_every_variant(oracle, variant, block, dtype):
    rng = np.random.default_rng(16)
    x = (rng.standard_normal((19, 2048)) * 2).astype(dtype)
    out = Guarded(x.shape, torch.float16)
    vec = 1 if variant == _lib.RED_STREAM_ROW else (8 if dtype == np.float16 else 4)
    ops.softmax(dev(x), out.t, cfg=cfg(variant=variant, block=block, vec=vec))
    _check(out.check(), oracle.c.softmax(x), oracle.np64.softmax(x))


def test_softmax_special_rows(oracle):
    x = np.zeros((4, 64), np.float16)
    x[0] = -3.0                      # constant row -> 1/64 exactly
    x[1, 5] = 30000                  # one dominant entry
    x[2] = np.linspace(-60000, 60000, 64).astype(np.float16)
    x[3, :] = -np.inf
    x[3, 7] = 0                      # -inf entries contribute exactly zero
    out = Guarded(x.shape, torch.float16)
    ops.softmax(dev(x), out.t)
    got = out.check()
    assert (got[0] == np.float16(1 / 64)).all()
    assert got[1, 5] == 1 and got[1].sum() == 1
    assert got[3, 7] == 1 and got[3].sum() == 1
    assert np.abs(got.astype(np.float64) - oracle.c.softmax(x).astype(np.float64)).max() < 2e-3


def test_register_variants_step_down_on_ragged_rows(oracle):
    # a bucket's config must serve every n in it: norm rows that are not a multiple of the vector width take
    # the element-access kernel even when the config names a register variant (softmax rows stay in it)
    rng = np.random.default_rng(21)
    x = rng.standard_normal((4, 100)).astype(np.float16)
    w = rng.uniform(0.5, 1.5, 100).astype(np.float16)
    for variant in (_lib.RED_WAVE_ROW, _lib.RED_BLOCK_ROW):
        out = Guarded(x.shape, torch.float16)
        ops.rms_norm(dev(x), dev(w), out.t, cfg=cfg(variant=variant, block=256, vec=8))
        _check(out.check(), oracle.c.rms_norm(x, w), oracle.np64.rms_norm(x, w))
    s = (rng.standard_normal((64, 37)) * 2).astype(np.float16)
    out = Guarded(s.shape, torch.float16)
    ops.softmax(dev(s), out.t, cfg=cfg(variant=_lib.RED_WAVE_ROW, block=64, vec=8))
    _check(out.check(), oracle.c.softmax(s), oracle.np64.softmax(s))


@pytest.mark.parametrize("variant,block", [v for v in RED_VARIANTS if v[0] != _lib.RED_STREAM_ROW])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("rows,cols", [(19, 2047), (19, 2049), (33, 1026), (7, 9), (64, 33), (5, 3), (40, 1)])
def test_softmax_rows_of_any_length_keep_the_register_kernels(oracle, variant, block, dtype, rows, cols):
    # the row length is softmax's dynamic extent: lengths that are not a multiple of the vector width, and rows
    # that start at any element, run in the register kernels with accesses at the rows' own alignment
    if variant == _lib.RED_WAVE_ROW and cols > 64 * 16 * (8 if dtype == np.float16 else 4):
        pytest.skip("row does not fit one wavefront's registers")
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 2).astype(dtype)
    out = Guarded(x.shape, torch.float16)
    ops.softmax(dev(x), out.t, cfg=cfg(variant=variant, block=block, vec=8 if dtype == np.float16 else 4))
    _check(out.check(), oracle.c.softmax(x), oracle.np64.softmax(x))


@pytest.mark.parametrize("n", [9, 33, 257, 1025, 1026, 2047])
def test_softmax_builtin_on_unaligned_lengths_and_buffers(oracle, n):
    rng = np.random.default_rng(n)
    for dtype, tdt in ((np.float16, torch.float16), (np.float32, torch.float32)):
        x = (rng.standard_normal((32 * min(n, 64), n)) * 2).astype(dtype)
        out = Guarded(x.shape, torch.float16)
        ops.softmax(dev(x), out.t)
        _check(out.check(), oracle.c.softmax(x, threads=8), oracle.np64.softmax(x))
        # aligned length, buffers that start one element off a 16-byte boundary
        y = (rng.standard_normal((16, 1024)) * 2).astype(dtype)
        src = torch.empty(16 * 1024 + 1, dtype=tdt, device="cuda")
        src[1:] = dev(y).reshape(-1)
        dst = torch.full((16 * 1024 + 2,), 3.0, dtype=torch.float16, device="cuda")
        ops.softmax(src[1:].view(16, 1024), dst[1:-1].view(16, 1024))
        torch.cuda.synchronize()
        assert dst[0] == 3.0 and dst[-1] == 3.0
        _check(dst[1:-1].view(16, 1024).cpu().numpy(), oracle.c.softmax(y), oracle.np64.softmax(y))


def test_softmax_ragged_special_rows(oracle):
    # the slot across the end of a row is filled with -inf: constant rows at the fp16 minimum, a row whose
    # maximum sits in the last, partial slot, and -inf entries all come out as in the oracle
    x = np.zeros((5, 67), np.float16)
    x[0] = -65504.0                  # the attention mask's value in every position -> 1/67
    x[1, 66] = 30000                 # the dominant entry is the row's last element
    x[2] = np.linspace(-60000, 60000, 67).astype(np.float16)
    x[3, :] = -np.inf
    x[3, 64] = 0
    x[4] = 5.0
    for variant, block in ((_lib.RED_WAVE_ROW, 64), (_lib.RED_BLOCK_ROW, 64), (_lib.RED_BLOCK_ROW, 256)):
        out = Guarded(x.shape, torch.float16)
        ops.softmax(dev(x), out.t, cfg=cfg(variant=variant, block=block, vec=8))
        got = out.check()
        assert (got[0] == np.float16(1 / 67)).all() and (got[4] == np.float16(1 / 67)).all()
        assert got[1, 66] == 1 and got[1].sum() == 1
        assert got[3, 64] == 1 and got[3].sum() == 1
        assert np.abs(got.astype(np.float64) - oracle.c.softmax(x).astype(np.float64)).max() < 2e-3


def test_reduction_errors():
    x = torch.zeros(4, 100, dtype=torch.float16, device="cuda")
    w = torch.ones(100, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match="overlaps"):
        ops.rms_norm(x, w, x)
    with pytest.raises(_lib.DtasError, match="block must be"):
        ops.rms_norm(x, w, torch.empty_like(x), cfg=cfg(variant=_lib.RED_STREAM_ROW, block=100, vec=1))


@pytest.mark.parametrize("rows,cols", [(1, 50280), (1, 1), (3, 4096), (2, 4100), (5, 16384), (2, 50281), (1, 65540), (4, 100000),
                                       (700, 64), (1, 128256), (2, 151936), (1, 65536), (3, 262144)])
@pytest.mark.parametrize("t", [0.7, 1.0, -0.8])
def test_softmax_temperature(oracle, rows, cols, t):
    rng = np.random.default_rng(rows * 7 + cols)
    x = (rng.standard_normal((rows, cols)) * 4).astype(np.float32)
    out = Guarded(x.shape, torch.float32)
    ops.softmax_temperature(dev(x), torch.tensor(t, dtype=torch.float32, device="cuda"), out.t)
    got = out.check().astype(np.float64)
    want = oracle.c.softmax_temperature(x, t, threads=8).astype(np.float64)
    assert np.abs(got - want).max() < 1e-2                                   # the stated tolerance of the reductions
    # the oracle sums the row in fp32 in index order, the kernel as a tree: both within fp32 summation error of the fp64 row
    assert np.abs(got / np.maximum(want, 1e-300) - 1)[want > 1e-30].max() < 1e-3
    want64 = oracle.np64.softmax(x.astype(np.float64) / float(np.float32(t)))
    assert np.abs(got / want64 - 1)[want64 > 1e-30].max() < 3e-5
    assert np.abs(got.sum(-1) - 1).max() < 1e-4
    assert np.array_equal(got.argmax(-1), (x if t > 0 else -x).argmax(-1))


def test_softmax_temperature_unaligned_and_errors(oracle):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(50280 + 1) * 4).astype(np.float32)
    xd = dev(x)[1:]                                                          # 4-byte aligned only: the element path
    out = Guarded((50280,), torch.float32)
    ops.softmax_temperature(xd, torch.tensor([0.9], dtype=torch.float32, device="cuda"), out.t)
    want = oracle.c.softmax_temperature(x[1:].copy(), 0.9)
    assert np.abs(out.check() - want).max() < 1e-4
    L = _lib.lib()
    assert L.dtas_softmax_temperature_f32(None, None, None, 0, 9, None) == 0
    assert L.dtas_softmax_temperature_f32(None, None, None, 1, 9, None) == -1 and b"NULL" in L.dtas_last_error()
    assert L.dtas_softmax_temperature_f32(None, None, None, -1, 9, None) == -1 and b"negative" in L.dtas_last_error()
    with pytest.raises(ValueError):
        ops.softmax_temperature(xd, torch.tensor(0.9, dtype=torch.float16, device="cuda"), out.t)


@pytest.mark.parametrize("rows,cols", [(1, 50280), (3, 4096), (2, 50281), (300, 1000), (1, 128256), (2, 151936)])
def test_softmax_f32(oracle, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 4).astype(np.float32)
    out = Guarded(x.shape, torch.float32)
    ops.softmax_f32(dev(x), out.t)
    got = out.check().astype(np.float64)
    assert np.abs(got - oracle.c.softmax_f32(x, threads=8)).max() < 1e-2
    assert np.abs(got / oracle.np64.softmax(x) - 1).max() < 3e-5 and np.abs(got.sum(-1) - 1).max() < 1e-4
    # divide2 then softmax2 on the device against softmax_with_temperature on the device (the shared-row kernel sums
    # exp2((x - max) * log2e / t) in one, exp2((x / t - max) * log2e) in the other: last-place differences)
    t = torch.tensor(0.7, dtype=torch.float32, device="cuda")
    div, two, one = torch.empty_like(out.t), torch.empty_like(out.t), torch.empty_like(out.t)
    ops.divide(dev(x), t, div)
    ops.softmax_f32(div, two)
    ops.softmax_temperature(dev(x), t, one)
    assert float(((one - two).abs() / one.clamp_min(1e-30)).max()) < 1e-5


@pytest.mark.parametrize("n,H", [(1, 2560), (37, 2560), (4096, 2560), (5, 1024), (3, 4096), (7, 4100), (6, 777), (2, 10000),
                                 (600, 1024), (520, 4096), (513, 1028), (515, 8), (2049, 2564),   # from 512 rows: a wavefront per row
                                 (3, 5120), (700, 6144), (5, 8192), (600, 8192), (2, 8196)])       # rows of up to 8192 in registers
def test_layer_norm_f32(oracle, n, H):
    rng = np.random.default_rng(n + H)
    x = (rng.standard_normal((n, H)) * 2 + 0.5).astype(np.float32)
    g, b = rng.uniform(0.5, 1.5, H).astype(np.float32), rng.uniform(-1, 1, H).astype(np.float32)
    out = Guarded((n, H), torch.float32)
    ops.layer_norm_f32(dev(x), dev(g), dev(b), out.t)
    got = out.check()
    assert np.abs(got - oracle.c.layer_norm_f32(x, g, b, threads=8)).max() < 1e-2       # the stated tolerance
    assert np.abs(got - oracle.np64.layer_norm(x, g, b)).max() < 2e-5                    # what fp32 gives


def test_layer_norm_f32_unaligned_and_errors(oracle):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((3, 2560))).astype(np.float32)
    g, b = rng.uniform(0.5, 1.5, 2560).astype(np.float32), rng.uniform(-1, 1, 2560).astype(np.float32)
    raw = dev(np.concatenate([[0.0], x.ravel()]).astype(np.float32))
    out = Guarded((3, 2560), torch.float32)
    ops.layer_norm_f32(raw[1:].view(3, 2560), dev(g), dev(b), out.t)                       # 4-byte aligned rows: element accesses
    assert np.abs(out.check() - oracle.np64.layer_norm(x, g, b)).max() < 2e-5
    L = _lib.lib()
    assert L.dtas_layer_norm_f32(None, None, None, None, 0, 2560, 1e-5, None) == 0
    assert L.dtas_layer_norm_f32(None, None, None, None, 2, 2560, 1e-5, None) == -1 and b"NULL" in L.dtas_last_error()
    with pytest.raises(ValueError):
        ops.layer_norm_f32(dev(x), dev(g[:100]), dev(b), out.t)

"""GPU parity, elementwise add / copy / cast through the C ABI: bit-exact against the CPU oracle
on the same seeded inputs, every kernel variant, ragged sizes, odd alignment, guard bands."""
import numpy as np
import pytest
import torch

from dtas_amd import _lib, ops
from gpu_util import Guarded, assert_bits_equal, cfg, dev

pytestmark = pytest.mark.gpu

N_SWEEP = [1, 16, 128, 1024, 4096]
# beyond the sweep: the buckets above 4096, the table's upper bound 8192 and the last bucket's own sizing past it
N_BEYOND = [4097, 8192, 8193, 20000]
ALL_F16 = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)


@pytest.mark.parametrize("n", N_SWEEP)
def test_add_f16_benchmark_config(oracle, n):
    rng0, rng1 = np.random.default_rng(0), np.random.default_rng(1)
    a = rng0.uniform(-1, 1, (n, 4096)).astype(np.float16)
    b = rng1.uniform(-1, 1, (n, 4096)).astype(np.float16)
    out = Guarded(a.shape, torch.float16)
    ops.add(dev(a), dev(b), out.t)
    assert_bits_equal(out.check(), oracle.c.add(a, b, threads=8))


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.int8])
@pytest.mark.parametrize("n,H", [(1, 2560), (3, 2560), (257, 2560), (5, 2561), (1, 7), (2, 1)])
def test_add_reference_shapes_and_ragged(oracle, dtype, n, H):
    rng = np.random.default_rng(n * 131 + H)
    if dtype == np.int8:
        a = rng.integers(-128, 128, (1, n, H)).astype(np.int8)
        b = rng.integers(-128, 128, (1, n, H)).astype(np.int8)
    else:
        a = rng.uniform(-1, 1, (1, n, H)).astype(dtype)
        b = rng.uniform(-1, 1, (1, n, H)).astype(dtype)
    out = Guarded(a.shape, torch.from_numpy(a).dtype)
    ops.add(dev(a), dev(b), out.t)
    assert_bits_equal(out.check(), oracle.c.add(a, b))


def test_add_f16_special_values(oracle):
    sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504, -65504, 6e-8, -6e-8, 6.1e-5, 1, -1, 3e-5], dtype=np.float16)
    a, b = np.meshgrid(sp, sp)
    a, b = np.ascontiguousarray(a.ravel()[None]), np.ascontiguousarray(b.ravel()[None])
    out = Guarded(a.shape, torch.float16)
    ops.add(dev(a), dev(b), out.t)
    assert_bits_equal(out.check(), oracle.c.add(a, b), nan_ok=True)
    # every fp16 pattern plus a subnormal / a large value: subnormal results are kept, overflow goes to inf
    for other in (np.float16(6e-8), np.float16(60000), np.float16(-1.5)):
        a = ALL_F16.reshape(16, 4096)
        b = np.full_like(a, other)
        out = Guarded(a.shape, torch.float16)
        ops.add(dev(a), dev(b), out.t)
        assert_bits_equal(out.check(), oracle.c.add(a, b), nan_ok=True)


def test_add_i8_wraps_exhaustive(oracle):
    a, b = np.meshgrid(np.arange(-128, 128, dtype=np.int8), np.arange(-128, 128, dtype=np.int8))
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    out = Guarded(a.shape, torch.int8)
    ops.add(dev(a), dev(b), out.t)
    assert_bits_equal(out.check(), oracle.c.add(a, b))


@pytest.mark.parametrize("n", N_SWEEP)
def test_cast_f32_to_f16_benchmark_config(oracle, n):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((n, 4096)) * 100).astype(np.float32)
    out = Guarded(x.shape, torch.float16)
    ops.cast(dev(x), out.t)
    assert_bits_equal(out.check(), oracle.c.cast(x, "float16", threads=8))


def test_cast_f32_to_f16_rounding_overflow_subnormals(oracle):
    rng = np.random.default_rng(12)
    x = (rng.standard_normal((64, 4096)) * 1e5).astype(np.float32)          # overflow to +-inf
    tiny = (rng.standard_normal((64, 4096)) * 1e-6).astype(np.float32)      # fp16 subnormal results
    patterns = rng.integers(0, 2 ** 32, size=(64, 4096), dtype=np.uint64).astype(np.uint32).view(np.float32)
    edge = np.array([65504.0, 65519.99, 65520.0, -65520.0, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26,
                     1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, 2049.5, np.inf, -np.inf, np.nan, 0.0, -0.0], np.float32)[None]
    for src in (x, tiny, patterns, edge):
        out = Guarded(src.shape, torch.float16)
        ops.cast(dev(src), out.t)
        got = out.check()
        assert_bits_equal(got, oracle.c.cast(src, "float16"), nan_ok=True)
    assert np.isinf(oracle.c.cast(x, "float16")).any() and (oracle.c.cast(tiny, "float16") != 0).any()


def test_cast_f16_to_f32_all_patterns(oracle):
    h = ALL_F16.reshape(1, 16, 4096)
    out = Guarded(h.shape, torch.float32)
    ops.cast(dev(h), out.t)
    got = out.check()
    want = oracle.c.cast(h, "float32")
    assert_bits_equal(got, want, nan_ok=True)
    assert np.array_equal(got[~np.isnan(got)], h.astype(np.float32)[~np.isnan(got)])


@pytest.mark.parametrize("n", N_BEYOND)
def test_add_cast_copy_beyond_the_sweep(oracle, n):
    H = 4096 if n <= 8193 else 2560
    rng = np.random.default_rng(n)
    a, b = rng.uniform(-1, 1, (n, H)).astype(np.float16), rng.uniform(-1, 1, (n, H)).astype(np.float16)
    out = Guarded(a.shape, torch.float16)
    ops.add(dev(a), dev(b), out.t)
    assert_bits_equal(out.check(), oracle.c.add(a, b, threads=8))
    x = (rng.standard_normal((n, H)) * 100).astype(np.float32)
    out = Guarded(x.shape, torch.float16)
    ops.cast(dev(x), out.t)
    assert_bits_equal(out.check(), oracle.c.cast(x, "float16", threads=8), nan_ok=True)
    h = x.astype(np.float16)
    out32 = Guarded(h.shape, torch.float32)
    ops.cast(dev(h), out32.t)
    assert_bits_equal(out32.check(), oracle.c.cast(h, "float32", threads=8), nan_ok=True)
    outc = Guarded(h.shape, torch.float16)
    ops.copy(dev(h), outc.t)
    assert np.array_equal(outc.check().view(np.uint16), oracle.c.copy(h, threads=8).view(np.uint16))


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.int8])
@pytest.mark.parametrize("n", [1, 16, 128, 1024, 4096])
def test_copy_is_identity_on_bits(oracle, dtype, n):
    rng = np.random.default_rng(3)
    raw = rng.integers(0, 256, size=n * 4096 * np.dtype(dtype).itemsize, dtype=np.uint8)
    a = raw.view(dtype).reshape(n, 4096)  # arbitrary bit patterns: NaN payloads, subnormals
    out = Guarded(a.shape, torch.from_numpy(a).dtype)
    ops.copy(dev(a), out.t)
    got = out.check()
    assert np.array_equal(got.view(np.uint8), oracle.c.copy(a).view(np.uint8))


VARIANTS = [(op, vec, unroll) for op, vecs in (("add16", (8, 4, 2)), ("add32", (4, 2, 1)), ("add8", (16, 8, 4)),
                                               ("castdown", (8, 4, 2)), ("castup", (8, 4, 2)))
            for vec in vecs for unroll in (1, 2, 4, 8)]


@pytest.mark.parametrize("op,vec,unroll", VARIANTS)
def test_every_vector_variant(oracle, op, vec, unroll):
    rng = np.random.default_rng(vec * 10 + unroll)
    shape = (37, 2568)  # not a multiple of the largest tiles; divisible by 8 so every width is aligned
    c = cfg(variant=_lib.ELT_VECTOR, vec=vec, unroll=unroll)
    if op == "add16":
        a, b = rng.uniform(-1, 1, shape).astype(np.float16), rng.uniform(-1, 1, shape).astype(np.float16)
        out = Guarded(shape, torch.float16)
        ops.add(dev(a), dev(b), out.t, c)
        want = oracle.c.add(a, b)
    elif op == "add32":
        a, b = rng.uniform(-1, 1, shape).astype(np.float32), rng.uniform(-1, 1, shape).astype(np.float32)
        out = Guarded(shape, torch.float32)
        ops.add(dev(a), dev(b), out.t, c)
        want = oracle.c.add(a, b)
    elif op == "add8":
        a, b = rng.integers(-128, 128, shape).astype(np.int8), rng.integers(-128, 128, shape).astype(np.int8)
        out = Guarded(shape, torch.int8)
        ops.add(dev(a), dev(b), out.t, c)
        want = oracle.c.add(a, b)
    elif op == "castdown":
        a = (rng.standard_normal(shape) * 100).astype(np.float32)
        out = Guarded(shape, torch.float16)
        ops.cast(dev(a), out.t, c)
        want = oracle.c.cast(a, "float16")
    else:
        a = rng.standard_normal(shape).astype(np.float16)
        out = Guarded(shape, torch.float32)
        ops.cast(dev(a), out.t, c)
        want = oracle.c.cast(a, "float32")
    assert_bits_equal(out.check(), want)


def test_grid_cap_makes_the_kernel_loop(oracle):
    rng = np.random.default_rng(4)
    a, b = rng.uniform(-1, 1, (300, 4096)).astype(np.float16), rng.uniform(-1, 1, (300, 4096)).astype(np.float16)
    out = Guarded(a.shape, torch.float16)
    ops.add(dev(a), dev(b), out.t, cfg(vec=8, unroll=2, grid_cap=7))
    assert_bits_equal(out.check(), oracle.c.add(a, b))


def test_odd_alignment_steps_down_to_element_accesses(oracle):
    rng = np.random.default_rng(5)
    base_a, base_b = rng.uniform(-1, 1, 5000).astype(np.float16), rng.uniform(-1, 1, 5000).astype(np.float16)
    da, db = dev(base_a), dev(base_b)
    raw = torch.full((5100,), 9.0, dtype=torch.float16, device="cuda")
    ops.add(da[1:4998], db[1:4998], raw[3:5000])            # 2-byte aligned views
    got = raw.cpu().numpy()
    assert_bits_equal(got[3:5000], oracle.c.add(base_a[1:4998].copy(), base_b[1:4998].copy()))
    assert (got[:3] == 9).all() and (got[5000:] == 9).all()
    # an explicit vector config steps down the same way: a bucket's row must serve every buffer
    raw.fill_(9.0)
    ops.add(da[1:4998], db[1:4998], raw[3:5000], cfg(vec=8, unroll=4))
    got = raw.cpu().numpy()
    assert_bits_equal(got[3:5000], oracle.c.add(base_a[1:4998].copy(), base_b[1:4998].copy()))
    assert (got[:3] == 9).all() and (got[5000:] == 9).all()


def test_errors_on_the_gpu_path():
    a = torch.zeros(4, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match="overlaps"):
        ops.add(a, a, a)
    with pytest.raises(ValueError):
        ops.add(a, a, torch.zeros(4, 64, dtype=torch.float32, device="cuda"))
    ops.add(a[:0], a[:0], torch.zeros(0, 64, dtype=torch.float16, device="cuda"))  # empty extent: no-op


def test_full_size_properties():
    # n = 8192 (the top of the dynamic range): add is commutative and copy(copy(x)) == x, bit for bit
    g = torch.Generator(device="cuda").manual_seed(0)
    a = (torch.rand(8192, 4096, device="cuda", generator=g) * 2 - 1).half()
    b = (torch.rand(8192, 4096, device="cuda", generator=g) * 2 - 1).half()
    ab, ba, c1, c2 = (torch.empty_like(a) for _ in range(4))
    ops.add(a, b, ab)
    ops.add(b, a, ba)
    ops.copy(a, c1)
    ops.copy(c1, c2)
    torch.cuda.synchronize()
    assert torch.equal(ab.view(torch.int16), ba.view(torch.int16))
    assert torch.equal(c2.view(torch.int16), a.view(torch.int16))
    # x + 0 == x and widening then narrowing is the identity on fp16
    z, f32, back = torch.zeros_like(a), torch.empty(8192, 4096, device="cuda"), torch.empty_like(a)
    ops.add(a, z, ab)
    ops.cast(a, f32)
    ops.cast(f32, back)
    torch.cuda.synchronize()
    assert torch.equal(ab.view(torch.int16), a.view(torch.int16))
    assert torch.equal(back.view(torch.int16), a.view(torch.int16))
    # checksum of the sum against an independent fp64 accumulation on the device
    assert abs(ab.double().sum().item() - a.double().sum().item()) == 0


@pytest.mark.parametrize("V,H,n", [(50280, 2560, 1), (50280, 2560, 300), (50280, 2560, 4096), (9, 8, 33), (100, 20, 7)])
def test_take_is_bit_exact(oracle, V, H, n):
    # the fp16 embedding lookup (take / take1): rows of bit patterns, copied untouched
    rng = np.random.default_rng(V + n)
    a = rng.integers(0, 2 ** 16, (V, H), dtype=np.uint16).view(np.float16)
    ids = rng.integers(0, V, n).astype(np.int32)
    ids[0], ids[-1] = V - 1, 0
    out = Guarded((n, H), torch.float16)
    ops.take(dev(a), dev(ids), out.t)
    assert_bits_equal(out.check(), oracle.c.take(a, ids, threads=8))


def test_take_clips_ids_scalar_path_descriptor_and_errors(oracle):
    from dtas_amd import primfuncs as pf
    from dtas_amd.arch import MI355X
    from dtas_amd.engine.tuner import Engine

    rng = np.random.default_rng(2)
    a = rng.standard_normal((10, 64)).astype(np.float16)
    ids = np.array([-5, 0, 9, 10, 2 ** 31 - 1, -2 ** 31], np.int32)
    want = oracle.c.take(a, np.clip(ids, 0, 9).astype(np.int32))
    for vec in (8, 1):
        out = Guarded((6, 64), torch.float16)
        ops.take(dev(a), dev(ids), out.t, cfg(variant=_lib.ELT_VECTOR, block=256, vec=vec))
        assert_bits_equal(out.check(), want)
    buf = torch.empty(6 * 64 + 1, dtype=torch.float16, device="cuda")            # 2-byte aligned output: element path
    ops.take(dev(a), dev(ids), buf[1:].view(6, 64))
    torch.cuda.synchronize()
    assert_bits_equal(buf[1:].cpu().numpy().reshape(6, 64), want)
    funcs = [pf.take(10, 64), pf.take(10, 64, decode=True)]
    assert [f.name for f in funcs] == ["take", "take1"]
    rt = Engine(topk=2, parallel_build=False).tune_module(pf.module(*funcs, upper_bound={"n": 512}), MI355X())
    o = torch.empty(6, 64, dtype=torch.float16, device="cuda")
    rt["take"](dev(a), dev(np.clip(ids, 0, 9).astype(np.int32)), o)
    o1 = torch.empty(1, 64, dtype=torch.float16, device="cuda")
    rt["take1"](dev(a), dev(np.array([9], np.int32)), o1)
    torch.cuda.synchronize()
    assert_bits_equal(o.cpu().numpy(), want)
    assert_bits_equal(o1.cpu().numpy(), a[9:10])
    L = _lib.lib()
    assert L.dtas_take_f16(None, None, None, 0, 10, 64, None, None) == 0
    assert L.dtas_take_f16(None, None, None, 3, 10, 64, None, None) == -1 and b"NULL" in L.dtas_last_error()
    assert L.dtas_take_f16(None, None, None, 3, 0, 64, None, None) == -1 and b"empty table" in L.dtas_last_error()
    with pytest.raises(ValueError, match="int32 ids"):
        ops.take(dev(a), torch.zeros(6, dtype=torch.int64, device="cuda"), torch.empty(6, 64, dtype=torch.float16, device="cuda"))


@pytest.mark.parametrize("n,m,heads,d,rot", [(1, 1, 32, 80, 20), (1, 2048, 32, 80, 20), (300, 300, 32, 80, 20), (257, 4096, 32, 80, 20),
                                             (7, 9, 3, 64, 64), (5, 5, 2, 16, 0), (33, 40, 4, 128, 32),
                                             # rot = 20 with rows of 3, 4, 7, 64 and 65 pieces; one row; rows that end a chunk early
                                             (19, 4096, 5, 24, 20), (130, 130, 3, 32, 20), (41, 50, 7, 56, 20), (9, 9, 2, 512, 20),
                                             (3, 3, 2, 520, 20), (1, 7, 1, 80, 20), (4096, 4096, 32, 80, 20),
                                             # rotated widths in whole 16-byte pieces (a multiple of 16): all of d, half, a quarter; 16 itself
                                             (300, 4096, 32, 128, 128), (1, 77, 40, 128, 128), (513, 600, 64, 128, 64), (50, 50, 12, 64, 64),
                                             (77, 100, 8, 64, 32), (9, 4000, 3, 48, 16), (2049, 2049, 32, 128, 128), (31, 31, 5, 96, 48),
                                             # other widths stay with the kernel for any width
                                             # a multiple of 4 (partners and table entries in pairs); other even widths (the kernel for any width)
                                             (40, 64, 32, 96, 24), (6, 6, 2, 40, 36), (300, 4096, 64, 96, 24), (5, 5, 2, 16, 4), (9, 20, 3, 40, 12),
                                             (33, 33, 4, 32, 28), (4, 4, 2, 24, 18), (7, 8, 3, 16, 6), (3, 3, 1, 8, 2)])
def test_rotary_is_bit_exact(oracle, n, m, heads, d, rot):
    rng = np.random.default_rng(n + m + d)
    a = rng.standard_normal((1, n, heads, d)).astype(np.float16)
    ang = rng.uniform(0, 6.28, (4096, rot))
    cos, sin = np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)
    out = Guarded(a.shape, torch.float16)
    ops.rotary(dev(a), dev(cos), dev(sin), out.t, m)
    want = oracle.c.rotary(a, cos, sin, m, threads=8)
    assert_bits_equal(out.check(), want)
    for unroll in (1, 2):                      # a piece per thread; the kernel for any rotated width, also where the model's has its own
        out = Guarded(a.shape, torch.float16)
        ops.rotary(dev(a), dev(cos), dev(sin), out.t, m, cfg(variant=_lib.ELT_VECTOR, block=256, vec=8, unroll=unroll))
        assert_bits_equal(out.check(), want)


def test_rotary_errors():
    a = torch.zeros(1, 4, 2, 80, dtype=torch.float16, device="cuda")
    t = torch.zeros(16, 20, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match="outside the tables"):
        ops.rotary(a, t, t, torch.empty_like(a), 3)          # m < n
    with pytest.raises(_lib.DtasError, match="outside the tables"):
        ops.rotary(a, t, t, torch.empty_like(a), 17)         # m > max_pos
    with pytest.raises(_lib.DtasError, match="overlaps"):
        ops.rotary(a, t, t, a, 4)
    with pytest.raises(_lib.DtasError, match="must be even"):
        ops.rotary(a, torch.zeros(16, 21, dtype=torch.float16, device="cuda"), torch.zeros(16, 21, dtype=torch.float16, device="cuda"),
                   torch.empty_like(a), 4)


@pytest.mark.parametrize("n,m", [(1, 1), (1, 2049), (7, 7), (33, 77), (300, 1025), (1024, 1024), (2047, 2047)])
def test_attn_mask_is_exact(oracle, n, m):
    out = Guarded((1, 1, n, m), torch.float16)
    ops.attn_mask(out.t)
    assert_bits_equal(out.check().reshape(n, m), oracle.layout.attn_mask(n, m))


def test_attn_mask_beyond_32_bit_indices():
    # n * m >= 2^31: the 64-bit index path, checked on the device block of rows by block of rows (the property
    # out[i, j] == (j - (m - n) > i ? -65504 : 65504) itself, evaluated by torch)
    n, m = 32768, 65537
    out = torch.empty(n, m, dtype=torch.float16, device="cuda")
    ops.attn_mask(out.view(1, 1, n, m))
    j = torch.arange(m, device="cuda")[None, :]
    for lo in range(0, n, 4096):
        i = torch.arange(lo, lo + 4096, device="cuda")[:, None]
        want = torch.where(j - (m - n) > i, -65504.0, 65504.0).half()
        assert torch.equal(out[lo:lo + 4096], want), f"rows {lo}.."
    del out


@pytest.mark.parametrize("a,b,d", [(1, 32, 80), (300, 32, 80), (32, 300, 80), (4096, 32, 80), (5, 3, 8), (9, 17, 8), (13, 8, 512),
                                   (4, 5, 520), (8, 8, 80), (2, 2, 24)])
def test_swap_axes_is_exact(oracle, a, b, d):
    rng = np.random.default_rng(a + b)
    x = rng.integers(0, 2 ** 16, (1, a, b, d), dtype=np.uint16).view(np.float16)
    out = Guarded((1, b, a, d), torch.float16)
    ops.swap_axes(dev(x), out.t)
    assert_bits_equal(out.check(), oracle.layout.swap_axes(x))


def test_mask_and_swap_errors():
    L = _lib.lib()
    assert L.dtas_attn_mask_f16(None, 0, 5, None) == 0 and L.dtas_swap_axes_f16(None, None, 0, 3, 8, None) == 0
    assert L.dtas_attn_mask_f16(None, 5, 3, None) == -1 and b"at least n" in L.dtas_last_error()
    assert L.dtas_attn_mask_f16(None, 3, 5, None) == -1 and b"NULL" in L.dtas_last_error()
    assert L.dtas_swap_axes_f16(None, None, 2, 3, 7, None) == -1 and b"multiple of 8" in L.dtas_last_error()
    x = torch.zeros(2, 3, 8, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.DtasError, match="overlaps"):
        _lib.check(L.dtas_swap_axes_f16(x.data_ptr(), x.data_ptr(), 2, 3, 8, None), "swap")


@pytest.mark.parametrize("lead,d", [((1, 1, 32), 80), ((1, 300, 32), 80), ((1, 4096, 32), 80), ((7,), 3), ((33, 5), 12),
                                    ((37,), 512), ((3, 11), 520), ((65,), 8), ((32,), 16)])
def test_split3_is_exact(oracle, lead, d):
    rng = np.random.default_rng(d + len(lead))
    x = rng.integers(0, 2 ** 16, lead + (3 * d,), dtype=np.uint16).view(np.float16)
    outs = [Guarded(lead + (d,), torch.float16) for _ in range(3)]
    ops.split3(dev(x), *[o.t for o in outs])
    for o, want in zip(outs, oracle.layout.split3(x)):
        assert_bits_equal(o.check(), want)


def test_split3_misaligned_and_errors(oracle):
    rng = np.random.default_rng(9)
    x = rng.integers(0, 2 ** 16, (50, 240), dtype=np.uint16).view(np.float16)
    raw = torch.empty(50 * 240 + 1, dtype=torch.float16, device="cuda")
    xd = raw[1:].view(50, 240)                                               # 2-byte aligned: element accesses
    xd.copy_(dev(x))
    outs = [Guarded((50, 80), torch.float16) for _ in range(3)]
    ops.split3(xd, *[o.t for o in outs])
    for o, want in zip(outs, oracle.layout.split3(x)):
        assert_bits_equal(o.check(), want)
    L = _lib.lib()
    assert L.dtas_split3_f16(None, None, None, None, 0, 80, None) == 0
    assert L.dtas_split3_f16(None, None, None, None, 4, 80, None) == -1 and b"NULL" in L.dtas_last_error()
    o = outs[0].t
    with pytest.raises(_lib.DtasError, match="overlap"):
        _lib.check(L.dtas_split3_f16(xd.data_ptr(), o.data_ptr(), o.data_ptr(), outs[2].t.data_ptr(), 50, 80, None), "split3")
    with pytest.raises(ValueError):
        ops.split3(xd[:, :239], *[o.t for o in outs])


def test_swap_and_split_beyond_32_bit_indices():
    # 2^31 pieces and more: the 64-bit index instantiations, checked on the device against torch's own views
    a, b = 65536, 32768
    g = torch.Generator(device="cuda").manual_seed(3)
    A = torch.randint(-2 ** 15, 2 ** 15, (a, b, 8), dtype=torch.int16, device="cuda", generator=g).view(torch.float16)
    out = torch.empty(b, a, 8, dtype=torch.float16, device="cuda")
    ops.swap_axes(A, out)
    for lo in range(0, b, 4096):
        assert torch.equal(out[lo:lo + 4096].view(torch.int16), A[:, lo:lo + 4096].transpose(0, 1).view(torch.int16)), f"rows {lo}.."
    del A, out
    rows, d = 2 ** 20, 683                                                      # 3 * rows * d elements > 2^31, one element per access
    A = torch.randint(-2 ** 15, 2 ** 15, (rows, 3 * d), dtype=torch.int16, device="cuda", generator=g).view(torch.float16)
    outs = [torch.empty(rows, d, dtype=torch.float16, device="cuda") for _ in range(3)]
    ops.split3(A, *outs)
    for sec, o in enumerate(outs):
        assert torch.equal(o.view(torch.int16), A[:, sec * d:(sec + 1) * d].view(torch.int16)), f"section {sec}"


@pytest.mark.parametrize("count", [1, 3, 4, 1023, 50280, 50281, 1 << 22])
@pytest.mark.parametrize("b", [0.7, -3.0])
def test_divide_is_exact(oracle, count, b):
    rng = np.random.default_rng(count)
    a = (rng.standard_normal(count) * 10).astype(np.float32)
    special = np.array([0.0, np.inf, -np.inf, 1e-45, 3.4e38, -0.0, 1.0], np.float32)[:count]
    a[:special.size] = special
    out = Guarded((count,), torch.float32)
    ops.divide(dev(a), torch.tensor(b, dtype=torch.float32, device="cuda"), out.t)
    assert_bits_equal(out.check(), oracle.c.divide(a, b))
    if count > 8:                                                                # 4-byte alignment only: element accesses
        raw = dev(np.concatenate([[0.0], a]).astype(np.float32))
        out = Guarded((count,), torch.float32)
        ops.divide(raw[1:], torch.tensor([b], dtype=torch.float32, device="cuda"), out.t)
        assert_bits_equal(out.check(), oracle.c.divide(a, b))


def test_divide_errors():
    L = _lib.lib()
    assert L.dtas_divide_f32(None, None, None, 0, None) == 0
    assert L.dtas_divide_f32(None, None, None, 5, None) == -1 and b"NULL" in L.dtas_last_error()
    assert L.dtas_divide_f32(None, None, None, -5, None) == -1 and b"negative" in L.dtas_last_error()
    x = torch.zeros(8, dtype=torch.float32, device="cuda")
    with pytest.raises(_lib.DtasError, match="overlaps"):
        _lib.check(L.dtas_divide_f32(x.data_ptr(), x.data_ptr() + 16, x.data_ptr(), 4, None), "divide")

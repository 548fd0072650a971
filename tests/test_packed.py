"""libdtas_packed.so: the reference's host signature -- int32_t f(TVMValue* args, int* type_codes, int num_args,
...) over DLTensor handles (experiment/dtas_tuned/elementwise/add/float16/top1_256/host.cc:38-63) -- in front of the
C ABI.  Host logic on fake tensors here (no kernel is launched); the GPU tests call through it for real."""
import ctypes
import os
import re

import numpy as np
import pytest

from dtas_amd import _packed as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = 0x7f0000000000  # never dereferenced: every call below fails, or is empty, before a launch


def _t(shape, dtype="float16", **kw):
    return P.make_tensor(kw.pop("ptr", FAKE), shape, dtype, **kw)


def _past_the_shim(msg: str) -> bool:
    """The call got through the shim's own checks: on a machine without a GPU making the device current fails,
    with one the C ABI's own argument check answers (the two buffers are the same fake memory)."""
    return "hipSetDevice" in msg or "overlaps" in msg


def test_packed_library_exports_what_its_header_declares():
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "dtas_packed.h")).read(), flags=re.S)
    declared = set(re.findall(r"int32_t\s+(\w+)\s*\(void\* args", header))
    assert declared == set(P.FUNCTIONS)
    h = ctypes.CDLL(P.PACKED_PATH)
    for name in list(declared) + ["dtas_packed_set_stream", "dtas_packed_last_error", "__tvm_module_ctx"]:
        assert hasattr(h, name), name
    assert ctypes.sizeof(P.DLTensor) == 48 and ctypes.sizeof(P.TVMValue) == 8


def test_argument_count_and_handle_kinds():
    a, b, c = _t((1, 4, 64)), _t((1, 4, 64)), _t((1, 4, 64))
    assert P.call("add", [a, b]) == -1 and "takes 3 buffers, got 2" in P.last_error()
    assert P.call("add", [a, b, c], codes=[7, P.TCODE_NULLPTR, 7]) == -1 and "argument 1 is a null handle" in P.last_error()
    assert P.call("add", [a, None, c]) == -1 and "null handle" in P.last_error()
    assert P.call("add", [a, b, c], codes=[7, 7, 0]) == -1 and "type code 0" in P.last_error()      # an int, not a handle
    assert P.call("copy", [a, b], codes=[P.TCODE_NDARRAY_HANDLE, P.TCODE_OPAQUE_HANDLE]) == -1      # both kinds accepted ...
    assert _past_the_shim(P.last_error())                                                            # ... what fails comes after the shim's checks


def test_element_types_select_the_entry_point_or_fail():
    assert P.call("add", [_t((1, 4, 64), "float16"), _t((1, 4, 64), "float32"), _t((1, 4, 64), "float16")]) == -1
    assert "share one of float16, float32, int8" in P.last_error()
    assert P.call("add", [_t((1, 4, 64), "float64")] * 3) == -1 and "unsupported" in P.last_error()
    assert P.call("cast", [_t((1, 4, 64), "float16"), _t((1, 4, 64), "float16", ptr=FAKE + (1 << 20))]) == -1
    assert "float16 -> float32 or float32 -> float16" in P.last_error()
    assert P.call("fused_layer_norm_cast1", [_t((1, 4, 64), "float16"), _t((64,), "float32"), _t((64,), "float32"), _t((1, 4, 64))]) == -1
    assert "float32 gamma" in P.last_error()
    assert P.call("fused_NT_matmul4_add1", [_t((1, 4, 64)), _t((32, 64), "float32"), _t((32,)), _t((1, 4, 32))]) == -1
    assert "argument 1 is float32" in P.last_error()


def test_shapes_and_strides():
    assert P.call("add", [_t((1, 4, 64)), _t((1, 4, 64)), _t((1, 5, 64))]) == -1 and "one shape" in P.last_error()
    strided = _t((1, 4, 64), strides=(512, 128, 1))
    assert P.call("copy", [strided, _t((1, 4, 64))]) == -1 and "not compact" in P.last_error()
    compact = _t((1, 4, 64), strides=(256, 64, 1))
    assert P.call("copy", [compact, compact]) == -1 and _past_the_shim(P.last_error())
    assert P.call("fused_NT_matmul4_add1", [_t((1, 4, 64)), _t((32, 48)), _t((32,)), _t((1, 4, 32))]) == -1
    assert "lv is (1, n, K)" in P.last_error()
    assert P.call("fused_NT_matmul10_add5", [_t((1, 2, 64)), _t((32, 64)), _t((32,)), _t((1, 2, 32))]) == -1
    assert "takes one row" in P.last_error()
    assert P.call("fused_layer_norm_cast1", [_t((1, 4, 64), "float32"), _t((32,), "float32"), _t((64,), "float32"), _t((1, 4, 64))]) == -1
    assert P.call("add", [_t((1, 4, 64), device_type=1)] * 3) == -1 and "not on a GPU" in P.last_error()      # kDLCPU
    assert P.call("add", [_t((1, 4, 64)), _t((1, 4, 64), device_id=1), _t((1, 4, 64))]) == -1 and "on device 1" in P.last_error()


def test_fused_attention_and_q8_functions_check_their_arguments():
    f16 = lambda *shape, **kw: _t(shape, "float16", **kw)
    # the fused-epilogue GEMMs: argument count by kind, element types, shapes
    assert P.call("fused_NT_matmul2_add1_add3_add3", [f16(1, 4, 64), f16(32, 64), f16(32), f16(1, 4, 32)]) == -1
    assert "takes 6 buffers, got 4" in P.last_error()
    six = [f16(1, 4, 64), f16(32, 64), f16(32), f16(1, 4, 32), f16(1, 4, 32), f16(1, 4, 32)]
    assert P.call("fused_NT_matmul2_add1_add3_add3_cast", six) == -1 and "the output is float32" in P.last_error()
    assert P.call("fused_NT_matmul8_add5_add7_add7", six[:3] + [f16(1, 4, 32), f16(1, 5, 32), f16(1, 4, 32)]) == -1
    assert "both residuals are (1, n, N)" in P.last_error()
    assert P.call("fused_NT_matmul3_add2_gelu", [f16(1, 4, 64), f16(32, 48), f16(32), f16(1, 4, 32)]) == -1 and "lv is (1, n, K)" in P.last_error()
    assert P.call("fused_NT_matmul9_add6_gelu1", [f16(1, 4, 64), _t((32, 64), "float32"), f16(32), f16(1, 4, 32)]) == -1
    assert "argument 1 is float32" in P.last_error()
    assert P.call("fused_NT_matmul2_add1_add3_add3", six) == -1 and _past_the_shim(P.last_error())
    # scores: (q, k, mask, out float32), four axes each
    q, k, mask = f16(1, 2, 5, 80), f16(1, 2, 7, 80), f16(1, 1, 5, 7)
    assert P.call("fused_NT_matmul1_divide_maximum_minimum_cast2", [q, k, mask, f16(1, 2, 5, 7)]) == -1 and "the output is float32" in P.last_error()
    out = _t((1, 2, 5, 7), "float32")
    assert P.call("fused_NT_matmul1_divide_maximum_minimum_cast2", [q, k, f16(1, 1, 5, 8), out]) == -1 and "the mask (1, 1, n, m)" in P.last_error()
    assert P.call("fused_NT_matmul7_divide1_maximum1_minimum1_cast7", [q, f16(1, 3, 7, 80), mask, out]) == -1
    assert P.call("fused_NT_matmul7_divide2_maximum1_minimum1_cast7", [f16(2, 5, 80), k, mask, out]) == -1 and "(1, heads, rows, columns)" in P.last_error()
    assert P.call("fused_NT_matmul1_divide1_maximum_minimum_cast2", [q, k, mask, out]) == -1 and _past_the_shim(P.last_error())
    # P.V: (A (1, H, n, m), B (1, H, m, d), out (1, H, n, d))
    assert P.call("matmul8", [f16(1, 2, 5, 7), f16(1, 2, 8, 80), f16(1, 2, 5, 80)]) == -1 and "B (1, H, m, d)" in P.last_error()
    assert P.call("matmul10", [f16(1, 2, 1, 7), f16(1, 2, 7, 80)]) == -1 and "takes 3 buffers" in P.last_error()
    assert P.call("matmul9", [f16(1, 2, 5, 7), f16(1, 2, 7, 80), f16(1, 2, 5, 80)]) == -1 and _past_the_shim(P.last_error())
    # 8-bit weights: (Wq uint32 (N, K/4), scale (N, K/32), lv (1, n, K), bias (N), out (1, n, N))
    wq, sc = _t((32, 16), "uint32"), f16(32, 2)
    assert P.call("fused_fused_decode2_fused_NT_matmul_add", [_t((32, 16), "int32"), sc, f16(1, 1, 64), f16(32), f16(1, 1, 32)]) == -1
    assert "packed weights are uint32" in P.last_error()
    assert P.call("fused_fused_decode2_fused_NT_matmul6_add4", [wq, f16(32, 4), f16(1, 4, 64), f16(32), f16(1, 4, 32)]) == -1
    assert "the scales (N, K/32)" in P.last_error()
    assert P.call("fused_fused_decode4_fused_NT_matmul3_add2_gelu", [wq, sc, f16(1, 1, 48), f16(32), f16(1, 1, 32)]) == -1
    assert P.call("fused_fused_decode5_fused_NT_matmul10_add5", [wq, sc, f16(1, 4, 64), f16(32), f16(1, 4, 32)]) == -1 and _past_the_shim(P.last_error())
    # empty extents need no device
    z = lambda *shape, dt="float16": _t(shape, dt, ptr=0)
    assert P.call("fused_NT_matmul3_add2_gelu", [z(1, 0, 64), f16(32, 64), f16(32), z(1, 0, 32)]) == 0
    assert P.call("matmul8", [z(1, 2, 0, 7), f16(1, 2, 7, 80), z(1, 2, 0, 80)]) == 0
    assert P.call("fused_NT_matmul1_divide_maximum_minimum_cast2", [z(1, 2, 0, 80), k, z(1, 1, 0, 7), z(1, 2, 0, 7, dt="float32")]) == 0


def test_an_empty_extent_is_a_successful_no_op():
    # n = shape[1] = 0: nothing to launch, no device needed (as the C ABI's n == 0)
    z = lambda dt="float16": _t((1, 0, 64), dt, ptr=0)
    assert P.call("add", [z(), z(), z()]) == 0
    assert P.call("cast", [z("float32"), z("float16")]) == 0
    assert P.call("fused_softmax_cast", [_t((1, 32, 0, 0), "float32", ptr=0), _t((1, 32, 0, 0), ptr=0)]) == 0


def test_header_is_plain_c(tmp_path):
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("needs gcc")
    src = tmp_path / "c.c"
    src.write_text('#include "dtas_packed.h"\nint main(void) { DLTensor t; TVMValue v; v.v_handle = &t; (void)v; return sizeof(DLTensor) == 48 ? 0 : 1; }\n')
    exe = tmp_path / "c"
    subprocess.check_call([gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    assert subprocess.run([str(exe)]).returncode == 0


@pytest.mark.gpu
def test_packed_calls_compute_what_the_c_abi_computes(oracle):
    import torch
    from gpu_util import Guarded, assert_bits_equal, dev

    rng = np.random.default_rng(21)
    n, H = 37, 2560
    dt = lambda t, shape, dtype: P.make_tensor(t.data_ptr(), shape, dtype, device_id=t.device.index or 0)
    # add, float16 and int8
    a, b = rng.uniform(-1, 1, (1, n, H)).astype(np.float16), rng.uniform(-1, 1, (1, n, H)).astype(np.float16)
    da, db, out = dev(a), dev(b), Guarded((1, n, H), torch.float16)
    assert P.call("add", [dt(da, a.shape, "float16"), dt(db, b.shape, "float16"), dt(out.t, a.shape, "float16")]) == 0, P.last_error()
    assert_bits_equal(out.check(), oracle.c.add(a, b))
    ai, bi = rng.integers(-128, 128, (1, n, H), dtype=np.int8), rng.integers(-128, 128, (1, n, H), dtype=np.int8)
    dai, dbi, outi = dev(ai), dev(bi), Guarded((1, n, H), torch.int8)
    assert P.call("add", [dt(dai, ai.shape, "int8"), dt(dbi, bi.shape, "int8"), dt(outi.t, ai.shape, "int8")]) == 0, P.last_error()
    assert np.array_equal(outi.check(), oracle.c.add(ai, bi))
    # cast float16 -> float32 (the reference's direction) with the type code of an NDArray handle, on a side stream
    x = (rng.standard_normal((1, n, H)) * 100).astype(np.float16)
    dx, outf = dev(x), Guarded((1, n, H), torch.float32)
    st = torch.cuda.Stream()
    st.wait_stream(torch.cuda.current_stream())
    P.lib().dtas_packed_set_stream(st.cuda_stream)
    try:
        assert P.call("cast", [dt(dx, x.shape, "float16"), dt(outf.t, x.shape, "float32")], codes=[13, 13]) == 0, P.last_error()
    finally:
        P.lib().dtas_packed_set_stream(None)
    st.synchronize()
    assert_bits_equal(outf.check(), oracle.c.cast(x, "float32"), nan_ok=True)
    # layer norm and softmax in the reference's shapes
    xf = rng.standard_normal((1, n, H)).astype(np.float32)
    gm, bt = rng.uniform(0.5, 1.5, H).astype(np.float32), rng.uniform(-1, 1, H).astype(np.float32)
    dxf, dg, dbt, outn = dev(xf), dev(gm), dev(bt), Guarded((1, n, H), torch.float16)
    assert P.call("fused_layer_norm_cast1", [dt(dxf, xf.shape, "float32"), dt(dg, gm.shape, "float32"), dt(dbt, bt.shape, "float32"),
                                             dt(outn.t, xf.shape, "float16")]) == 0, P.last_error()
    want = oracle.c.layer_norm(xf.reshape(n, H), gm, bt).reshape(1, n, H)
    assert np.abs(outn.check().astype(np.float32) - want.astype(np.float32)).max() <= 2e-3 * max(1.0, float(np.abs(want).max()))
    s = (rng.standard_normal((1, 32, 5, 77)) * 2).astype(np.float32)
    ds, outs = dev(s), Guarded(s.shape, torch.float16)
    assert P.call("fused_softmax_cast", [dt(ds, s.shape, "float32"), dt(outs.t, s.shape, "float16")]) == 0, P.last_error()
    assert np.abs(outs.check().astype(np.float32) - oracle.c.softmax(s.reshape(160, 77)).reshape(s.shape).astype(np.float32)).max() <= 1e-3
    # the two matmuls
    K, N = 256, 200
    lv, w, bias = rng.standard_normal((1, n, K)).astype(np.float16), (rng.standard_normal((N, K)) * 0.05).astype(np.float16), rng.uniform(-1, 1, N).astype(np.float16)
    dlv, dw, dbias, outm = dev(lv), dev(w), dev(bias), Guarded((1, n, N), torch.float16)
    assert P.call("fused_NT_matmul4_add1", [dt(dlv, lv.shape, "float16"), dt(dw, w.shape, "float16"), dt(dbias, bias.shape, "float16"),
                                            dt(outm.t, (1, n, N), "float16")]) == 0, P.last_error()
    ref = oracle.c.gemm(lv.reshape(n, K), w, bias).reshape(1, n, N).astype(np.float32)
    assert np.abs(outm.check().astype(np.float32) - ref).max() <= 2e-2
    row, outv = dev(lv[:, :1]), Guarded((1, 1, N), torch.float16)
    assert P.call("fused_NT_matmul10_add5", [dt(row, (1, 1, K), "float16"), dt(dw, w.shape, "float16"), dt(dbias, bias.shape, "float16"),
                                             dt(outv.t, (1, 1, N), "float16")]) == 0, P.last_error()
    assert np.abs(outv.check().astype(np.float32) - ref[:, :1]).max() <= 2e-2


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 37])
def test_packed_fused_attention_and_q8_calls_against_the_oracle(oracle, n):
    """One call of every PrimFunc family added for the model graph, prefill (n = 37) and decode (n = 1) names, through the
    PackedFunc signature in the parameter order of its TVMScript, against the oracle."""
    import torch
    from gpu_util import Guarded, dev

    rng = np.random.default_rng(100 + n)
    dt = lambda t, shape, dtype: P.make_tensor(t.data_ptr(), shape, dtype, device_id=t.device.index or 0)
    f16 = lambda *shape, s=1.0: (rng.standard_normal(shape) * s).astype(np.float16)
    K, N = 256, 320
    lv, w, bias = f16(1, n, K), f16(N, K, s=0.05), rng.uniform(-1, 1, N).astype(np.float16)
    r1, r2 = f16(1, n, N), f16(1, n, N)
    dlv, dw, dbias, dr1, dr2 = dev(lv), dev(w), dev(bias), dev(r1), dev(r2)
    common = [dt(dlv, lv.shape, "float16"), dt(dw, w.shape, "float16"), dt(dbias, bias.shape, "float16")]
    res = [dt(dr1, r1.shape, "float16"), dt(dr2, r2.shape, "float16")]

    def close(got, want, ulps=2):
        g, wv = got.astype(np.float64), want.astype(np.float64)
        assert np.isfinite(g).all()
        assert (np.abs(g - wv) <= 1e-3 + ulps * 2.0 ** -10 * np.abs(wv)).all(), float(np.abs(g - wv).max())

    add_names = ("fused_NT_matmul2_add1_add3_add3", "fused_NT_matmul8_add5_add7_add7")
    for name in add_names:
        out = Guarded((1, n, N), torch.float16)
        assert P.call(name, common + res + [dt(out.t, (1, n, N), "float16")]) == 0, P.last_error()
        close(out.check(), oracle.c.gemm_fused(lv.reshape(n, K), w, bias, r1.reshape(n, N), r2.reshape(n, N), 1).reshape(1, n, N))
    for name in ("fused_NT_matmul2_add1_add3_add3_cast", "fused_NT_matmul8_add5_add7_add7_cast5"):
        out = Guarded((1, n, N), torch.float32)
        assert P.call(name, common + res + [dt(out.t, (1, n, N), "float32")]) == 0, P.last_error()
        close(out.check(), oracle.c.gemm_fused(lv.reshape(n, K), w, bias, r1.reshape(n, N), r2.reshape(n, N), 2).reshape(1, n, N))
    for name in ("fused_NT_matmul3_add2_gelu", "fused_NT_matmul9_add6_gelu1"):
        out = Guarded((1, n, N), torch.float16)
        assert P.call(name, common + [dt(out.t, (1, n, N), "float16")]) == 0, P.last_error()
        close(out.check(), oracle.c.gemm_fused(lv.reshape(n, K), w, bias, None, None, 3).reshape(1, n, N), ulps=3)
    out = Guarded((1, n, N), torch.float16)
    assert P.call("fused_NT_matmul_add", common + [dt(out.t, (1, n, N), "float16")]) == 0, P.last_error()
    close(out.check(), oracle.c.gemm(lv.reshape(n, K), w, bias).reshape(1, n, N))

    # attention: 4 heads of 80, m keys
    H, d, m = 4, 80, 45
    q, k, v = f16(1, H, n, d), f16(1, H, m, d), f16(1, H, m, d)
    mask = np.where(rng.random((1, 1, n, m)) < 0.7, 65504.0, -65504.0).astype(np.float16)
    dq, dk, dv, dmask = dev(q), dev(k), dev(v), dev(mask)
    want = oracle.c.attn_scores(q[0], k[0], mask[0, 0], 0.11179039301310044)
    for name in ("fused_NT_matmul1_divide_maximum_minimum_cast2", "fused_NT_matmul7_divide1_maximum1_minimum1_cast7",
                 "fused_NT_matmul1_divide1_maximum_minimum_cast2", "fused_NT_matmul7_divide2_maximum1_minimum1_cast7"):
        out = Guarded((1, H, n, m), torch.float32)
        assert P.call(name, [dt(dq, q.shape, "float16"), dt(dk, k.shape, "float16"), dt(dmask, mask.shape, "float16"),
                             dt(out.t, (1, H, n, m), "float32")]) == 0, P.last_error()
        got = out.check()[0]
        assert (np.abs(got.astype(np.float64) - want) <= 1e-3 + 2.0 ** -9 * np.abs(want)).all()
    p = rng.random((1, H, n, m)).astype(np.float32)
    p = (p / p.sum(-1, keepdims=True)).astype(np.float16)
    dp = dev(p)
    wantv = oracle.c.attn_pv(p[0], v[0])
    for name in ("matmul8", "matmul10", "matmul9", "matmul1"):
        out = Guarded((1, H, n, d), torch.float16)
        assert P.call(name, [dt(dp, p.shape, "float16"), dt(dv, v.shape, "float16"), dt(out.t, (1, H, n, d), "float16")]) == 0, P.last_error()
        close(out.check()[0], wantv)

    # 8-bit weights
    wq = rng.integers(0, 2 ** 32, (N, K // 4), dtype=np.uint64).astype(np.uint32)
    sc = rng.uniform(0.001, 0.02, (N, K // 32)).astype(np.float16)
    dwq, dsc = torch.from_numpy(wq.view(np.int32)).cuda(), dev(sc)
    wdec = oracle.c.decode_q8(wq, sc)
    q8 = [dt(dwq, wq.shape, "uint32"), dt(dsc, sc.shape, "float16"), dt(dlv, lv.shape, "float16"), dt(dbias, bias.shape, "float16")]
    for name, kind in (("fused_fused_decode2_fused_NT_matmul_add", 0), ("fused_fused_decode2_fused_NT_matmul6_add4", 0),
                       ("fused_fused_decode5_fused_NT_matmul4_add1", 0), ("fused_fused_decode5_fused_NT_matmul10_add5", 0),
                       ("fused_fused_decode4_fused_NT_matmul3_add2_gelu", 3), ("fused_fused_decode4_fused_NT_matmul9_add6_gelu1", 3)):
        out = Guarded((1, n, N), torch.float16)
        assert P.call(name, q8 + [dt(out.t, (1, n, N), "float16")]) == 0, P.last_error()
        close(out.check(), oracle.c.gemm_fused(lv.reshape(n, K), wdec, bias, None, None, kind).reshape(1, n, N), ulps=3)

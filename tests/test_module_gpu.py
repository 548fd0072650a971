"""End-to-end on the GPU through the reference's Python entry points: Engine.tune_module with
on-device timing of the candidates, the runtime module's dispatch, load_module_from_file."""
import numpy as np
import pytest
import torch

from dtas_amd import _lib, primfuncs as pf
from dtas_amd.arch import MI355X
from dtas_amd.codegen.runtime_packer import load_module_from_file
from dtas_amd.engine.tuner import Engine

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tuned(tmp_path_factory):
    work_dir = str(tmp_path_factory.mktemp("tuned"))
    mod = pf.module(pf.add("float16", 4096), pf.cast("float32", "float16", 4096), pf.rms_norm(4096),
                    pf.softmax_scores(32), pf.fused_layer_norm_cast1(2560),
                    pf.fused_NT_matmul_add_gemv(4096, 4096, bias=True), pf.fused_NT_matmul_add_gemm(4096, 4096, bias=True),
                    pf.fused_NT_matmul_add_add_add(2560, 2560), pf.fused_NT_matmul_add_add_add(2560, 2560, cast=True),
                    pf.fused_NT_matmul_add_gelu(2560, 2560), upper_bound={"n": 1024})
    eng = Engine(topk=4, parallel_build=True, work_dir=work_dir)
    rt = eng.tune_module(mod, arch=MI355X(0, require_device=True), range_div_factor=256)
    return rt, work_dir


def test_candidates_were_timed_on_the_device(tuned):
    import json, os

    _, work_dir = tuned
    records = json.load(open(os.path.join(work_dir, "data_base", "best_record.json")))
    timed = [v["latency(ms)"] for rec in records for v in rec.values() if v["latency(ms)"] is not None]
    assert timed and all(0 < t < 1000 for t in timed)


@pytest.mark.parametrize("n", [1, 255, 256, 300, 1024, 2000])
def test_module_functions_match_the_oracle(tuned, oracle, n):
    rt, work_dir = tuned
    again = load_module_from_file(work_dir)
    rng = np.random.default_rng(n)
    for mod in (rt, again):
        a = rng.uniform(-1, 1, (1, n, 4096)).astype(np.float16)
        b = rng.uniform(-1, 1, (1, n, 4096)).astype(np.float16)
        out = torch.empty(1, n, 4096, dtype=torch.float16, device="cuda")
        mod["add"](torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), out)
        assert np.array_equal(out.cpu().numpy().view(np.uint16), oracle.c.add(a, b).view(np.uint16))

        x32 = (rng.standard_normal((1, n, 4096)) * 100).astype(np.float32)
        mod["cast"](torch.from_numpy(x32).cuda(), out)
        assert np.array_equal(out.cpu().numpy().view(np.uint16), oracle.c.cast(x32, "float16").view(np.uint16))

        x = rng.standard_normal((n, 4096)).astype(np.float16)
        w = rng.uniform(0.5, 1.5, 4096).astype(np.float16)
        o2 = torch.empty(n, 4096, dtype=torch.float16, device="cuda")
        mod["rms_norm"](torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), o2)
        assert np.abs(o2.cpu().numpy().astype(np.float64) - oracle.np64.rms_norm(x, w)).max() < 1e-2


def test_gemm_gemv_and_softmax_through_the_module(tuned, oracle):
    rt, _ = tuned
    rng = np.random.default_rng(0)
    W = (rng.standard_normal((4096, 4096)) * 0.02).astype(np.float16)
    bias = rng.uniform(-1, 1, 4096).astype(np.float16)
    for n in (3, 130, 700):
        A = rng.standard_normal((1, n, 4096)).astype(np.float16)
        C = torch.empty(1, n, 4096, dtype=torch.float16, device="cuda")
        rt["fused_NT_matmul4_add1"](torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda(), torch.from_numpy(bias).cuda(), C)
        want = oracle.np64.gemm(A[0], W, bias)
        assert (np.abs(C.cpu().numpy()[0].astype(np.float64) - want) <= 2e-3 + 1e-2 * np.abs(want)).all()
    x = rng.standard_normal((1, 1, 4096)).astype(np.float16)
    y = torch.empty(1, 1, 4096, dtype=torch.float16, device="cuda")
    rt["fused_NT_matmul10_add5"](torch.from_numpy(x).cuda(), torch.from_numpy(W).cuda(), torch.from_numpy(bias).cuda(), y)
    want = oracle.np64.gemm(x[0], W, bias)
    assert (np.abs(y.cpu().numpy()[0].astype(np.float64) - want) <= 2e-3 + 1e-2 * np.abs(want)).all()
    for n in (5, 64, 257):
        s = (rng.standard_normal((32, n, n)) * 2).astype(np.float16)
        so = torch.empty(32, n, n, dtype=torch.float16, device="cuda")
        rt["softmax_scores"](torch.from_numpy(s).cuda(), so)
        assert np.abs(so.cpu().numpy().astype(np.float64) - oracle.np64.softmax(s)).max() < 1e-2


def test_time_evaluator_and_signature_errors(tuned):
    rt, _ = tuned
    a = torch.zeros(1, 64, 4096, dtype=torch.float16, device="cuda")
    out = torch.empty_like(a)
    res = rt.time_evaluator("add", number=5, min_repeat_ms=5)(a, a.clone(), out)
    assert 0 < res.mean < 1e-2
    with pytest.raises(TypeError):
        rt["add"](a, a)
    with pytest.raises(ValueError):
        rt["add"](a, a.clone(), torch.empty(1, 64, 2560, dtype=torch.float16, device="cuda"))
    with pytest.raises(_lib.DtasError, match="overlaps"):
        rt["add"](a, a, a)


def test_fused_epilogues_through_the_module(tuned, oracle):
    rt, work_dir = tuned
    again = load_module_from_file(work_dir)
    rng = np.random.default_rng(4)
    W = (rng.standard_normal((2560, 2560)) * 0.02).astype(np.float16)
    bias = rng.uniform(-1, 1, 2560).astype(np.float16)
    t = lambda a: torch.from_numpy(a).cuda()
    for mod in (rt, again):
        for n in (2, 300):
            A = rng.standard_normal((1, n, 2560)).astype(np.float16)
            r1 = rng.standard_normal((1, n, 2560)).astype(np.float16)
            r2 = rng.standard_normal((1, n, 2560)).astype(np.float16)
            out = torch.empty(1, n, 2560, dtype=torch.float16, device="cuda")
            mod["fused_NT_matmul2_add1_add3_add3"](t(A), t(W), t(bias), t(r1), t(r2), out)
            want = oracle.np64.gemm_fused(A[0], W, bias, r1[0], r2[0], 1)
            scale = np.maximum(np.abs(want), np.maximum(np.abs(r1[0]), np.abs(r2[0])).astype(np.float64))
            assert (np.abs(out.cpu().numpy()[0].astype(np.float64) - want) <= 4e-3 + 1e-2 * scale).all()
            out32 = torch.empty(1, n, 2560, dtype=torch.float32, device="cuda")
            mod["fused_NT_matmul2_add1_add3_add3_cast"](t(A), t(W), t(bias), t(r1), t(r2), out32)
            assert torch.equal(out32, out.float())
            mod["fused_NT_matmul3_add2_gelu"](t(A), t(W), t(bias), out)
            want = oracle.np64.gemm_fused(A[0], W, bias, None, None, 3)
            assert (np.abs(out.cpu().numpy()[0].astype(np.float64) - want) <= 4e-3 + 1e-2 * np.abs(want)).all()


def test_decode_forms_of_the_fused_matmuls_go_through_the_gemv_rule(tmp_path, oracle):
    """fused_NT_matmul8_add5_add7_add7(_cast5) and fused_NT_matmul9_add6_gelu1: one static row, tuned as GEMVs."""
    from dtas_amd.common.analisys import FuncInfo, FuncKind

    funcs = [pf.fused_NT_matmul_add_add_add(2560, 2560, decode=True), pf.fused_NT_matmul_add_add_add(2560, 2560, cast=True, decode=True),
             pf.fused_NT_matmul_add_gelu(10240, 2560, decode=True)]
    assert [f.name for f in funcs] == ["fused_NT_matmul8_add5_add7_add7", "fused_NT_matmul8_add5_add7_add7_cast5",
                                       "fused_NT_matmul9_add6_gelu1"]
    assert all(FuncInfo(f).kind == FuncKind.kFunc_GEMV for f in funcs)
    work_dir = str(tmp_path / "decode")
    rt = Engine(topk=3, parallel_build=False, work_dir=work_dir).tune_module(pf.module(*funcs), arch=MI355X(0, require_device=True))
    rng = np.random.default_rng(9)
    t = lambda a: torch.from_numpy(a).cuda()
    x = rng.standard_normal((1, 1, 2560)).astype(np.float16)
    W = (rng.standard_normal((2560, 2560)) * 0.02).astype(np.float16)
    W2 = (rng.standard_normal((10240, 2560)) * 0.02).astype(np.float16)
    bias, bias2 = rng.uniform(-1, 1, 2560).astype(np.float16), rng.uniform(-1, 1, 10240).astype(np.float16)
    r1, r2 = rng.standard_normal((1, 1, 2560)).astype(np.float16), rng.standard_normal((1, 1, 2560)).astype(np.float16)
    for mod in (rt, load_module_from_file(work_dir)):
        out = torch.empty(1, 1, 2560, dtype=torch.float16, device="cuda")
        mod["fused_NT_matmul8_add5_add7_add7"](t(x), t(W), t(bias), t(r1), t(r2), out)
        want = oracle.c.gemm_fused(x[0], W, bias, r1[0], r2[0], 1)
        got = out.cpu().numpy()[0]
        assert (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 2e-3 + 2.0 ** -8 * np.maximum(np.abs(r1[0]), np.abs(r2[0]))).all()
        out32 = torch.empty(1, 1, 2560, dtype=torch.float32, device="cuda")
        mod["fused_NT_matmul8_add5_add7_add7_cast5"](t(x), t(W), t(bias), t(r1), t(r2), out32)
        assert (np.abs(out32.cpu().numpy()[0].astype(np.float64) - want.astype(np.float64)) <= 2e-3 + 2.0 ** -8 * np.maximum(np.abs(r1[0]), np.abs(r2[0]))).all()
        out2 = torch.empty(1, 1, 10240, dtype=torch.float16, device="cuda")
        mod["fused_NT_matmul9_add6_gelu1"](t(x), t(W2), t(bias2), out2)
        want = oracle.np64.gemm_fused(x[0], W2, bias2, None, None, 3)
        assert (np.abs(out2.cpu().numpy()[0].astype(np.float64) - want) <= 4e-3 + 1e-2 * np.abs(want)).all()


def test_layout_and_sampling_primfuncs_through_the_module(tmp_path, oracle):
    """split / fused_reshape7_split1, transpose6 / 7 / 8 and softmax_with_temperature: served by the library's own choice."""
    funcs = [pf.split(), pf.split(decode=True), pf.transpose(), pf.transpose(back=True), pf.transpose(decode=True),
             pf.softmax_with_temperature(), pf.divide(), pf.softmax2(), pf.layer_norm(), pf.layer_norm(decode=True)]
    work_dir = str(tmp_path / "layout")
    rt = Engine(topk=2, parallel_build=False, work_dir=work_dir).tune_module(pf.module(*funcs), arch=MI355X(0, require_device=True))
    rng = np.random.default_rng(12)
    t = lambda a: torch.from_numpy(a).cuda()
    bits = lambda x: x.cpu().numpy().view(np.uint16)
    for mod in (rt, load_module_from_file(work_dir)):
        for name, n in (("split", 37), ("fused_reshape7_split1", 1)):
            a = rng.integers(0, 2 ** 16, (1, n, 32, 240), dtype=np.uint16).view(np.float16)
            outs = [torch.empty(1, n, 32, 80, dtype=torch.float16, device="cuda") for _ in range(3)]
            mod[name](t(a if n > 1 else a.reshape(1, 1, 7680)), *outs)
            for got, want in zip(outs, oracle.layout.split3(a)):
                assert np.array_equal(bits(got), want.view(np.uint16))
        a = rng.integers(0, 2 ** 16, (1, 21, 32, 80), dtype=np.uint16).view(np.float16)
        out = torch.empty(1, 32, 21, 80, dtype=torch.float16, device="cuda")
        mod["transpose6"](t(a), out)
        assert np.array_equal(bits(out), oracle.layout.swap_axes(a).view(np.uint16))
        back = torch.empty(1, 21, 32, 80, dtype=torch.float16, device="cuda")
        mod["transpose7"](out, back)
        assert np.array_equal(bits(back), a.view(np.uint16))
        one = torch.empty(1, 32, 1, 80, dtype=torch.float16, device="cuda")
        mod["transpose8"](t(a[:, :1].copy()), one)
        assert np.array_equal(bits(one).reshape(32, 80), a[0, 0].view(np.uint16))
        logits = (rng.standard_normal((1, 1, 50280)) * 4).astype(np.float32)
        probs = torch.empty(1, 1, 50280, dtype=torch.float32, device="cuda")
        mod["softmax_with_temperature"](t(logits), torch.tensor(0.8, dtype=torch.float32, device="cuda"), probs)
        want = oracle.c.softmax_temperature(logits, 0.8)
        assert np.abs(probs.cpu().numpy() - want).max() < 1e-2 and np.abs(probs.cpu().numpy() / want - 1).max() < 1e-3
        for name, n in (("layer_norm", 9), ("layer_norm1", 1)):
            x = rng.standard_normal((1, n, 2560)).astype(np.float32)
            gm, bt = rng.uniform(0.5, 1.5, 2560).astype(np.float32), rng.uniform(-1, 1, 2560).astype(np.float32)
            y = torch.empty(1, n, 2560, dtype=torch.float32, device="cuda")
            mod[name](t(x), t(gm), t(bt), y)
            assert np.abs(y.cpu().numpy() - oracle.c.layer_norm_f32(x, gm, bt)).max() < 1e-4
        div, two = torch.empty_like(probs), torch.empty_like(probs)
        mod["divide2"](t(logits), torch.tensor(0.8, dtype=torch.float32, device="cuda"), div)
        assert np.array_equal(div.cpu().numpy().view(np.uint32), oracle.c.divide(logits, 0.8).view(np.uint32))
        mod["softmax2"](div, two)
        assert np.abs(two.cpu().numpy() / want - 1).max() < 1e-3


def test_profile_sweep_writes_the_reference_file_format(tmp_path):
    """tune -> reload from the work_dir -> sweep: latency.json / bandwidth.json as the reference's profile scripts
    write them ({"<n>": us}, {"<n>": GiB/s}; experiment/dtas_tuned/elementwise/add/profile_add.py)."""
    import json
    import os

    from dtas_amd import primfuncs as pf
    from dtas_amd.arch import MI355X
    from dtas_amd.codegen.runtime_packer import load_module_from_file
    from dtas_amd.engine.tuner import Engine
    from dtas_amd.tuning_test import profile_add

    work_dir = str(tmp_path / "add_f16")
    Engine(1, parallel_build=False, work_dir=work_dir).tune_module(
        pf.module(pf.add("float16", 2560), upper_bound={"n": 1024}), arch=MI355X(0, require_device=True), range_div_factor=256)
    rt_mod = load_module_from_file(work_dir)

    def make(n):
        a = torch.rand(1, n, 2560, device="cuda").half()
        return a, torch.rand(1, n, 2560, device="cuda").half(), torch.empty_like(a)

    latency, bandwidth = profile_add.sweep(rt_mod, "add", make, lambda n: n * 2560 * 3 * 2, (1, 300, 1024), number=3, min_repeat_ms=2)
    profile_add.save_to_json(latency, os.path.join(work_dir, "latency.json"))
    profile_add.save_to_json(bandwidth, os.path.join(work_dir, "bandwidth.json"))
    lat = json.load(open(os.path.join(work_dir, "latency.json")))
    bw = json.load(open(os.path.join(work_dir, "bandwidth.json")))
    assert list(lat) == ["1", "300", "1024"] and all(0.5 < v < 1000 for v in lat.values())
    assert bw["1024"] > bw["1"] > 0                       # the launch floor dominates n = 1
    assert abs(bw["1024"] - 1024 * 2560 * 6 / 2 ** 30 / (lat["1024"] * 1e-6)) < 1e-6 * bw["1024"]

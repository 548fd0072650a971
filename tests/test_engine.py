"""Host-side flow of the reference's entry points on CPU: Engine.tune_module -> runtime module ->
load_module_from_file; bucket index statement; argument binding.  No kernel is launched."""
import json
import os

import pytest
import torch

import dtas_amd
from dtas_amd import _lib, primfuncs as pf
from dtas_amd.arch import MI355X
from dtas_amd.codegen.runtime_packer import bind_extents, extents_of, load_module_from_file, op_id_of
from dtas_amd.common.analisys import FuncInfo, FuncKind
from dtas_amd.common.config import Range
from dtas_amd.engine.tuner import Engine


def _module():
    return pf.module(pf.add("float16", 4096), pf.cast("float32", "float16", 4096), pf.copy("float16", 4096),
                     pf.rms_norm(4096), pf.fused_layer_norm_cast1(2560), pf.softmax_scores(32),
                     pf.fused_softmax_cast3(32), pf.fused_NT_matmul_add_gemv(4096, 4096, bias=False),
                     pf.fused_NT_matmul_add_gemm(11008, 4096, bias=True), upper_bound={"n": 4096, "m": 512})


def test_rule_selection():
    kinds = {name: FuncInfo(f).kind for name, f in _module().functions_items()}
    assert kinds["add"] == kinds["cast"] == kinds["copy"] == FuncKind.kFunc_Elementwise
    assert kinds["rms_norm"] == kinds["fused_layer_norm_cast1"] == kinds["softmax_scores"] == FuncKind.kFunc_Reduction
    assert kinds["NT_matmul10"] == FuncKind.kFunc_GEMV and kinds["fused_NT_matmul4_add1"] == FuncKind.kFunc_GEMM
    assert [v.name for v in pf.fused_softmax_cast3().dynamic_args] == ["n", "m"]
    assert op_id_of(pf.cast("float32", "float16")) == _lib.OP_CAST_F32_F16
    assert op_id_of(pf.add("int8")) == _lib.OP_ADD_I8


def test_tune_module_writes_tables_and_reloads(tmp_path):
    eng = Engine(topk=10, parallel_build=True, work_dir=str(tmp_path))
    rt = eng.tune_module(_module(), arch=MI355X(), range_div_factor=256)
    assert os.path.exists(tmp_path / "dispatch_table.json") and os.path.exists(tmp_path / "dispatch_tables.h")
    assert os.path.exists(tmp_path / "data_base" / "best_record.json")
    records = json.load(open(tmp_path / "data_base" / "best_record.json"))
    assert any(k.startswith("add_<n: Range(1, 256)>") for rec in records for k in rec)
    add = rt.tables["add"]
    assert len(add.index_table) == 16 and add.index_stmt() == "  int64_t index = (n/256) > 15 ? 15 : n/256;\n"
    # every call-table row is launchable according to the C library
    for name, table in rt.tables.items():
        for entry in table.call_table:
            hi = {r.var.name: r.end for r in entry.ranges}
            _lib.describe_launch(op_id_of(table.func), *extents_of(table.func, hi), entry.abi)
    # GEMM picks the weight-streaming kernel only where M fits it, big tiles at big M
    gemm = rt.tables["fused_NT_matmul4_add1"]
    assert gemm.select({"n": 4096}).abi.variant == _lib.GEMM_MFMA
    assert list(gemm.select({"n": 4000}).abi.tile)[:2] == [256, 256]
    # a static function (GEMV) has one row and no index table
    assert rt.tables["NT_matmul10"].index_table == [] and len(rt.tables["NT_matmul10"].call_table) == 1

    again = load_module_from_file(str(tmp_path))
    for name, table in rt.tables.items():
        other = again.tables[name]
        assert other.index_table == table.index_table
        assert [e.abi.to_dict() for e in other.call_table] == [e.abi.to_dict() for e in table.call_table]
        assert [e.name for e in other.call_table] == [e.name for e in table.call_table]
    with pytest.raises(FileNotFoundError):
        load_module_from_file(str(tmp_path / "nope"))


def test_index_statement_semantics(tmp_path):
    rt = Engine(1, work_dir=str(tmp_path)).tune_module(pf.module(pf.rms_norm(4096), pf.fused_softmax_cast3(),
                                                                 upper_bound={"n": 4096, "m": 512}), MI355X(), 256)
    t = rt.tables["rms_norm"]
    # C integer division, clamped: n = 255 -> 0, n = 256 -> 1 (the reference's n / div), n >= 4096 -> 15
    assert [t.index({"n": n}) for n in (1, 255, 256, 511, 512, 4095, 4096, 10 ** 6)] == [0, 0, 1, 1, 2, 15, 15, 15]
    t2 = rt.tables["fused_softmax_cast3"]
    assert len(t2.index_table) == 16 * 2
    assert t2.index({"n": 300, "m": 100}) == 1 * 2 + 0 and t2.index({"n": 300, "m": 300}) == 1 * 2 + 1
    assert t2.index({"n": 10 ** 6, "m": 10 ** 6}) == 31
    # each cell of the 2-D table points at the merged entry whose rectangle contains it
    for a in range(16):
        for b in range(2):
            entry = t2.call_table[t2.index_table[a * 2 + b]]
            rn, rm = entry.ranges
            assert rn.start <= a * 256 + 1 <= rn.end and rm.start <= b * 256 + 1 <= rm.end


def test_past_the_upper_bound_the_library_sizes_the_launch(tmp_path):
    """A row is validated up to its bucket's end only: above the table's bound select() hands the
    choice to the library, whose own config is launchable for any extent."""
    rt = Engine(3, work_dir=str(tmp_path)).tune_module(_module(), MI355X(), 256)
    for name, table in rt.tables.items():
        if not table.dynamic_args:
            continue
        ub = table.upper_bound
        inside = {a: ub[a] for a in table.dynamic_args}
        assert table.select(inside) is not None
        for factor_plus in ((1, 1), (8, 0)):
            for a in table.dynamic_args:
                beyond = dict(inside)
                beyond[a] = ub[a] * factor_plus[0] + factor_plus[1]
                assert table.select(beyond) is None, (name, beyond)
                ext = extents_of(table.func, beyond)
                info = _lib.select_bucket(op_id_of(table.func), *ext)   # the library's own config fits
                assert info.launch_args[0] >= 1 and info.launch_args[3] >= 64


def test_generated_header_and_python_dispatcher_agree_also_past_the_upper_bound(tmp_path):
    """The C text written beside the tables (<func>_select) and FunctionTable.select() choose the same row for the
    same extents, and both hand extents above the upper bound to the library (NULL / None)."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("needs gcc")
    rt = Engine(3, work_dir=str(tmp_path)).tune_module(_module(), MI355X(), 256)
    probes = {1: [1, 255, 256, 257, 1024, 4095, 4096, 4097, 40000],
              2: [(1, 1), (300, 511), (4096, 512), (4096, 1), (4097, 5), (17, 513), (9000, 9000)]}
    cases, body = [], []
    for name, table in rt.tables.items():
        args = table.dynamic_args[:2]
        if not args or not table.index_table:
            continue
        for probe in probes[len(args)]:
            vals = (probe,) if len(args) == 1 else probe
            cases.append((name, table, dict(zip(args, vals))))
            call = f"{name}_select({', '.join(str(v) for v in vals)})"
            body.append(f'  printf("%ld\\n", {call} ? (long)({call} - {name}_call_table) : -1L);')
    assert len(cases) > 30
    src = tmp_path / "sel.c"
    src.write_text('#include <stdio.h>\n#include "dispatch_tables.h"\nint main(void) {\n' + "\n".join(body) + "\n  return 0;\n}\n")
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    exe = tmp_path / "sel"
    subprocess.check_call([gcc, "-std=c99", "-Wall", "-Wno-unused-function", "-Wno-unused-const-variable", "-Werror", "-I", include, "-I", str(tmp_path), str(src), "-o", str(exe)])
    got = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    for (name, table, values), row in zip(cases, got):
        entry = table.select(values)
        want = -1 if entry is None else table.call_table.index(entry)
        assert row == want, (name, values, row, want)
        beyond = any(values[a] > table.upper_bound[a] for a in values)
        assert (want == -1) == beyond, (name, values)


def test_merge_two_dynamic_extents(tmp_path):
    from dtas_amd.codegen.compile_result import CompileResult
    from dtas_amd.common.config import ReductionConfig

    def cr(tx):
        c = ReductionConfig()
        c.len_tx = tx
        return CompileResult(c, c.to_abi(), "f")

    eng = Engine(1, work_dir=str(tmp_path))
    eng.upper_bound.update({"n": 768, "m": 512})
    best = {}
    for i, n0 in enumerate((1, 257, 513)):
        for j, m0 in enumerate((1, 257)):
            tx = 128 if i == 0 and j == 0 else 256 if i == 0 else 512
            best[(Range("n", n0, n0 + 255), Range("m", m0, m0 + 255))] = cr(tx)
    merged = eng.merge_same_configs(best)
    got = [(rt[0].start, rt[0].end, rt[1].start, rt[1].end, c.config.len_tx) for rt, c in merged.items()]
    assert got == [(1, 256, 1, 256, 128), (1, 256, 257, 512, 256), (257, 768, 1, 512, 512)]
    table, stmt = eng.get_index_table(merged, 256)
    assert table == [0, 1, 2, 2, 2, 2]


def test_bind_extents_checks_the_signature():
    f = pf.add("float16", 64)
    a = torch.zeros(1, 5, 64, dtype=torch.float16)
    assert bind_extents(f, [a, a, a]) == {"n": 5}
    with pytest.raises(TypeError, match="takes 3 buffers"):
        bind_extents(f, [a, a])
    with pytest.raises(TypeError, match="float16"):
        bind_extents(f, [a, a.float(), a])
    with pytest.raises(ValueError, match="expects shape"):
        bind_extents(f, [a, a, torch.zeros(1, 5, 32, dtype=torch.float16)])
    with pytest.raises(ValueError, match="extent n"):
        bind_extents(f, [a, a, torch.zeros(1, 6, 64, dtype=torch.float16)])


def test_layout_and_sampling_descriptors_follow_the_graph_signatures():
    from dtas_amd.codegen.runtime_packer import LIBRARY_CHOSEN_OPS

    sp = pf.split()
    assert sp.name == "split" and [p.shape for p in sp.params] == [(1, "n", 32, 240)] + [(1, "n", 32, 80)] * 3
    a, o = torch.zeros(1, 6, 32, 240, dtype=torch.float16), torch.zeros(1, 6, 32, 80, dtype=torch.float16)
    assert bind_extents(sp, [a, o, o, o]) == {"n": 6}
    dec = pf.split(decode=True)
    assert dec.name == "fused_reshape7_split1" and dec.params[0].shape == (1, 1, 7680) and dec.params[1].shape == (1, 1, 32, 80)
    t6, t7, t8 = pf.transpose(), pf.transpose(back=True), pf.transpose(decode=True)
    assert (t6.name, t7.name, t8.name) == ("transpose6", "transpose7", "transpose8")
    assert t6.params[0].shape == t7.params[1].shape == (1, "n", 32, 80) and t6.params[1].shape == t7.params[0].shape == (1, 32, "n", 80)
    assert t8.params[0].shape == (1, 1, 32, 80) and t8.params[1].shape == (1, 32, 1, 80)
    sm = pf.softmax_with_temperature()
    assert [p.shape for p in sm.params] == [(1, 1, 50280), (), (1, 1, 50280)] and all(p.dtype == "float32" for p in sm.params)
    assert bind_extents(sm, [torch.zeros(1, 1, 50280), torch.tensor(0.7), torch.zeros(1, 1, 50280)]) == {}
    dv, s2 = pf.divide(), pf.softmax2()
    assert (dv.name, s2.name) == ("divide2", "softmax2") and [p.shape for p in dv.params] == [(1, 1, 50280), (), (1, 1, 50280)]
    assert [p.shape for p in s2.params] == [(1, 1, 50280)] * 2 and s2.params[1].dtype == "float32"
    assert all(f.op in LIBRARY_CHOSEN_OPS for f in (sp, dec, t6, t7, t8, sm, dv, s2))


def test_cpu_tensors_are_refused_not_computed_elsewhere():
    from dtas_amd import ops

    a = torch.zeros(4, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.add(a, a, a.clone())


def _first_candidate(func, ranges):
    from dtas_amd.schedule.schedule import get_config_emiter_template  # the rule -> emitter mapping the Engine uses
    info = FuncInfo(func)
    return get_config_emiter_template(info.kind)(info, MI355X()).emit_config(ranges, 20)[0].to_abi().to_dict()


@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (4096, 11008), (2560, 10240), (4096, 1024), (1024, 1024), (8192, 8192)])
def test_gemm_emitter_leads_with_the_librarys_builtin_choice(N, K):
    # the closed-form policy exists twice (C tables for cfg == NULL, Python emitter for the tuner's
    # first candidate): they must not drift apart
    func = pf.fused_NT_matmul_add_gemm(N, K, bias=True)
    for m_hi in (16, 32, 48, 64, 128, 256, 512, 1024, 2048, 4096, 8192):
        want = _lib.select_bucket(_lib.OP_GEMM_F16, m_hi, N, K).config.to_dict()
        got = _first_candidate(func, (Range("n", m_hi - 15, m_hi),))
        keys = ("variant", "tile", "split_k") if want["variant"] == _lib.GEMM_SKINNY else ("variant", "block", "tile", "unroll", "split_k")
        if want["variant"] == _lib.GEMM_MFMA and want["block"] == 512:
            keys = ("variant", "block", "tile", "split_k")   # the 8-wavefront ring loops have no stage count
        assert {k: got[k] for k in keys} == {k: want[k] for k in keys}, (m_hi, got, want)


def test_reduction_emitters_lead_with_the_librarys_builtin_choice():
    cases = [(mk(H), op, H) for H in (1024, 2560, 4096, 5120, 6144, 8192, 16384)
             for mk, op in ((pf.rms_norm, _lib.OP_RMS_NORM_F16), (pf.fused_layer_norm_cast1, _lib.OP_LAYER_NORM_F32_F16))]
    for func, op, H in cases:
        for n_hi in (16, 256, 1024, 1040, 1536, 2032, 2048, 2064, 3072, 3088, 4096, 4112, 6144, 6160, 8192):
            want = _lib.select_bucket(op, n_hi, H, 0).config.to_dict()
            got = _first_candidate(func, (Range("n", n_hi - 15, n_hi),))
            for k in ("variant", "block", "vec", "unroll"):
                assert got[k] == want[k], (func.name, n_hi, got, want)


@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (4096, 11008), (2560, 2560), (28672, 1024), (5120, 1024),
                                 (8192, 2048), (4096, 520), (32000, 4096), (2560, 10240), (50280, 512), (4096, 512)])
def test_gemv_emitter_leads_with_the_librarys_builtin_choice(N, K):
    want = _lib.select_bucket(_lib.OP_GEMV_F16, 1, N, K).config.to_dict()
    got = _first_candidate(pf.fused_NT_matmul_add_gemv(N, K, bias=True), ())
    assert (got["block"], got["tile"][0]) == (want["block"], want["tile"][0]), (got, want)


def test_elementwise_emitter_leads_with_the_librarys_builtin_choice():
    # the deepest unroll that leaves every CU a few workgroups -- and one access per thread (two for the cast to
    # fp16) once eight per thread no longer fit the chip in one round
    cases = [(pf.add("float16", H), _lib.OP_ADD_F16, H) for H in (2560, 4096)] + \
            [(pf.cast("float32", "float16", H), _lib.OP_CAST_F32_F16, H) for H in (2560, 4096)] + \
            [(pf.cast("float16", "float32", 4096), _lib.OP_CAST_F16_F32, 4096), (pf.copy("float16", 4096), _lib.OP_COPY_F16, 4096),
             (pf.add("float32", 4096), _lib.OP_ADD_F32, 4096), (pf.add("int8", 4096), _lib.OP_ADD_I8, 4096)]
    seen = set()
    for func, op, H in cases:
        for n_hi in (16, 128, 512, 1024, 2048, 4096, 4112, 5120, 6144, 6160, 7168, 8192):
            want = _lib.select_bucket(op, n_hi, H, 0).config.to_dict()
            got = _first_candidate(func, (Range("n", n_hi - 15, n_hi),))
            for k in ("variant", "block", "vec", "unroll"):
                assert got[k] == want[k], (func.name, H, n_hi, got, want)
            seen.add((op, want["unroll"]))
    assert {(_lib.OP_ADD_F16, 8), (_lib.OP_ADD_F16, 1), (_lib.OP_CAST_F32_F16, 2), (_lib.OP_COPY_F16, 8)} <= seen


def test_builtin_reduction_rows_are_launchable_for_every_extent():
    # the table row for any row count x row length must be a form the register kernels exist in (select_bucket
    # describes its launch and fails otherwise): LayerNorm over rows of 16384 once named 832 threads x 2 rows
    lengths = (1, 8, 64, 100, 777, 1024, 2048, 2560, 3072, 4096, 4100, 5120, 6144, 8192, 10240, 12288, 16384, 20000, 32768, 65536)
    for n_hi in (1, 16, 512, 1024, 1040, 2047, 2048, 3000, 4096, 4097, 6144, 8192, 10 ** 5):
        for H in lengths:
            for op in (_lib.OP_RMS_NORM_F16, _lib.OP_LAYER_NORM_F32_F16):
                info = _lib.select_bucket(op, n_hi, H, 0)
                assert info.launch_args[0] >= 1 and 64 <= info.launch_args[3] <= 1024, (op, n_hi, H)
            for op in (_lib.OP_SOFTMAX_F32_F16, _lib.OP_SOFTMAX_F16):
                info = _lib.select_bucket(op, H, 32 * n_hi, H)
                assert info.launch_args[0] >= 1 and 64 <= info.launch_args[3] <= 1024, (op, n_hi, H)


def test_softmax_emitter_leads_with_the_librarys_builtin_choice():
    # rows of dynamic length m, 32 * n of them: a wavefront per row up to 512 vectors, then four wavefronts per row
    # up to 2048, then wider workgroups
    for func, op in ((pf.fused_softmax_cast3(32), _lib.OP_SOFTMAX_F32_F16), (pf.softmax_scores(32), _lib.OP_SOFTMAX_F16)):
        for n_hi in (16, 128, 1024):
            for m_hi in (64, 256, 1024, 2048, 4096, 8192, 16384, 32768):
                names = [v.name for v in func.dynamic_args]
                if names == ["n"]:
                    n_hi = m_hi                     # square scores: one extent is both the row factor and the row length
                want = _lib.select_bucket(op, m_hi, 32 * n_hi, m_hi).config.to_dict()
                ranges = tuple(Range(nm, (n_hi if nm == "n" else m_hi) - 15, n_hi if nm == "n" else m_hi) for nm in names)
                got = _first_candidate(func, ranges)
                for k in ("variant", "block", "vec", "unroll"):
                    assert got[k] == want[k], (func.name, n_hi, m_hi, got, want)


def test_builtin_tables_name_a_launchable_kernel_for_every_bucket_and_shape():
    # whatever the extents, the row the built-in table returns must be one its own launch description accepts
    # (no GPU needed: both are host code), with a tile the kernels exist for and a split that keeps 8 k tiles
    for N in (1, 7, 64, 100, 2560, 4096, 7680, 11008, 32000, 50280, 250000):
        for K in (8, 64, 80, 520, 2560, 4096, 11008, 32768):
            for M in (1, 2, 15, 16, 17, 64, 100, 256, 257, 1000, 2048, 4096, 4097, 10 ** 5):
                info = _lib.select_bucket(_lib.OP_GEMM_F16, M, N, K)
                c = info.config
                again = _lib.describe_launch(_lib.OP_GEMM_F16, M, N, K, c)
                assert list(again.launch_args) == list(info.launch_args), (M, N, K)
                assert info.bucket_lo <= max(M, 1) and (M <= info.bucket_hi or info.index == 511), (M, N, K, info.bucket_lo, info.bucket_hi)
                if c.variant == _lib.GEMM_MFMA:
                    assert (c.tile[0], c.tile[1]) in {(256, 256), (192, 256), (256, 128), (192, 128), (128, 128), (128, 64), (64, 64)} and c.tile[2] == 64
                    # (split_k = 0, the 8-wavefront 256x256 tile only: the library splits just the tiles of a partly filled last round)
                    assert (c.split_k == 0 and tuple(c.tile[:2]) == (256, 256) and c.block == 512) or \
                        (1 <= c.split_k <= 4 and (c.split_k == 1 or -(-K // 64) // c.split_k >= 8)), (M, N, K, c.split_k)
                elif c.variant == _lib.GEMM_STREAM and c.tile[2] == 256:
                    # the looping form: one round of the chip, two one-wavefront workgroups or one of four wavefronts per CU
                    assert M <= 16 and K <= 4096 and (list(c.tile[:2]), c.block) in (([16, 16], 64), ([16, 64], 256))
                    assert (256 < info.launch_args[0] <= 512) if c.tile[1] == 16 else (128 <= info.launch_args[0] <= 256)
                elif c.variant == _lib.GEMM_STREAM:
                    # at most one workgroup per CU: 64 columns x 1024 of K each up to 16 rows, x 512 of K for 17 .. 32
                    assert c.block == 256 and info.launch_args[0] <= 256
                    assert (M <= 16 and list(c.tile) == [16, 64, 1024]) or (16 < M <= 32 and list(c.tile) == [32, 64, 512] and info.launch_args[0] >= 64)
                else:
                    assert c.variant == _lib.GEMM_SKINNY and M <= 32 and c.tile[0] >= min(M, 32)
            info = _lib.select_bucket(_lib.OP_GEMV_F16, 1, N, K)
            assert list(_lib.describe_launch(_lib.OP_GEMV_F16, 1, N, K, info.config).launch_args) == list(info.launch_args)
    for op, H in ((_lib.OP_ADD_F16, 4096), (_lib.OP_CAST_F32_F16, 2560), (_lib.OP_COPY_I8, 4096), (_lib.OP_RMS_NORM_F16, 4096),
                  (_lib.OP_LAYER_NORM_F32_F16, 2560)):
        for n in (1, 16, 17, 255, 256, 257, 4096, 4097, 10 ** 6):
            info = _lib.select_bucket(op, n, H, 0)
            assert list(_lib.describe_launch(op, n, H, 0, info.config).launch_args) == list(info.launch_args), (op, n)
    for op in (_lib.OP_SOFTMAX_F16, _lib.OP_SOFTMAX_F32_F16):
        for n in (1, 7, 8, 33, 256, 257, 1025, 2047, 4096, 4097, 20000):
            info = _lib.select_bucket(op, n, 32 * n, n)
            assert list(_lib.describe_launch(op, n, 32 * n, n, info.config).launch_args) == list(info.launch_args), (op, n)

"""Known-answer tests for the host-side dispatcher logic against data the reference holds.

tests/golden/dispatch_kats.json was extracted from the reference's committed tuning artefacts
(host.cc call/index tables, data_base/best_record.json, data_base/tuning_record.py) by
tests/golden/make_dispatch_kats.py.  Feeding the reference's per-bucket winners into this package's
merge_same_configs / get_index_table must reproduce the tables the reference's Engine emitted, and
the config emitters evaluated with the reference's architecture constants (RTX 3090) must
reproduce the candidates it recorded."""
import json
import os

import pytest

from dtas_amd import primfuncs as pf
from dtas_amd.arch import RTX3090
from dtas_amd.codegen.compile_result import CompileResult
from dtas_amd.common.analisys import FuncInfo, FuncKind
from dtas_amd.common.config import ElementwiseConfig, Range, ReductionConfig, generate_range_list
from dtas_amd.engine.tuner import Engine
from dtas_amd.policy import ElementwiseConfigEmiter, ReductionConfigEmiter

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "dispatch_kats.json")))
DYNAMIC = {k: v for k, v in KATS.items() if "call_table" in v["host"]}
STATIC = {k: v for k, v in KATS.items() if "call_table" not in v["host"]}


def test_fixture_covers_every_artefact_dir():
    assert len(KATS) == 19 and len(DYNAMIC) == 17 and len(STATIC) == 2


def test_generate_range_list_matches_recorded_buckets():
    ranges = generate_range_list("n", 1, 4096, 256)
    assert [(r.start, r.end) for r in ranges] == [(1 + 256 * i, 256 * (i + 1)) for i in range(16)]
    for kat in KATS.values():
        got = [[r.var.name, r.start, r.end] for r in ranges]
        assert [b["ranges"][0] for b in kat["best_record"]] == got
    assert [(r.start, r.end) for r in generate_range_list("n", 1, 200, 256)] == [(1, 256)]   # end-start <= div
    assert [(r.start, r.end) for r in generate_range_list("m", 1, 512, 256)] == [(1, 256), (257, 512)]
    assert ranges[0].to_suffix() == "_n_1_to_256_"


def _cfg(kind_hint, dic):
    cls = ReductionConfig if "temp_storage" in dic else ElementwiseConfig
    c = cls().from_dict(dic)
    if cls is ReductionConfig:
        c.max_active_blocks_per_sm = dic.get("max_active_blocks_per_sm", 0)
    return c


def _engine(tmp_path):
    e = Engine(10, work_dir=str(tmp_path))
    e.upper_bound["n"] = 4096
    return e


@pytest.mark.parametrize("name", sorted(DYNAMIC))
def test_merge_and_index_table_reproduce_host_cc(name, tmp_path):
    kat = DYNAMIC[name]
    func = kat["host"]["func"]
    best = {}
    for b in kat["best_record"]:
        rt = tuple(Range(v, lo, hi) for v, lo, hi in b["ranges"])
        cfg = _cfg(func, b["config"])
        best[rt] = CompileResult(cfg, cfg.to_abi(), func)
    eng = _engine(tmp_path)
    merged = eng.merge_same_configs(best)
    index_table, index_stmt = eng.get_index_table(merged, 256)
    host = kat["host"]
    assert index_table == host["index_table"]
    assert index_stmt == host["index_stmt"]
    names = [f"{func}{''.join(r.to_suffix() for r in rt)}_kernel" for rt in merged]
    assert names == [row["name"] for row in host["call_table"]]
    # launch_args of each row = {grid, block[, dyn smem]} of the merged range's config
    for (rt, cr), row in zip(merged.items(), host["call_table"]):
        d = cr.config.to_dict()
        if "grid_size" in d:
            assert row["launch_args"] == [d["grid_size"], d["len_tx"]]
        else:
            assert row["launch_args"][1] == d["len_tx"]


@pytest.mark.parametrize("name", sorted(STATIC))
def test_one_config_for_all_buckets_gives_a_single_unsuffixed_kernel(name, tmp_path):
    kat = STATIC[name]
    best = {}
    for b in kat["best_record"]:
        rt = tuple(Range(v, lo, hi) for v, lo, hi in b["ranges"])
        cfg = _cfg("", b["config"])
        best[rt] = CompileResult(cfg, cfg.to_abi(), "fused_layer_norm_cast1")
    merged = _engine(tmp_path).merge_same_configs(best)
    assert len(merged) == 1
    (rt,) = merged.keys()
    assert (rt[0].start, rt[0].end) == (1, 4096)
    assert kat["host"]["single_kernel"] == ["fused_layer_norm_cast1_kernel"]


def test_softmax_kat_in_closed_form(tmp_path):
    # per-bucket best len_tx recorded for softmax row_12800 -> 8 kernels and this index table
    txs = [128, 128, 128, 128, 160, 160, 256, 192, 288, 224, 256, 256, 288, 288, 288, 288]
    best = {}
    for i, tx in enumerate(txs):
        c = ReductionConfig()
        c.len_tx, c.temp_storage, c.vector_size = tx, "cache", None
        best[(Range("n", 1 + 256 * i, 256 * (i + 1)),)] = CompileResult(c, c.to_abi(), "fused_softmax_cast")
    eng = _engine(tmp_path)
    merged = eng.merge_same_configs(best)
    table, _ = eng.get_index_table(merged, 256)
    assert table == [0, 0, 0, 0, 1, 1, 2, 3, 4, 5, 6, 6, 7, 7, 7, 7]
    assert len(merged) == 8


@pytest.mark.parametrize("dtype,vecs", [("float16", [8, 4, 2]), ("float32", [4, 3, 2, 1]), ("int8", [16, 8, 4])])
def test_elementwise_emitter_reproduces_recorded_candidates(dtype, vecs):
    info = FuncInfo(pf.add(dtype, 2560))
    assert info.kind == FuncKind.kFunc_Elementwise
    em = ElementwiseConfigEmiter(info, RTX3090())
    kat = KATS[f"experiment/dtas_tuned/elementwise/add/{dtype}/top10_256"]
    for bucket in kat["candidates"]:
        rt = tuple(Range(v, lo, hi) for v, lo, hi in bucket["ranges"])
        got = em.emit_config(rt, 10)
        assert [c.vector_size for c in got] == vecs
        want = {c["config"]["vector_size"]: c["config"]["grid_size"] for c in bucket["configs"]}
        assert {c.vector_size: c.grid_size for c in got} == want
        assert all(c.len_tx == 256 and c.unroll_depth == 256 for c in got)


def test_elementwise_grid_cap():
    em = ElementwiseConfigEmiter(FuncInfo(pf.add("float16", 2560)), RTX3090())
    assert em.get_num_blocks(2560 * 256, 8, 82, 1536) == 320
    assert em.get_num_blocks(10 ** 12, 8, 82, 1536) == 15744  # 82 * 1536 / 256 * 32
    assert em.get_num_blocks(1, 8, 82, 1536) == 1


def test_reduction_emitter_reproduces_recorded_occupancy():
    # softmax artefacts: "cache" mode, max_active = min(1536 // tx, 16)
    info = FuncInfo(pf.fused_softmax_cast(12800))
    assert info.kind == FuncKind.kFunc_Reduction and info.dyn_red
    em = ReductionConfigEmiter(info, RTX3090())
    kat = KATS["experiment/dtas_tuned/general_reduction/softmax/row_12800/top10_256_10_nounroll"]
    recorded = {}
    for bucket in kat["candidates"]:
        for c in bucket["configs"]:
            recorded[c["config"]["len_tx"]] = c["config"]["max_active_blocks_per_sm"]
    got = em.emit_config((Range("n", 3841, 4096),), 1000)
    mine = {c.len_tx: c.max_active_blocks_per_sm for c in got}
    assert {tx: mine[tx] for tx in recorded} == recorded
    assert {128: 12, 160: 9, 192: 8, 224: 6, 256: 6, 288: 5}.items() <= mine.items()
    # top-k order: (max_active, len_tx) descending
    top = em.emit_config((Range("n", 3841, 4096),), 10)
    keys = [(c.max_active_blocks_per_sm, c.len_tx) for c in top]
    assert keys == sorted(keys, reverse=True)
    # block sizes never exceed the row length of the bucket
    small = em.emit_config((Range("n", 1, 256),), 1000)
    assert max(c.len_tx for c in small) <= 256 and min(c.len_tx for c in small) == 128

    # layer-norm artefacts: "shared.dyn" with one fp32 row (2560 * 4 bytes) of shared memory
    info = FuncInfo(pf.fused_layer_norm_cast1(2560))
    em = ReductionConfigEmiter(info, RTX3090())
    em.cuda_temp_storage, em.cuda_smem_usage = "shared.dyn", 2560 * 4
    got = {c.len_tx: c for c in em.emit_config((Range("n", 1, 256),), 1000)}
    kat = KATS["experiment/dtas_tuned/general_reduction/layernorm/top10_256_2"]
    for b in kat["best_record"]:
        cfg = b["config"]
        assert got[cfg["len_tx"]].max_active_blocks_per_sm == cfg["max_active_blocks_per_sm"]
        assert got[cfg["len_tx"]].vector_size == cfg["vector_size"] == 4
    assert {tx: got[tx].max_active_blocks_per_sm for tx in (128, 192, 256, 320, 512)} == {128: 10, 192: 8, 256: 6, 320: 4, 512: 3}

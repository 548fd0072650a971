"""The tuning engine: bucket ranges, per-bucket selection, bucket merging, index table.

Same entry points and results as the reference's ``Engine`` (python/dtas/engine/tuner.py:22-299):
``Engine(topk, parallel_build, work_dir).tune_module(mod, arch, range_div_factor)`` returns a runtime
module whose functions dispatch on the dynamic extents.  What differs is underneath: candidates are
rows of the C library's call table (prebuilt gfx950 kernel variants), not TIR schedules to compile.
"""
from __future__ import annotations

import os
import tempfile
from itertools import product
from typing import Dict, List, Tuple

from ..arch import Arch
from ..codegen.code_gen import CodeGenerator
from ..codegen.compile_result import CompileResult
from ..codegen.runtime_packer import LIBRARY_CHOSEN_OPS, RuntimeModule, RuntimePacker
from ..common.analisys import FuncInfo, IRModule, PrimFunc
from ..common.config import Range, generate_range_list
from ..logging import debug_info, get_log_level
from ..schedule.schedule import get_config_emiter_template, get_scheduler_template
from .database import DataBase

DEFAULT_UPPER_BOUND = 2048  # for a dynamic extent without tir_var_upper_bound (tuner.py:147)


class Engine:
    def __init__(self, topk: int = 10, parallel_build: bool = True, work_dir: str = None):
        self.topk = topk
        self.parallel_build = parallel_build
        self.upper_bound: Dict[str, int] = {}
        if work_dir is None:
            work_dir = tempfile.mkdtemp(prefix="dtas_")
        self.work_dir = work_dir
        os.makedirs(work_dir, exist_ok=True)
        database_dir = os.path.join(work_dir, "data_base")
        os.makedirs(database_dir, exist_ok=True)
        self.database = DataBase(os.path.join(database_dir, "best_record.json"),
                                 os.path.join(database_dir, "tuning_record.py"))
        if get_log_level() >= 1:
            debug_info(f"Using database dir {database_dir}")

    # ------------------------------------------------------------------------------------
    def tune_module(self, mod: IRModule, arch: Arch, range_div_factor: int = 256) -> RuntimeModule:
        for var, bound in mod.attrs.get("tir_var_upper_bound", {}).items():
            self.upper_bound[var] = bound
        for _, func in mod.functions_items():
            for var, bound in func.attrs.get("tir_var_upper_bound", {}).items():
                self.upper_bound[var] = bound
        cg = CodeGenerator(getattr(arch, "target", "gfx950"))
        for name, func in mod.functions_items():
            if not isinstance(func, PrimFunc):
                continue
            if func.op in LIBRARY_CHOSEN_OPS:   # served with the library's built-in choice: an empty call table
                cg.gen_code_for_func(func, {}, [], range_div_factor,
                                     {v.name: self.upper_bound.setdefault(v.name, DEFAULT_UPPER_BOUND) for v in func.dynamic_args})
                continue
            ranges_best_result, _, _ = self.tune_func(func, name, arch, True, range_div_factor)
            index_table, index_stmt = self.get_index_table(ranges_best_result, range_div_factor)
            if get_log_level() >= 2:
                debug_info(f"index_table: {index_table}, index_stmt: {index_stmt}")
            cg.gen_code_for_func(func, ranges_best_result, index_table, range_div_factor,
                                 {v.name: self.upper_bound[v.name] for v in func.dynamic_args})
        return RuntimePacker(cg.tables, self.work_dir).pack_to_runtime()

    def tune_func(self, func: PrimFunc, name: str, arch: Arch, use_tc: bool = False, range_div_factor: int = 256):
        assert isinstance(func, PrimFunc), "tune_func can only accept primfunc"
        func_info = FuncInfo(func, name)
        scheduler = get_scheduler_template(func_info.kind, use_tc, arch.compute_capability)(func_info)
        emiter_template = get_config_emiter_template(func_info.kind, use_tc)
        range_to_best: Dict[Tuple[Range, ...], CompileResult] = {}
        for range_tuple in self.gen_range_tuples(func_info, range_div_factor):
            configs = emiter_template(func_info, arch).emit_config(range_tuple, self.topk)
            _, best = scheduler.select_best(range_tuple, configs, arch, name, self.database, self.parallel_build)
            if best is None:
                raise RuntimeError(f"{name}: no launchable config for bucket {range_tuple}")
            range_to_best[range_tuple] = best
        merged = self.merge_same_configs(range_to_best)
        return merged, func_info.use_fp16, len(func_info.dynamic_args)

    # ------------------------------------------------------------------------------------
    def gen_range_tuples(self, func_info: FuncInfo, range_div_factor: int) -> List[Tuple[Range, ...]]:
        """One tuple of bucket ranges per combination of the dynamic extents' buckets
        (tuner.py:135-154); ``[()]`` for a static function."""
        if len(func_info.dynamic_args) == 0:
            return [()]
        range_lists = []
        for dyn_arg in func_info.dynamic_args:
            upper = self.upper_bound.setdefault(dyn_arg.name, DEFAULT_UPPER_BOUND)
            range_lists.append(generate_range_list(dyn_arg, 1, upper, range_div_factor))
        return list(product(*range_lists))

    def get_index_table(self, ranges_best_result: Dict[Tuple[Range, ...], CompileResult],
                        range_div_factor: int) -> Tuple[List[int], str]:
        """index_table[j] = row of the call table serving the j-th ``range_div_factor``-wide step,
        plus the C statement that computes j from the dynamic extents (tuner.py:156-209)."""
        index_table: List[int] = []
        index_stmt = "  int64_t index = "
        items = list(ranges_best_result.items())
        ndyn = len(items[0][0])
        if ndyn == 0:
            return index_table, index_stmt
        div = range_div_factor
        if ndyn == 1:
            name = items[0][0][0].var.name
            index_len = (self.upper_bound[name] + div - 1) // div - 1
            index_stmt += f"({name}/{div}) > {index_len} ? {index_len} : {name}/{div};\n"
            for i, (range_tuple, _) in enumerate(items):
                for _ in range(range_tuple[0].start, range_tuple[0].end + 1, div):
                    index_table.append(i)
            return index_table, index_stmt
        name0, name1 = items[0][0][0].var.name, items[0][0][1].var.name
        size0 = (self.upper_bound[name0] + div - 1) // div
        size1 = (self.upper_bound[name1] + div - 1) // div
        index_len = size0 * size1 - 1
        expr = f"({name0}/{div} * {size1} + {name1}/{div})"
        index_stmt += f"{expr} > {index_len} ? {index_len} : {expr};\n"
        # row-major over (extent 0 step, extent 1 step); merged rectangles fill their cells
        cells = [0] * (size0 * size1)
        for i, (range_tuple, _) in enumerate(items):
            for a in range(range_tuple[0].start, range_tuple[0].end + 1, div):
                for b in range(range_tuple[1].start, range_tuple[1].end + 1, div):
                    cells[((a - 1) // div) * size1 + (b - 1) // div] = i
        return cells, index_stmt

    def merge_same_configs(self, best_compile_results: Dict[Tuple[Range, ...], CompileResult]
                           ) -> Dict[Tuple[Range, ...], CompileResult]:
        """Merge adjacent buckets whose best config is the same (tuner.py:211-299): along the last
        dynamic extent first, then (two extents) along the first for entries whose second range
        agrees; the result is ordered by range start."""
        items = list(best_compile_results.items())
        ndyn = len(items[0][0])
        if ndyn == 0:
            return dict(items)
        if ndyn > 2:
            raise ValueError("only support two dynamic args")
        # per config, the list of [ranges, result] entries built so far, in arrival order
        by_config: Dict = {}
        for range_tuple, cr in items:
            entries = by_config.setdefault(cr.config, [])
            merged = False
            if entries:
                ranges = entries[-1][0]
                same_outer = ndyn == 1 or ranges[0] == range_tuple[0]
                if same_outer:
                    try:
                        ranges[-1] = ranges[-1].merge(range_tuple[-1])
                        merged = True
                    except ValueError:
                        merged = False
            if not merged:
                entries.append([list(range_tuple), cr])
        if ndyn == 2:
            for config, entries in by_config.items():
                folded: List = []
                for ranges, cr in entries:
                    if folded and folded[-1][0][1] == ranges[1]:
                        try:
                            folded[-1][0][0] = folded[-1][0][0].merge(ranges[0])
                            continue
                        except ValueError:
                            pass
                    folded.append([ranges, cr])
                by_config[config] = folded
        merged_results = {}
        for entries in by_config.values():
            for ranges, cr in entries:
                merged_results[tuple(ranges)] = cr
        return dict(sorted(merged_results.items(), key=lambda kv: tuple(r.start for r in kv[0])))

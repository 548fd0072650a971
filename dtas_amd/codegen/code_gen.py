"""Collects, per function, the dispatcher tables that the runtime packer writes out.

The reference's CodeGenerator text-splices ``call_table`` / ``index_table`` / launch arguments into
TVM's generated host C (python/dtas/codegen/code_gen.py:242-405).  No host code is generated here --
the host function is fixed C in libdtas_gfx950.so -- so the generator's product is the table data.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

from ..common.analisys import PrimFunc
from ..common.config import Range
from .compile_result import CompileResult
from .runtime_packer import FunctionTable, KernelEntryInfo


class CodeGenerator:
    def __init__(self, target: str = "amdgcn-amd-amdhsa--gfx950"):
        self.target = target
        self.tables: Dict[str, FunctionTable] = {}
        self.func_names: List[str] = []

    def gen_code_for_func(self, func: PrimFunc, ranges_best_result: Dict[Tuple[Range, ...], CompileResult],
                          index_table: List[int], range_div_factor: int, upper_bound: Dict[str, int]) -> FunctionTable:
        call_table = []
        merged = len(ranges_best_result) == 1
        for range_tuple, cr in ranges_best_result.items():
            # one config for every bucket -> a single un-suffixed kernel (code_gen.py:261-284)
            suffix = "" if merged or not range_tuple else "".join(r.to_suffix() for r in range_tuple)
            kernel_name = f"{func.name}{suffix}_kernel"
            call_table.append(KernelEntryInfo(range_tuple, cr.config, kernel_name, cr.launch_args))
        table = FunctionTable(func, call_table, index_table, range_div_factor, upper_bound)
        self.tables[func.name] = table
        self.func_names.append(func.name)
        return table

"""Scheduler templates: config -> launchable call-table row, and the per-bucket selection.

In the reference a scheduler template turns a config into a scheduled TIR module
(``apply_config``) and ``select_best`` builds every candidate and times it on ~10 evenly spaced
shapes of the bucket (python/dtas/schedule/tir_base.py:109-145, :150-298).  Here ``apply_config``
turns a config into the ``dtas_config`` row that selects a prebuilt gfx950 kernel variant;
``select_best`` validates each row against the C library and, when a GPU is present, times it on
sample shapes the same way.  Without a GPU the analytical order of the emitter decides.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .. import _lib
from ..common.analisys import FuncInfo, FuncKind
from ..common.config import Config, Range
from ..codegen.compile_result import CompileResult
from ..logging import debug_info, get_log_level
from ..reference import get_ref_tensor


class TIRSchedulerBase:
    num_sample_shapes = 3   # the reference samples 10 (parallel) / 64 (serial) shapes per bucket
    number = 5
    min_repeat_ms = 2.0

    def __init__(self, func_info: FuncInfo) -> None:
        self.func_info = func_info
        self.func = func_info.func

    # -- config -> call-table row -------------------------------------------------------
    def apply_config(self, config: Config) -> _lib.DtasConfig:
        return config.to_abi()

    def op_id(self) -> int:
        from ..codegen.runtime_packer import op_id_of

        return op_id_of(self.func)

    # -- sample inputs of a bucket --------------------------------------------------------
    def sample_values(self, range_tuple: Tuple[Range, ...]) -> List[Dict[str, int]]:
        if not range_tuple:
            return [{}]
        cols = []
        for r in range_tuple:
            pts = np.linspace(r.start, r.end, self.num_sample_shapes)
            cols.append(sorted({max(1, int(round(p))) for p in pts}))
        out = []
        for i in range(max(len(c) for c in cols)):
            out.append({r.var.name: c[min(i, len(c) - 1)] for r, c in zip(range_tuple, cols)})
        return out

    def generate_tensors(self, values: Dict[str, int], device) -> list:
        import torch

        tensors = []
        for buf in self.func.params:
            shape = tuple(values[e] if isinstance(e, str) else e for e in buf.shape)
            tensors.append(torch.from_numpy(get_ref_tensor(shape, "cpu", buf.dtype)).to(device))
        return tensors

    # -- selection ----------------------------------------------------------------------------
    def select_best(self, range_tuple: Tuple[Range, ...], configs: Sequence[Config], arch, name: str, database=None,
                    parallel_build: bool = True) -> Tuple[List[CompileResult], Optional[CompileResult]]:
        del parallel_build  # nothing is compiled per candidate
        from ..codegen.runtime_packer import call_primfunc, extents_of

        results: List[CompileResult] = []
        hi_values = {r.var.name: r.end for r in range_tuple}
        for cfg in configs:
            cr = CompileResult(cfg, self.apply_config(cfg), name)
            try:
                n, d0, d1 = extents_of(self.func, hi_values)
                cr.launch_args = list(_lib.describe_launch(self.op_id(), n, d0, d1, cr.abi).launch_args)
            except _lib.DtasError as exc:
                cr.error = str(exc)
                if get_log_level() >= 2:
                    debug_info(f"config rejected: {cfg}: {exc}")
                continue
            results.append(cr)
        if not results:
            return results, None
        device = getattr(arch, "device", None)
        if device is not None and len(results) > 1:
            tensor_sets = [self.generate_tensors(v, device) for v in self.sample_values(range_tuple)]
            for cr in results:
                cr.profile(lambda ts, abi: call_primfunc(self.func, ts, abi), tensor_sets, self.number, self.min_repeat_ms)
                if database is not None:
                    database.commit_tuning_record(range_tuple, cr)
            alive = [cr for cr in results if cr.error is None]
            best = min(alive, key=lambda cr: cr.latency) if alive else None
        else:
            best = results[0]  # the emitter's analytical order
        if best is not None and database is not None:
            database.commit_best_record(range_tuple, best)
        return results, best


class TIRElementwiseScheduler(TIRSchedulerBase):
    """python/dtas/schedule/tir_elementwise.py:23-47."""


class TIRReductionScheduler(TIRSchedulerBase):
    """python/dtas/schedule/tir_reduction.py:36-105."""


class TIRGEMVScheduler(TIRSchedulerBase):
    """python/dtas/schedule/tir_gemv.py:33-249."""


class TIRMFMAScheduler(TIRSchedulerBase):
    """python/dtas/schedule/tir_wmma.py:20-222."""

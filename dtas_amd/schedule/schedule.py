"""Rule selection: function kind -> scheduler template / config emitter
(python/dtas/schedule/schedule.py:21-77)."""
from ..common.analisys import FuncKind
from ..policy import ElementwiseConfigEmiter, GEMVConfigEmiter, MFMAConfigEmiter, ReductionConfigEmiter
from .tir_base import TIRElementwiseScheduler, TIRGEMVScheduler, TIRMFMAScheduler, TIRReductionScheduler


def get_scheduler_template(func_kind: FuncKind, use_tc: bool = True, compute_capability: str = "gfx950"):
    del use_tc, compute_capability  # one architecture, matrix cores always used for GEMM
    if func_kind == FuncKind.kFunc_GEMM:
        return TIRMFMAScheduler
    if func_kind == FuncKind.kFunc_GEMV:
        return TIRGEMVScheduler
    if func_kind == FuncKind.kFunc_Reduction:
        return TIRReductionScheduler
    if func_kind == FuncKind.kFunc_Elementwise:
        return TIRElementwiseScheduler
    raise ValueError(f"no schedule rule for {func_kind}")


def get_config_emiter_template(func_kind: FuncKind, use_tc: bool = True):
    del use_tc
    if func_kind == FuncKind.kFunc_GEMM:
        return MFMAConfigEmiter
    if func_kind == FuncKind.kFunc_GEMV:
        return GEMVConfigEmiter
    if func_kind == FuncKind.kFunc_Reduction:
        return ReductionConfigEmiter
    if func_kind == FuncKind.kFunc_Elementwise:
        return ElementwiseConfigEmiter
    raise ValueError(f"no config emitter for {func_kind}")

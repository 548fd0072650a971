"""PrimFunc descriptors and their classification.

The reference works on TVM TIR: ``FuncInfo`` normalises a ``tir.PrimFunc`` and ``get_func_kind``
sorts it into GEMM / GEMV / Reduction / Elementwise (python/dtas/common/analisys.py:49-55,
:371-452), which picks the schedule rule.  TVM is not part of this package, so a PrimFunc is
described by its *signature* -- name, parameter buffers in order (output last, destination passing),
symbolic extents, and the iteration pattern of its compute blocks -- and the same four-way
classification is made from that pattern.  (The file name keeps the reference's spelling.)
"""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import Dict, List, Optional, Sequence, Tuple, Union

from .config import Var

Extent = Union[int, str]


class FuncKind(Enum):
    kFunc_GEMM = 0
    kFunc_GEMV = 1
    kFunc_Reduction = 2
    kFunc_Elementwise = 3
    kFunc_Transpose = 4
    KFunc_Fallback = 5


@dataclass
class Buffer:
    """One PrimFunc parameter: T.match_buffer(handle, shape, dtype)."""

    name: str
    shape: Tuple[Extent, ...]
    dtype: str


@dataclass
class Block:
    """One compute block: iterator kinds ("S" spatial / "R" reduction) and the buffers it touches."""

    name: str
    iter_kinds: str
    reads: Sequence[str]
    writes: Sequence[str]


@dataclass
class PrimFunc:
    """Signature-level stand-in for a tir.PrimFunc."""

    name: str
    params: List[Buffer]
    blocks: List[Block]
    op: str  # which kernel family implements it: add / copy / cast / layer_norm / rms_norm / softmax / matmul
    attrs: Dict = field(default_factory=dict)

    @property
    def dynamic_args(self) -> List[Var]:
        """Symbolic extents in order of first appearance over the parameter list."""
        seen: List[str] = []
        for buf in self.params:
            for e in buf.shape:
                if isinstance(e, str) and e not in seen:
                    seen.append(e)
        return [Var(s) for s in seen]


class IRModule:
    """A set of PrimFuncs plus module attributes (``tir_var_upper_bound``)."""

    def __init__(self, functions: Union[Dict[str, PrimFunc], Sequence[PrimFunc]], attrs: Optional[Dict] = None):
        if not isinstance(functions, dict):
            functions = {f.name: f for f in functions}
        self.functions: Dict[str, PrimFunc] = dict(functions)
        self.attrs = dict(attrs or {})

    def functions_items(self):
        return list(self.functions.items())

    def __getitem__(self, name: str) -> PrimFunc:
        return self.functions[name]


class FuncInfo:
    """What the tuner needs to know about one PrimFunc."""

    def __init__(self, func: PrimFunc, name: Optional[str] = None):
        self.func = func
        self.name = name or func.name
        self.dynamic_args = func.dynamic_args
        self.kind = self.get_func_kind()
        self.in_dtype = func.params[0].dtype
        self.out_dtype = func.params[-1].dtype
        self.use_fp16 = any(p.dtype == "float16" for p in func.params)
        out = func.params[-1]
        # static element count (product of the constant extents of the output)
        self.num_elements = 1
        for e in out.shape:
            if isinstance(e, int):
                self.num_elements *= e
        self.red_len, self.rows, self.dyn_red = self._reduction_shape()

    def get_func_kind(self) -> FuncKind:
        """GEMM: a reduction block reading two operands whose output keeps a spatial extent from
        each; GEMV: the same with a single output row; Reduction: any other block with an "R"
        iterator; Elementwise: spatial iterators only."""
        red_blocks = [b for b in self.func.blocks if "R" in b.iter_kinds]
        if not red_blocks:
            return FuncKind.kFunc_Elementwise
        b = red_blocks[0]
        if self.func.op in ("attn_scores", "attn_pv"):      # batched matmuls over the heads
            return FuncKind.kFunc_GEMM
        if self.func.op in ("matmul", "gemv_q8", "gemv_q8_f32", "gemm_q8", "gemv_f32") and len(b.reads) == 2:
            lhs = next(p for p in self.func.params if p.name == b.reads[0])
            rows = 1
            for e in lhs.shape[:-1]:
                rows = rows * e if isinstance(e, int) and isinstance(rows, int) else "dyn"
            return FuncKind.kFunc_GEMV if rows == 1 else FuncKind.kFunc_GEMM
        return FuncKind.kFunc_Reduction

    def _reduction_shape(self):
        if self.kind != FuncKind.kFunc_Reduction:
            return None, None, False
        x = self.func.params[0]
        red = x.shape[-1]
        rows = 1
        for e in x.shape[:-1]:
            if isinstance(e, int):
                rows *= e
        if isinstance(red, str):
            return Var(red), rows, True
        return red, rows, False

"""Runtime module: the object ``Engine.tune_module`` returns and ``load_module_from_file`` reloads.

In the reference ``RuntimePacker`` writes the spliced host C and the kernels to ``work_dir``, builds
``host.so`` + ``tvm_device.cubin`` and returns a ``tvm.runtime.Module`` whose functions are called as
``rt_mod["add"](A, B, out)`` (python/dtas/codegen/runtime_packer.py:43-258);
``load_module_from_file(work_dir)`` reloads the two files (:260-283).  Here the kernels already live
in libdtas_gfx950.so, so what is packed is only the dispatcher's data -- per function the call
table, the index table and the index statement -- written to ``work_dir/dispatch_table.json`` (and,
for C callers, as ``dispatch_tables.h``).  ``RuntimeModule.__getitem__`` returns the function's host
side: read the dynamic extents from the argument shapes, ``index = min(n / div, last)``,
``info = call_table[index_table[index]]``, launch (the statements of
experiment/dtas_tuned/elementwise/add/float16/top1_256/host.cc:105-143).
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional, Sequence, Tuple

from .. import _lib, ops
from ..common.analisys import Block, Buffer, FuncInfo, FuncKind, PrimFunc
from ..common.config import Config, Range, config_from_dict

TABLE_FILE = "dispatch_table.json"
HEADER_FILE = "dispatch_tables.h"

_TORCH_DTYPES = None


def _torch_dtype(name: str):
    global _TORCH_DTYPES
    if _TORCH_DTYPES is None:
        import torch

        _TORCH_DTYPES = {"float16": torch.float16, "float32": torch.float32, "int8": torch.int8, "uint32": torch.uint32,
                         "int32": torch.int32}
    return _TORCH_DTYPES[name]


def op_id_of(func: PrimFunc) -> int:
    """The C library's op id for a PrimFunc descriptor."""
    dt_in, dt_out = func.params[0].dtype, func.params[-1].dtype
    sfx = {"float16": "F16", "float32": "F32", "int8": "I8"}
    if func.op in ("add", "copy"):
        return getattr(_lib, f"OP_{func.op.upper()}_{sfx[dt_in]}")
    if func.op == "cast":
        return getattr(_lib, f"OP_CAST_{sfx[dt_in]}_{sfx[dt_out]}")
    if func.op == "layer_norm":
        return _lib.OP_LAYER_NORM_F32_F16
    if func.op == "rms_norm":
        return _lib.OP_RMS_NORM_F16
    if func.op == "softmax":
        return _lib.OP_SOFTMAX_F16 if dt_in == "float16" else _lib.OP_SOFTMAX_F32_F16
    if func.op == "matmul":
        return _lib.OP_GEMV_F16 if FuncInfo(func).kind == FuncKind.kFunc_GEMV else _lib.OP_GEMM_F16
    raise ValueError(f"no kernel family for op {func.op!r}")


# PrimFuncs the tuner does not search: the library picks their kernel and launch shape per call
LIBRARY_CHOSEN_OPS = ("attn_scores", "attn_pv", "decode_q8", "take", "take_q8", "gemv_q8", "gemv_q8_f32", "gemm_q8", "gemv_f32",
                      "split3", "swap_axes", "softmax_temperature", "divide", "softmax_f32", "layer_norm_f32")


def _concrete(shape, values: Dict[str, int]) -> Tuple[int, ...]:
    return tuple(values[e] if isinstance(e, str) else e for e in shape)


def extents_of(func: PrimFunc, values: Dict[str, int]) -> Tuple[int, int, int]:
    """(n, d0, d1) as dtas_select_bucket / dtas_describe_launch take them."""
    first = _concrete(func.params[0].shape, values)
    if func.op in ("add", "copy", "cast"):
        H = first[-1]
        total = 1
        for e in first:
            total *= e
        return total // H if H else 0, H, 0
    if func.op in ("layer_norm", "rms_norm"):
        H = first[-1]
        rows = 1
        for e in first[:-1]:
            rows *= e
        return rows, H, 0
    if func.op == "softmax":
        cols = first[-1]
        rows = 1
        for e in first[:-1]:
            rows *= e
        return cols, rows, cols
    if func.op == "matmul":
        N, K = func.params[1].shape
        M = 1
        for e in first[:-1]:
            M *= e
        return M, N, K
    raise ValueError(func.op)


def bind_extents(func: PrimFunc, tensors: Sequence) -> Dict[str, int]:
    """Checks the arguments against the signature and reads the dynamic extents from the shapes
    (the generated host reads ``n`` from ``shape[1]`` of the first buffer, host.cc:54-55)."""
    if len(tensors) != len(func.params):
        raise TypeError(f"{func.name} takes {len(func.params)} buffers ({', '.join(p.name for p in func.params)}), "
                        f"got {len(tensors)}")
    values: Dict[str, int] = {}
    for buf, t in zip(func.params, tensors):
        # (a uint32 buffer is also accepted as int32: the same words, and the dtype torch is fluent in)
        if t.dtype != _torch_dtype(buf.dtype) and not (buf.dtype == "uint32" and str(t.dtype) == "torch.int32"):
            raise TypeError(f"{func.name}: buffer {buf.name} is {buf.dtype}, got {t.dtype}")
        if t.dim() != len(buf.shape):
            raise ValueError(f"{func.name}: buffer {buf.name} has {len(buf.shape)} dims, got shape {tuple(t.shape)}")
        for e, actual in zip(buf.shape, t.shape):
            if isinstance(e, str):
                if values.setdefault(e, int(actual)) != int(actual):
                    raise ValueError(f"{func.name}: extent {e} is {values[e]} and {actual} in different buffers")
            elif int(actual) != e:
                raise ValueError(f"{func.name}: buffer {buf.name} expects shape {buf.shape}, got {tuple(t.shape)}")
    return values


def call_primfunc(func: PrimFunc, tensors: Sequence, abi: Optional[_lib.DtasConfig] = None) -> None:
    """Enqueue one call of ``func`` on the given buffers with an explicit call-table row (or the
    library's built-in table when ``abi`` is None)."""
    op = func.op
    if op == "add":
        ops.add(tensors[0], tensors[1], tensors[2], abi)
    elif op == "copy":
        ops.copy(tensors[0], tensors[1], abi)
    elif op == "cast":
        ops.cast(tensors[0], tensors[1], abi)
    elif op == "layer_norm":
        ops.layer_norm(tensors[0], tensors[1], tensors[2], tensors[3], func.attrs.get("eps", 1e-5), abi)
    elif op == "rms_norm":
        ops.rms_norm(tensors[0], tensors[1], tensors[2], func.attrs.get("eps", 1e-5), abi)
    elif op == "softmax":
        ops.softmax(tensors[0], tensors[1], abi)
    elif op == "attn_scores":                                                 # Q, K, mask, out
        ops.attn_scores(tensors[0], tensors[1], tensors[2], tensors[3], func.attrs.get("scale", 0.11179039301310044), abi)
    elif op == "attn_pv":                                                     # P, V, out
        ops.attn_pv(tensors[0], tensors[1], tensors[2], abi)
    elif op == "gemv_f32":                                                    # x, W, y
        ops.gemv_f32(tensors[0], tensors[1], tensors[2], abi)
    elif op == "decode_q8":                                                   # Wq, scale, W
        ops.decode_q8(tensors[0], tensors[1], tensors[2], abi)
    elif op == "take":                                                        # A, ids, out
        ops.take(tensors[0], tensors[1], tensors[2], abi)
    elif op == "split3":                                                      # A, three sections
        heads, d = int(func.attrs["heads"]), int(func.attrs["d"])
        ops.split3(tensors[0].view(-1, heads, 3 * d), tensors[1], tensors[2], tensors[3])
    elif op == "swap_axes":                                                   # A, out
        ops.swap_axes(tensors[0], tensors[1])
    elif op == "layer_norm_f32":                                              # A, gamma, beta, out
        ops.layer_norm_f32(tensors[0], tensors[1], tensors[2], tensors[3], func.attrs.get("eps", 1e-5))
    elif op == "divide":                                                      # A, B (0-d), out
        ops.divide(tensors[0], tensors[1], tensors[2])
    elif op == "softmax_f32":                                                 # A, out
        ops.softmax_f32(tensors[0], tensors[1])
    elif op == "softmax_temperature":                                         # logits, temperature, out
        ops.softmax_temperature(tensors[0], tensors[1], tensors[2])
    elif op == "take_q8":                                                     # Wq, scale, ids, out
        ops.take_q8(tensors[0], tensors[1], tensors[2], tensors[3], abi)
    elif op == "gemv_q8_f32":                                                 # Wq, scale, x, y
        ops.gemv_q8_f32(tensors[2], tensors[0], tensors[1], tensors[3], abi)
    elif op == "gemm_q8":                                                     # Wq, scale, A, bias, out; n dynamic
        ops.gemm_q8(tensors[2], tensors[0], tensors[1], tensors[3], tensors[4], abi, int(func.attrs.get("epilogue", 0)))
    elif op == "gemv_q8":                                                     # Wq, scale, x, bias, y
        ops.gemv_q8(tensors[2], tensors[0], tensors[1], tensors[3], tensors[4], abi, int(func.attrs.get("epilogue", 0)))
    elif op == "matmul":
        epilogue = int(func.attrs.get("epilogue", 0))
        mm = ops.gemv if FuncInfo(func).kind == FuncKind.kFunc_GEMV else ops.gemm   # one static row: the decode forms
        if epilogue in (_lib.EPI_BIAS_ADD2, _lib.EPI_BIAS_ADD2_CAST_F32):   # A, W, bias, res1, res2, out
            mm(tensors[0], tensors[1], tensors[2], tensors[5], abi, epilogue=epilogue, res1=tensors[3], res2=tensors[4])
        elif epilogue == _lib.EPI_BIAS_GELU:                                  # A, W, bias, out
            mm(tensors[0], tensors[1], tensors[2], tensors[3], abi, epilogue=epilogue)
        else:
            bias = tensors[2] if len(tensors) == 4 else None
            if FuncInfo(func).kind == FuncKind.kFunc_GEMV:
                ops.gemv(tensors[0], tensors[1], bias, tensors[-1], abi)
            else:
                ops.gemm(tensors[0], tensors[1], bias, tensors[-1], abi)
    else:
        raise ValueError(f"no kernel family for op {op!r}")


# ---- (de)serialisation of PrimFunc descriptors ----------------------------------------------
def _func_to_json(f: PrimFunc) -> dict:
    return {"name": f.name, "op": f.op, "attrs": {k: v for k, v in f.attrs.items() if k != "tir_var_upper_bound"},
            "params": [{"name": b.name, "shape": list(b.shape), "dtype": b.dtype} for b in f.params],
            "blocks": [{"name": b.name, "iter_kinds": b.iter_kinds, "reads": list(b.reads), "writes": list(b.writes)}
                       for b in f.blocks]}


def _func_from_json(d: dict) -> PrimFunc:
    return PrimFunc(d["name"], [Buffer(p["name"], tuple(p["shape"]), p["dtype"]) for p in d["params"]],
                    [Block(b["name"], b["iter_kinds"], b["reads"], b["writes"]) for b in d["blocks"]], op=d["op"],
                    attrs=dict(d.get("attrs", {})))


class KernelEntryInfo:
    """One call-table row: merged bucket ranges, config and the launch arguments at the upper end
    (the reference's ``kernel_entry_info``, python/dtas/codegen/runtime_packer.py:32-40)."""

    def __init__(self, ranges: Sequence[Range], config: Config, name: str, launch_args: Sequence[int]):
        self.ranges = list(ranges)
        self.config = config
        self.abi = config.to_abi()
        self.name = name
        self.launch_args = list(launch_args)

    def to_json(self) -> dict:
        return {"ranges": [[r.var.name, r.start, r.end] for r in self.ranges], "config_kind": self.config.config_kind,
                "config": self.config.to_dict(), "abi": self.abi.to_dict(), "name": self.name,
                "launch_args": self.launch_args}

    @classmethod
    def from_json(cls, d: dict) -> "KernelEntryInfo":
        cfg = config_from_dict(d["config_kind"], d["config"])
        entry = cls([Range(v, lo, hi) for v, lo, hi in d["ranges"]], cfg, d["name"], d["launch_args"])
        entry.abi = _lib.DtasConfig.from_dict(d["abi"])  # the row as tuned, not re-derived
        return entry


class FunctionTable:
    """Dispatcher data of one function."""

    def __init__(self, func: PrimFunc, call_table: List[KernelEntryInfo], index_table: List[int],
                 range_div_factor: int, upper_bound: Dict[str, int]):
        self.func = func
        self.call_table = call_table
        self.index_table = index_table
        self.range_div_factor = range_div_factor
        self.upper_bound = dict(upper_bound)
        self.dynamic_args = [v.name for v in func.dynamic_args]

    def index(self, values: Dict[str, int]) -> int:
        """The reference's index statement (python/dtas/engine/tuner.py:166-208): C integer
        division of each dynamic extent by the bucket width, clamped to the table's last slot.
        With two extents the row stride is the second extent's bucket count."""
        div = self.range_div_factor
        if not self.dynamic_args or not self.index_table:
            return 0
        sizes = [-(-self.upper_bound[a] // div) for a in self.dynamic_args]
        if len(self.dynamic_args) == 1:
            idx = values[self.dynamic_args[0]] // div
        else:
            a, b = self.dynamic_args[:2]
            idx = min(values[a] // div, sizes[0] - 1) * sizes[1] + min(values[b] // div, sizes[1] - 1)
        return min(idx, len(self.index_table) - 1)

    def index_stmt(self) -> str:
        div = self.range_div_factor
        last = len(self.index_table) - 1
        if not self.dynamic_args or not self.index_table:
            return "  int64_t index = 0;\n"
        if len(self.dynamic_args) == 1:
            a = self.dynamic_args[0]
            return f"  int64_t index = ({a}/{div}) > {last} ? {last} : {a}/{div};\n"
        a, b = self.dynamic_args[:2]
        s1 = -(-self.upper_bound[b] // div)
        expr = f"({a}/{div} * {s1} + {b}/{div})"
        return f"  int64_t index = {expr} > {last} ? {last} : {expr};\n"

    def select_function_text(self, name: str) -> List[str]:
        """C text of ``<name>_select(extents...)``: what select() does, for C callers of the generated
        header -- the index statement behind a guard that returns NULL (the library sizes the launch
        itself) for any extent above its upper bound, so both dispatchers run the same thing there."""
        args = [a for a in self.dynamic_args[:2]]
        if not args or not self.index_table or not self.call_table:
            body = f"  return {'&' + name + '_call_table[0]' if self.call_table else '0'};"
            return [f"static inline const dtas_config* {name}_select(void) {{", body, "}"]
        params = ", ".join(f"int64_t {a}" for a in args)
        guard = " || ".join(f"{a} > {self.upper_bound[a]}" for a in args if a in self.upper_bound)
        lines = [f"static inline const dtas_config* {name}_select({params}) {{"]
        if guard:
            lines.append(f"  if ({guard}) return 0;  /* above the tuned range: cfg = NULL, the library's own choice */")
        if len(args) == 2:   # each extent's bucket is clamped on its own before the two are combined
            div = self.range_div_factor
            sizes = [-(-self.upper_bound[a] // div) for a in args]
            a, b = args
            lines.append(f"  int64_t ia = {a}/{div} > {sizes[0] - 1} ? {sizes[0] - 1} : {a}/{div}, ib = {b}/{div} > {sizes[1] - 1} ? {sizes[1] - 1} : {b}/{div};")
            last = len(self.index_table) - 1
            lines.append(f"  int64_t index = ia * {sizes[1]} + ib > {last} ? {last} : ia * {sizes[1]} + ib;")
        else:
            lines.append(self.index_stmt().rstrip("\n"))
        lines.append(f"  return &{name}_call_table[{name}_index_table[index]];")
        lines.append("}")
        return lines

    def select(self, values: Dict[str, int]) -> Optional[KernelEntryInfo]:
        """The row for these extents, or None where the library sizes the launch itself: a
        function without tuned rows, and any extent above its upper bound.  The reference runs the
        last bucket's predicated kernel there (python/dtas/engine/tuner.py:166-208 clamps the
        index); a row here was validated only up to its bucket's end and may not fit a larger
        extent (rows per wavefront, a skinny tile), while the library's own choice fits any."""
        if not self.call_table:      # a function whose launch shape the library chooses itself
            return None
        if any(values[a] > self.upper_bound[a] for a in self.dynamic_args if a in self.upper_bound):
            return None
        if not self.index_table:
            return self.call_table[0]
        return self.call_table[self.index_table[self.index(values)]]

    def to_json(self) -> dict:
        return {"primfunc": _func_to_json(self.func), "range_div_factor": self.range_div_factor,
                "upper_bound": self.upper_bound, "dynamic_args": self.dynamic_args,
                "call_table": [e.to_json() for e in self.call_table], "index_table": self.index_table,
                "index_stmt": self.index_stmt()}

    @classmethod
    def from_json(cls, d: dict) -> "FunctionTable":
        return cls(_func_from_json(d["primfunc"]), [KernelEntryInfo.from_json(e) for e in d["call_table"]],
                   list(d["index_table"]), d["range_div_factor"], d["upper_bound"])


class TimingResult:
    """What ``time_evaluator(...)(*args)`` returns: ``.mean`` in seconds, like TVM's."""

    def __init__(self, results: List[float]):
        self.results = results
        self.mean = sum(results) / len(results)
        self.min = min(results)
        self.max = max(results)

    def __repr__(self):
        return f"TimingResult(mean={self.mean:.3e} s, n={len(self.results)})"


class RuntimeModule:
    """``rt_mod[name](*buffers)`` launches; ``rt_mod.time_evaluator(name, dev, number, min_repeat_ms)``
    times (experiment/dtas_tuned/elementwise/add/profile_add.py:8-9,26)."""

    def __init__(self, tables: Dict[str, FunctionTable], work_dir: Optional[str] = None):
        self.tables = tables
        self.work_dir = work_dir
        _lib.lib()  # fail now, not at the first call, if the kernels are not built

    def __getitem__(self, name: str):
        table = self.tables[name]

        def packed_func(*tensors):
            values = bind_extents(table.func, tensors)
            entry = table.select(values)
            call_primfunc(table.func, tensors, entry.abi if entry is not None else None)

        packed_func.__name__ = name
        return packed_func

    def get_function(self, name: str):
        return self[name]

    def entry_for(self, name: str, **values: int) -> Optional[KernelEntryInfo]:
        """Which call-table row a call with these dynamic extents uses (None: the library's own choice)."""
        return self.tables[name].select(values)

    def time_evaluator(self, func_name: str, dev=None, number: int = 10, repeat: int = 1, min_repeat_ms: float = 0):
        import torch

        fn = self[func_name]

        def evaluator(*tensors) -> TimingResult:
            fn(*tensors)
            torch.cuda.synchronize(dev)
            results = []
            for _ in range(repeat):
                n = number
                while True:
                    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    start.record()
                    for _ in range(n):
                        fn(*tensors)
                    stop.record()
                    stop.synchronize()
                    ms = start.elapsed_time(stop)
                    if ms >= min_repeat_ms or n >= (1 << 20):
                        break
                    n = max(n + 1, int(n * max(1.5, min_repeat_ms / max(ms, 1e-3))))
                results.append(ms * 1e-3 / n)
            return TimingResult(results)

        return evaluator


class RuntimePacker:
    """Writes the dispatcher data to ``work_dir`` and returns the runtime module."""

    def __init__(self, tables: Dict[str, FunctionTable], work_dir: str):
        self.tables = tables
        self.work_dir = work_dir

    def header_text(self) -> str:
        out = ["/* Generated dispatcher tables (same information as dispatch_table.json) for C callers:",
               " * <func>_select(extents) returns the row for these extents -- index with the index statement, then",
               " * &<func>_call_table[<func>_index_table[index]] -- or NULL above the tuned range; pass it as the `cfg`",
               " * argument of the entry point in dtas_abi.h. */", '#include "dtas_abi.h"', ""]
        for name, t in self.tables.items():
            rows = []
            for e in t.call_table:
                a = e.abi
                rows.append(f"  /* {e.name} */ {{{a.variant}, {a.block}, {a.vec}, {a.unroll}, "
                            f"{{{a.tile[0]}, {a.tile[1]}, {a.tile[2]}}}, {a.split_k}, {a.grid_cap}}},")
            out.append(f"static const dtas_config {name}_call_table[] = {{")
            out += rows
            out.append("};")
            idx = ",".join(str(i) for i in t.index_table) or "0"
            out.append(f"static const int64_t {name}_index_table[] = {{{idx}}};")
            out.append(f"/* {t.index_stmt().strip()} */")
            out += t.select_function_text(name)
            out.append("")
        return "\n".join(out)

    def pack_to_runtime(self) -> RuntimeModule:
        os.makedirs(self.work_dir, exist_ok=True)
        doc = {"format": "dtas_amd.dispatch_table/1", "library": os.path.basename(_lib.LIB_PATH),
               "functions": {name: t.to_json() for name, t in self.tables.items()}}
        with open(os.path.join(self.work_dir, TABLE_FILE), "w") as f:
            json.dump(doc, f, indent=2)
        with open(os.path.join(self.work_dir, HEADER_FILE), "w") as f:
            f.write(self.header_text())
        return RuntimeModule(self.tables, self.work_dir)

    # the reference's method name
    pack_to_tvm_runtime = pack_to_runtime


def load_module_from_file(work_dir: str) -> RuntimeModule:
    """Reload a tuned module from ``work_dir`` (python/dtas/codegen/runtime_packer.py:260-283)."""
    if not os.path.exists(work_dir):
        raise FileNotFoundError(f"Directory {work_dir} not found.")
    path = os.path.join(work_dir, TABLE_FILE)
    if not os.path.exists(path):
        raise FileNotFoundError(f"{TABLE_FILE} not found in the specified directory.")
    with open(path) as f:
        doc = json.load(f)
    tables = {name: FunctionTable.from_json(d) for name, d in doc["functions"].items()}
    return RuntimeModule(tables, work_dir)

"""Bucket ranges and per-family launch configs.

Same vocabulary as the reference (python/dtas/common/config.py): ``Range`` with ``to_suffix`` /
``merge`` (:21-61), ``generate_range_list`` (:64-78), ``Config`` equality by ``to_dict`` (:97-127) and
one config class per function kind.  The fields are the gfx950 launch parameters (what a row of the
C call table holds, ``struct dtas_config``), not CUDA schedule knobs.
"""
from __future__ import annotations

import json
from typing import Dict, List, Union

from .. import _lib


class Var:
    """A symbolic extent (the reference uses tir.Var); identity is the name."""

    def __init__(self, name: str, dtype: str = "int64"):
        self.name = name
        self.dtype = dtype

    def __eq__(self, other):
        return isinstance(other, Var) and other.name == self.name

    def __hash__(self):
        return hash(("Var", self.name))

    def __repr__(self):
        return self.name


class Range:
    """Closed range [start, end] of one dynamic extent: one bucket (or several merged ones)."""

    def __init__(self, var: Union[Var, str], start: int, end: int) -> None:
        self.var = var if isinstance(var, Var) else Var(var)
        self.start = int(start)
        self.end = int(end)
        self.tuned = False

    def to_suffix(self) -> str:
        # kernel-name suffix, e.g. "_n_1_to_256_" -> add_n_1_to_256__kernel
        return "_" + self.var.name + "_" + str(self.start) + "_to_" + str(self.end) + "_"

    def merge(self, other: "Range") -> "Range":
        """Union with an adjacent range of the same variable; ValueError otherwise."""
        if self.var.name != other.var.name:
            raise ValueError("can not merge different var")
        if self.end == other.start - 1:
            return Range(self.var, self.start, other.end)
        if self.start == other.end + 1:
            return Range(self.var, other.start, self.end)
        raise ValueError("can not merge non-adjacent ranges")

    def __repr__(self) -> str:
        return f"<{self.var.name}: Range({self.start}, {self.end})>"

    __str__ = __repr__

    def __eq__(self, o) -> bool:
        return isinstance(o, Range) and self.var == o.var and self.start == o.start and self.end == o.end

    def __hash__(self) -> int:
        return hash((self.var, self.start, self.end))


def generate_range_list(var: Union[Var, str], start: int, end: int, div_factor: int) -> List[Range]:
    """[start, start+div-1], [start+div, ...] while start < end; one bucket if end-start <= div."""
    assert start < end
    assert div_factor > 0
    if end - start <= div_factor:
        return [Range(var, start, start + div_factor - 1)]
    ranges = []
    while start < end:
        ranges.append(Range(var, start, start + div_factor - 1))
        start += div_factor
    return ranges


class Config:
    """Base: two configs are the same kernel iff their dicts agree (used when merging buckets)."""

    config_kind = "Config"

    def to_dict(self) -> Dict:
        raise NotImplementedError

    def from_dict(self, dic: Dict) -> "Config":
        raise NotImplementedError

    def to_abi(self) -> "_lib.DtasConfig":
        """The C-side call-table row for this config."""
        raise NotImplementedError

    def __repr__(self) -> str:
        return str(self.to_dict())

    def __str__(self) -> str:
        return self.config_kind + ": " + str(self.to_dict())

    def __hash__(self):
        return hash(json.dumps(self.to_dict(), sort_keys=True).encode())

    def __eq__(self, other):
        if not isinstance(other, Config):
            return False
        mine, theirs = self.to_dict(), other.to_dict()
        return all(k in theirs and theirs[k] == v for k, v in mine.items())


class ElementwiseConfig(Config):
    config_kind = "ElementwiseConfig"

    def __init__(self) -> None:
        self.len_tx = 256       # threads per workgroup, fixed
        self.vector_size = 4    # elements per access
        self.grid_size = 4      # workgroups for the bucket's upper end (informational, like the reference's)
        self.unroll_depth = 0   # accesses in flight per thread (1, 2, 4, 8); 0 = reference artefact
        self.scalar = False     # element accesses, any alignment

    def to_dict(self) -> Dict:
        return {"len_tx": self.len_tx, "vector_size": self.vector_size, "grid_size": self.grid_size,
                "unroll_depth": self.unroll_depth}

    def from_dict(self, dic: Dict) -> "ElementwiseConfig":
        self.__init__()
        self.len_tx = dic["len_tx"]
        self.vector_size = dic["vector_size"]
        self.grid_size = dic["grid_size"]
        self.unroll_depth = dic["unroll_depth"]
        return self

    def to_abi(self):
        c = _lib.DtasConfig()
        c.variant = _lib.ELT_SCALAR if self.scalar else _lib.ELT_VECTOR
        c.block, c.vec = self.len_tx, self.vector_size
        c.unroll = self.unroll_depth if self.unroll_depth in (1, 2, 4, 8) else 1
        c.split_k, c.grid_cap = 1, 0
        return c


class ReductionConfig(Config):
    config_kind = "ReductionConfig"

    def __init__(self) -> None:
        self.bx = None
        self.bx_factor = 1
        self.len_tx = 128
        self.unroll_depth = 256
        self.vector_size = 4
        # where the row lives between the passes: "local" = registers, one wavefront per row;
        # "shared.dyn" = registers + LDS staging of partials, one workgroup per row;
        # "cache" = re-read from L2 per pass (the reference's softmax artefacts)
        self.temp_storage = "shared.dyn"
        self.max_active_blocks_per_sm = 0
        # rows a wavefront / workgroup takes per trip (1, 2, 4): they share barriers and parameter loads
        self.rows_per_trip = 1

    def to_dict(self) -> Dict:
        return {"bx": self.bx, "len_tx": self.len_tx, "unroll_depth": self.unroll_depth,
                "vector_size": self.vector_size, "temp_storage": self.temp_storage,
                "max_active_blocks_per_sm": self.max_active_blocks_per_sm, "rows_per_trip": self.rows_per_trip}

    def from_dict(self, dic: Dict) -> "ReductionConfig":
        self.__init__()
        self.len_tx = dic["len_tx"]
        self.unroll_depth = dic["unroll_depth"]
        self.vector_size = dic["vector_size"]
        self.temp_storage = dic["temp_storage"]
        self.bx = dic.get("bx")
        self.max_active_blocks_per_sm = dic.get("max_active_blocks_per_sm", 0)
        self.rows_per_trip = dic.get("rows_per_trip", 1)
        return self

    def to_abi(self):
        c = _lib.DtasConfig()
        c.variant = {"local": _lib.RED_WAVE_ROW, "shared.dyn": _lib.RED_BLOCK_ROW,
                     "cache": _lib.RED_STREAM_ROW}[self.temp_storage]
        c.block = self.len_tx
        c.vec = 1 if self.temp_storage == "cache" else (self.vector_size or 1)
        c.unroll, c.split_k = (1 if self.temp_storage == "cache" else self.rows_per_trip), 1
        c.grid_cap = self.bx or 0
        return c


class GEMVConfig(Config):
    config_kind = "GEMVConfig"

    def __init__(self) -> None:
        self.TS = 1            # wavefront rows of threads along the spatial axis (kept for vocabulary)
        self.TILE_S = 4        # rows of W per workgroup
        self.TR = 256          # threads splitting K
        self.TILE_R = 8
        self.VEC_C = 8         # fp16 elements per 128-bit access
        self.TAG_S, self.TAG_R = "blockIdx.x", "threadIdx.x"
        self.LOAD_V_SHARED = False
        self.LOAD_V_VEC = 8
        self.UNROLL = 2
        # every sum in fp16, in the order of the reference's scheduled kernel (TS x TR = 16 x 32 threads there:
        # 32 threads x 8 chains per row, experiment/testIR/GEMV/m1n2560k10240/IR/5wt.py:11-92)
        self.ACC_F16 = False

    def to_dict(self) -> Dict:
        return {"acc_f16": self.ACC_F16, "sapctial_thread": self.TS, "sapctial_tile": self.TILE_S, "reduction_thread": self.TR,
                "reduction_tile": self.TILE_R, "vec_c": self.VEC_C, "tag_s": self.TAG_S, "tag_r": self.TAG_R,
                "load_v_shared": self.LOAD_V_SHARED, "load_v_vec": self.LOAD_V_VEC, "unroll_factor": self.UNROLL}

    def from_dict(self, dic: Dict) -> "GEMVConfig":
        self.__init__()
        self.TS, self.TILE_S = dic["sapctial_thread"], dic["sapctial_tile"]
        self.TR, self.TILE_R, self.VEC_C = dic["reduction_thread"], dic["reduction_tile"], dic["vec_c"]
        self.UNROLL = dic.get("unroll_factor", 2)
        self.ACC_F16 = dic.get("acc_f16", False)
        return self

    def to_abi(self):
        c = _lib.DtasConfig()
        c.variant, c.block, c.vec, c.unroll = _lib.GEMV_SPLITK, self.TR, self.VEC_C, self.UNROLL
        c.tile[0] = self.TILE_S
        if self.ACC_F16:   # half a wavefront per row, 8 rows per workgroup of 256
            c.variant, c.block, c.tile[0] = _lib.GEMV_RF16, 256, 8
        c.split_k = 1
        return c


class MFMAConfig(Config):
    """GEMM tile config; sits where the reference has WMMAConfig (config.py:193-294): i x j
    wavefronts, each micro_shape_x x micro_shape_y matrix-core blocks, k tile micro_shape_k blocks."""

    config_kind = "MFMAConfig"

    def __init__(self) -> None:
        self.i = 2
        self.j = 2
        self.micro_shape_x = 4
        self.micro_shape_y = 4
        self.micro_shape_k = 4
        self.mfma_m, self.mfma_n, self.mfma_k = 32, 32, 16
        self.skinny = False      # small M: weight-streaming 16x16x32 kernel, K split over wavefronts
        self.stream = False      # M <= 64: W streamed through the LDS in 1 KiB row pieces, K sliced over workgroups
        self.block_threads = 256
        self.stages = 0          # LDS stages of the load pipeline (0 = as many as the tile allows)
        self.split_k = 1         # workgroups that share a tile and split its K extent
        # the reference's scheduled arithmetic: an fp16 accumulator rounded once per k step of 16 (its wmma 16x16x16
        # fragments with a float16 accumulator, experiment/testIR/GEMM/m_n2560_k10240/wmma/16x16x16/i2j4_x7y2_in8.py:19,37)
        self.acc_f16 = False
        self.in_vec_len_a = 8
        self.in_vec_len_b = 8
        self.swizzle = True
        self.performance = 0.0   # analytical score that ranked this candidate
        self.num_wave = 0

    @property
    def tile_size_m(self):
        return self.i * self.micro_shape_x * self.mfma_m

    @property
    def tile_size_n(self):
        return self.j * self.micro_shape_y * self.mfma_n

    @property
    def tile_size_k(self):
        return self.micro_shape_k * self.mfma_k

    def to_dict(self) -> Dict:
        return {"tile_shape": (self.tile_size_m, self.tile_size_n, self.tile_size_k),
                "mfma_shape": (self.mfma_m, self.mfma_n, self.mfma_k), "i": self.i, "j": self.j,
                "micro_shape": (self.micro_shape_x, self.micro_shape_y, self.micro_shape_k),
                "skinny": self.skinny, "stream": self.stream, "block_threads": self.block_threads, "stages": self.stages,
                "split_k": self.split_k, "acc_f16": self.acc_f16, "in_vec_len_a": self.in_vec_len_a, "in_vec_len_b": self.in_vec_len_b}

    def from_dict(self, dic: Dict) -> "MFMAConfig":
        self.__init__()
        self.mfma_m, self.mfma_n, self.mfma_k = dic["mfma_shape"]
        self.i, self.j = dic["i"], dic["j"]
        self.micro_shape_x, self.micro_shape_y, self.micro_shape_k = dic["micro_shape"]
        self.skinny = dic.get("skinny", False)
        self.stream = dic.get("stream", False)
        self.block_threads = dic.get("block_threads", 256)
        self.stages = dic.get("stages", 0)
        self.split_k = dic.get("split_k", 1)
        self.acc_f16 = dic.get("acc_f16", False)
        return self

    def to_abi(self):
        c = _lib.DtasConfig()
        if self.acc_f16:   # one kernel shape: 64x64 per workgroup, a k step of 16 per instruction
            c.variant, c.block, c.vec, c.unroll, c.split_k = _lib.GEMM_MFMA_ACC16, 256, 8, 1, 1
            c.tile[0], c.tile[1], c.tile[2] = 64, 64, 16
            return c
        c.variant = _lib.GEMM_SKINNY if self.skinny else _lib.GEMM_STREAM if self.stream else _lib.GEMM_MFMA
        c.block, c.vec = self.block_threads, 8
        c.unroll = 4 if self.skinny else 1 if self.stream else self.stages
        c.tile[0], c.tile[1], c.tile[2] = self.tile_size_m, self.tile_size_n, self.tile_size_k
        c.split_k = 1 if self.skinny or self.stream else self.split_k
        return c


# the reference's name for the GEMM config slot
WMMAConfig = MFMAConfig


def config_from_dict(kind: str, dic: Dict) -> Config:
    cls = {"ElementwiseConfig": ElementwiseConfig, "ReductionConfig": ReductionConfig, "GEMVConfig": GEMVConfig,
           "MFMAConfig": MFMAConfig, "WMMAConfig": MFMAConfig}[kind]
    return cls().from_dict(dic)

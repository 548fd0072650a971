"""dtas_amd: the GPU hot path of DTAS (dynamic-shape TIR PrimFunc kernels behind a shape-bucket
dispatcher) as hand-written gfx950 kernels in libdtas_gfx950.so, with the reference's Python entry
points on top: ``Engine.tune_module``, ``load_module_from_file``, ``rt_mod[name](*buffers)``."""
from . import arch, primfuncs
from .codegen.code_gen import CodeGenerator
from .codegen.runtime_packer import RuntimeModule, load_module_from_file
from .common.config import Config
from .engine.tuner import Engine
from .logging import get_log_level, set_log_level

__all__ = ["arch", "primfuncs", "CodeGenerator", "RuntimeModule", "load_module_from_file", "Config", "Engine",
           "get_log_level", "set_log_level"]

from .config import (Config, ElementwiseConfig, GEMVConfig, MFMAConfig, Range, ReductionConfig, Var, WMMAConfig,
                     generate_range_list)
from .analisys import Block, Buffer, FuncInfo, FuncKind, IRModule, PrimFunc

"""Base of the analytical config emitters (python/dtas/policy/base_config_emiter.py)."""
from typing import List, Tuple

from ..arch import Arch
from ..common.analisys import FuncInfo
from ..common.config import Config, Range


class BaseConfigEmiter:
    def __init__(self, func_info: FuncInfo, arch: Arch) -> None:
        self.func_info = func_info
        self.arch = arch

    def emit_config(self, range_tuple: Tuple[Range, ...], topk: int = 20) -> List[Config]:
        raise NotImplementedError


def dtype_bits(dtype: str) -> int:
    return {"int8": 8, "uint8": 8, "float16": 16, "bfloat16": 16, "float32": 32, "int32": 32, "float64": 64}[dtype]

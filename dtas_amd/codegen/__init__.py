from .code_gen import CodeGenerator
from .compile_result import CompileResult
from .runtime_packer import RuntimeModule, RuntimePacker, load_module_from_file

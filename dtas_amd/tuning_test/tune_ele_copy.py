"""Tune the elementwise copy PrimFunc over (1, n, 2560) (tuning_test/tune_ele_copy.py:10-41, fp32 in the
committed script).  Needs a GPU."""
import sys
import time

import torch

from dtas_amd import primfuncs as pf
from dtas_amd.arch import MI355X
from dtas_amd.engine.tuner import Engine


def main(dtype: str = "float32", work_dir: str = "/tmp/dtas_tuned/elementwise/copy/top10_256") -> None:
    mod = pf.module(pf.copy(dtype, 2560), upper_bound={"m": 512, "n": 4096})
    engine = Engine(10, parallel_build=True, work_dir=work_dir)
    start = time.time()
    rt_mod = engine.tune_module(mod, arch=MI355X(0, require_device=True), range_div_factor=256)
    print(f"tune copy : {time.time() - start} s")
    tdt = {"int8": torch.int8, "float16": torch.float16, "float32": torch.float32}[dtype]
    a = torch.rand(1, 300, 2560, device="cuda").to(tdt)
    b = torch.empty_like(a)
    rt_mod["copy"](a, b)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    print(rt_mod.time_evaluator(func_name="copy", number=5, min_repeat_ms=50)(a, b))


if __name__ == "__main__":
    main(*sys.argv[1:])

"""Tune the fp16 -> fp32 cast PrimFunc over (1, n, 2560), n <= 4096, and run it once.

The reference script of the same name (tuning_test/tune_cast.py:10-46) defines the PrimFunc in
TVMScript, tunes it with ``Engine(1, parallel_build=True, work_dir=...)`` for an RTX 3090 and prints
the elapsed tuning time.  Same flow here on an MI355X; needs a GPU."""
import sys
import time

import torch

from dtas_amd import primfuncs as pf
from dtas_amd.arch import MI355X
from dtas_amd.engine.tuner import Engine


def main(work_dir: str = "/tmp/dtas_tuned/cast/top1_256") -> None:
    mod = pf.module(pf.cast("float16", "float32", 2560), upper_bound={"m": 512, "n": 4096})
    engine = Engine(1, parallel_build=True, work_dir=work_dir)
    start = time.time()
    rt_mod = engine.tune_module(mod, arch=MI355X(0, require_device=True), range_div_factor=256)
    print(f"tune cast : {time.time() - start} s")
    x = torch.rand(1, 100, 2560, device="cuda").half()
    y = torch.empty(1, 100, 2560, device="cuda", dtype=torch.float32)
    rt_mod["cast"](x, y)
    timer = rt_mod.time_evaluator(func_name="cast", number=5, min_repeat_ms=50)
    print(timer(x, y))
    assert torch.equal(y, x.float())


if __name__ == "__main__":
    main(*sys.argv[1:])

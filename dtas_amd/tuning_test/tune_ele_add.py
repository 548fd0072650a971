"""Tune the elementwise add PrimFunc over (1, n, 2560) and sweep it (tuning_test/tune_ele_add.py:10-46;
the committed reference script is int8 and only lowers the function, the fp16 / fp32 / int8 artefacts
under experiment/dtas_tuned/elementwise/add/ came from the same flow with the Engine enabled).
Needs a GPU."""
import sys
import time

import torch

from dtas_amd import primfuncs as pf
from dtas_amd.arch import MI355X
from dtas_amd.engine.tuner import Engine


def main(dtype: str = "int8", work_dir: str = "/tmp/dtas_tuned/elementwise/add/top10_256") -> None:
    mod = pf.module(pf.add(dtype, 2560), upper_bound={"m": 512, "n": 4096})
    engine = Engine(10, parallel_build=True, work_dir=work_dir)
    start = time.time()
    rt_mod = engine.tune_module(mod, arch=MI355X(0, require_device=True), range_div_factor=256)
    print(f"tune add : {time.time() - start} s")
    tdt = {"int8": torch.int8, "float16": torch.float16, "float32": torch.float32}[dtype]
    timer = rt_mod.time_evaluator(func_name="add", number=5, min_repeat_ms=50)
    for n in (1, 16, 128, 1024, 4096):
        a = (torch.rand(1, n, 2560, device="cuda") * 100).to(tdt)
        b = (torch.rand(1, n, 2560, device="cuda") * 100).to(tdt)
        out = torch.empty_like(a)
        t = timer(a, b, out).mean
        nbytes = 3 * a.numel() * a.element_size()
        print(f"n={n}: {t * 1e6:.2f} us, {nbytes / t / 2 ** 30:.1f} GiB/s ({rt_mod.entry_for('add', n=n).name})")


if __name__ == "__main__":
    main(*sys.argv[1:])

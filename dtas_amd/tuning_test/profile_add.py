"""Sweep a tuned ``add`` module over n and write ``latency.json`` / ``bandwidth.json`` into its work_dir, in the
reference's format: {"<n>": microseconds} and {"<n>": GiB/s} (experiment/dtas_tuned/elementwise/add/profile_add.py:8-46).
Needs a GPU and a work_dir that ``tune_ele_add.py`` (or ``Engine.tune_module``) filled."""
import json
import os
import sys
from typing import Callable, Dict, Iterable, Sequence, Tuple

import torch

from dtas_amd.codegen.runtime_packer import RuntimeModule, load_module_from_file


def sweep(rt_mod: RuntimeModule, func_name: str, make_buffers: Callable[[int], Sequence[torch.Tensor]],
          bytes_moved: Callable[[int], int], n_values: Iterable[int], number: int = 5,
          min_repeat_ms: float = 50) -> Tuple[Dict[int, float], Dict[int, float]]:
    """(latency in us, bandwidth in GiB/s) per n, measured as the reference does: ``time_evaluator`` with
    ``number`` launches per sample and samples repeated until ``min_repeat_ms`` have passed."""
    timer = rt_mod.time_evaluator(func_name=func_name, number=number, min_repeat_ms=min_repeat_ms)
    latency, bandwidth = {}, {}
    for n in n_values:
        buffers = make_buffers(n)
        t = timer(*buffers).mean
        latency[n] = t * 1e6
        bandwidth[n] = bytes_moved(n) / (1024 * 1024 * 1024) / t
        del buffers
    return latency, bandwidth


def save_to_json(profile: Dict[int, float], filename: str) -> None:
    with open(filename, "w") as f:
        f.write(json.dumps(profile, indent=4))


def main(work_dir: str = "/tmp/dtas_tuned/elementwise/add/top10_256", dtype: str = "int8", upper: str = "4096") -> None:
    tdt = {"int8": torch.int8, "float16": torch.float16, "float32": torch.float32}[dtype]
    hidden_size = 2560
    rt_mod = load_module_from_file(work_dir)

    def make(n):
        a = (torch.rand(1, n, hidden_size, device="cuda") * 100).to(tdt)
        return a, (torch.rand(1, n, hidden_size, device="cuda") * 100).to(tdt), torch.empty_like(a)

    latency, bandwidth = sweep(rt_mod, "add", make, lambda n: n * hidden_size * 3 * torch.empty((), dtype=tdt).element_size(),
                               range(1, int(upper) + 1))
    save_to_json(latency, os.path.join(work_dir, "latency.json"))
    save_to_json(bandwidth, os.path.join(work_dir, "bandwidth.json"))
    print(f"n={max(latency)}: {latency[max(latency)]:.2f} us, {bandwidth[max(latency)]:.1f} GiB/s")


if __name__ == "__main__":
    main(*sys.argv[1:])

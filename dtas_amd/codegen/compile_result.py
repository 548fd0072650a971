"""One candidate of one bucket: its config, the C call-table row it resolves to, and its latency.

Stands where the reference has CompileResult (python/dtas/codegen/compile_result.py:23-36): there
it wraps a built TVM module and ``profile`` averages ``time_evaluator`` over sample shapes of the
bucket; here nothing is compiled per candidate (every kernel variant is already in
libdtas_gfx950.so) and ``profile`` times the entry point with the candidate's explicit config.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence

from .._lib import DtasConfig
from ..common.config import Config


class CompileResult:
    def __init__(self, config: Config, abi: DtasConfig, name: str):
        self.config = config
        self.abi = abi
        self.name = name
        self.latency: float = float("inf")  # ms, mean over the sample shapes
        self.launch_args: List[int] = []
        self.error: Optional[str] = None

    def profile(self, run: Callable[[Sequence, DtasConfig], None], tensor_sets: Sequence[Sequence], number: int = 5,
                min_repeat_ms: float = 5.0) -> float:
        """Mean latency in ms over ``tensor_sets`` (one per sample shape).  ``run(tensors, abi)``
        enqueues one call.  Device events on torch's current stream; a candidate that raises is
        recorded as failed and never chosen (the reference skips configs whose build or launch
        throws, python/dtas/schedule/tir_base.py:170-174,222-224)."""
        import torch

        total = 0.0
        try:
            for tensors in tensor_sets:
                run(tensors, self.abi)  # warm-up, also surfaces config errors
                torch.cuda.synchronize()
                reps, elapsed = 0, 0.0
                while reps == 0 or elapsed < min_repeat_ms:
                    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    start.record()
                    for _ in range(number):
                        run(tensors, self.abi)
                    stop.record()
                    stop.synchronize()
                    elapsed += start.elapsed_time(stop)
                    reps += number
                total += elapsed / reps
            self.latency = total / max(1, len(tensor_sets))
        except Exception as exc:  # noqa: BLE001 - any failure disqualifies the candidate
            self.error = str(exc)
            self.latency = float("inf")
        return self.latency

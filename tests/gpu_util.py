"""Helpers of the GPU parity tests: seeded inputs made on the CPU (so the oracle and the kernel see
the same bits), guard bands around device outputs, explicit call-table rows."""
import numpy as np
import torch

from dtas_amd import _lib

GUARD = 64  # elements on each side of an output buffer


def dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


class Guarded:
    """A device output with canary elements before and after it: a kernel that writes past its
    extent (a vector tail, a row overrun) trips ``check``."""

    def __init__(self, shape, dtype: torch.dtype):
        n = int(np.prod(shape))
        self.raw = torch.empty(n + 2 * GUARD, dtype=dtype, device="cuda")
        self.fill = 77 if dtype == torch.int8 else 1234.5
        self.raw.fill_(self.fill)
        self.t = self.raw[GUARD:GUARD + n].view(*shape)

    def check(self) -> np.ndarray:
        torch.cuda.synchronize()
        lo, hi = self.raw[:GUARD].cpu(), self.raw[-GUARD:].cpu()
        assert bool((lo == self.fill).all()) and bool((hi == self.fill).all()), "kernel wrote outside its output"
        return self.t.cpu().numpy()


def cfg(**kw) -> _lib.DtasConfig:
    base = {"variant": 0, "block": 256, "vec": 8, "unroll": 1, "tile": [0, 0, 0], "split_k": 1, "grid_cap": 0}
    base.update(kw)
    return _lib.DtasConfig.from_dict(base)


def bits(a: np.ndarray) -> np.ndarray:
    return a.view({2: np.uint16, 4: np.uint32, 1: np.uint8}[a.dtype.itemsize])


def assert_bits_equal(got: np.ndarray, want: np.ndarray, nan_ok: bool = False) -> None:
    assert got.shape == want.shape and got.dtype == want.dtype
    if nan_ok:
        gn, wn = np.isnan(got), np.isnan(want)
        assert np.array_equal(gn, wn), "NaN positions differ"
        assert np.array_equal(bits(got)[~gn], bits(want)[~wn])
    else:
        bad = np.nonzero(bits(got).ravel() != bits(want).ravel())[0]
        assert bad.size == 0, f"{bad.size} elements differ, first at {bad[:5]}: {got.ravel()[bad[:5]]} vs {want.ravel()[bad[:5]]}"

"""Profile-input generator used while timing candidates (python/dtas/reference.py:8-16):
floats uniform(0, 1), integers randint(0, 100).  Tuning inputs only; parity tests use their own
seeded inputs."""
import numpy as np


def get_ref_tensor(shape, device: str, dtype: str, seed: int = 0) -> np.ndarray:
    del device
    rng = np.random.default_rng(seed)
    if dtype.startswith("float"):
        return rng.uniform(0, 1, size=shape).astype(dtype)
    return rng.integers(0, 100, size=shape).astype(dtype)

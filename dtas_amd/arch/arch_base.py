"""Architecture description consumed by the launch heuristics.

Same slot and field vocabulary as the reference's ``Arch`` (python/dtas/arch/arch_base.py:2-27):
the policies read ``num_sm``, ``max_resident_threads_per_sm``, ``max_smem_per_sm`` ...  On AMD
parts an "SM" is a compute unit, "smem" is LDS and a "warp" is a 64-lane wavefront.
"""


class Arch:
    def __init__(self) -> None:
        self.reg_cap = 0
        self.smem_cap = 0
        self.compute_max_core = 0
        self.num_sm = 0
        self.max_resident_threads_per_sm = 0
        self.max_resident_blocks_per_sm = 0
        self.max_registers_per_sm = 0
        self.max_registers_per_block = 0
        self.max_smem_per_sm = 0
        self.max_smem_per_block = 0
        self.max_threads_per_block = 0
        self.warp_size = 0
        self.sm_partition = 0
        self.transaction_size = [0, 0]
        # half, single, double, matrix-core TFLOP/s
        self.processing_power = [0, 0, 0, 0]
        # GB/s: device memory, L2[, shared]
        self.bandwidth = [0, 0]
        self.l2_cache_size = 0
        self.device = None
        self.platform = "unknown"
        self.compute_capability = "unknown"
        self.target = "unknown"

"""AMD Instinct MI355X (gfx950, CDNA4): the one architecture this package generates launches for."""
from .arch_base import Arch


class MI355X(Arch):
    def __init__(self, dev_id: int = 0, require_device: bool = False):
        super().__init__()
        self.num_sm = 256                      # compute units
        self.num_xcd = 8                       # accelerator complex dies, one L2 each
        self.warp_size = 64                    # wavefront
        self.sm_partition = 4                  # SIMDs per CU
        self.max_resident_threads_per_sm = 2048  # 8 wavefronts per SIMD
        self.max_resident_blocks_per_sm = 32
        self.max_threads_per_block = 1024
        self.reg_cap = 512 * 64 * 4            # 32-bit registers per CU (VGPR + AGPR)
        self.max_registers_per_sm = self.reg_cap
        self.max_registers_per_block = self.reg_cap
        self.smem_cap = 160 * 1024             # LDS per CU = per workgroup
        self.max_smem_per_sm = 160 * 1024
        self.max_smem_per_block = 160 * 1024
        self.transaction_size = [64, 128]
        self.l2_cache_size = 4 * 1024          # KiB per XCD; 256 MiB Infinity Cache behind it
        self.bandwidth = [8000, 20000]         # GB/s: HBM3E peak, aggregate L2 (approximate)
        # dense peaks, TFLOP/s: fp16 vector, fp32 vector, fp64 vector, fp16 MFMA
        self.processing_power = [157.3, 157.3, 78.6, 2500.0]
        self.platform = "ROCm"
        self.compute_capability = "gfx950"
        self.target = "amdgcn-amd-amdhsa--gfx950"
        self.dev_id = dev_id
        self.device = None
        try:
            import torch

            if torch.cuda.is_available():
                self.device = torch.device("cuda", dev_id)
        except Exception:  # pragma: no cover - torch always importable here
            self.device = None
        if require_device and self.device is None:
            raise RuntimeError(f"Cannot find HIP device {dev_id}.")

"""Tile candidates for the dynamic-M GEMM on the MFMA matrix cores.

Plays the part of the reference's WMMAConfigEmiter (python/dtas/policy/wmma_config_emiter.py:15-353):
enumerate block tiles as i x j wavefronts of micro_x x micro_y matrix-core blocks (:72-115), drop
those that do not fit shared memory / registers (:46-70) and rank by a roofline estimate in which a
tile's throughput is min(matrix-core peak, bandwidth * flops-per-byte of the tile) and the job costs
ceil(tiles / SMs) rounds (:148-262).  The tile set is the one libdtas_gfx950.so has kernels for:
2x2 wavefronts of 32x32x16 MFMA blocks, k tile 64; plus, for M <= 64, the weight-streaming
16x16x32 kernel whose wavefronts split K.
"""
from typing import List, Tuple

from ..common.config import MFMAConfig, Range
from .base_config_emiter import BaseConfigEmiter

# (micro_x, micro_y) per wavefront for the 2x2-wavefront kernels, and the measured-order-of-merit
# efficiency of each tile relative to the largest (LDS bytes moved per flop grow as tiles shrink)
_TILES = [((4, 4), 1.00), ((4, 2), 0.85), ((2, 4), 0.85), ((2, 2), 0.70), ((1, 2), 0.50), ((2, 1), 0.50),
          ((1, 1), 0.35)]


class MFMAConfigEmiter(BaseConfigEmiter):
    def check_valid(self, c: MFMAConfig) -> bool:
        lds = 2 * (c.tile_size_m + c.tile_size_n) * c.tile_size_k * 2  # double-buffered fp16 stages
        acc = c.micro_shape_x * c.micro_shape_y * 16                   # fp32 accumulators per lane
        return lds <= self.arch.max_smem_per_block and acc <= 256

    def emit_config(self, range_tuple: Tuple[Range, ...], topk: int = 20) -> List[MFMAConfig]:
        params = self.func_info.func.params
        N, K = params[1].shape
        m_hi = range_tuple[0].end if range_tuple else 1
        if range_tuple:
            m_hi = range_tuple[0].end
        else:
            m_hi = 1
            for e in params[0].shape[:-1]:
                m_hi *= e
        out: List[MFMAConfig] = []
        if m_hi <= 64:
            for threads in (512, 256):
                c = MFMAConfig()
                c.skinny, c.block_threads = True, threads
                c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.micro_shape_k = 1, 1, -(-m_hi // 16), 1, 1
                c.mfma_m, c.mfma_n, c.mfma_k = 16, 16, 32
                out.append(c)
        scored = []
        for (mx, my), eff in _TILES:
            c = MFMAConfig()
            c.micro_shape_x, c.micro_shape_y = mx, my
            if (mx, my) == (4, 4):
                # the 256x256 kernel runs 2x4 wavefronts of 128x64 (two per SIMD)
                c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.block_threads = 2, 4, 4, 2, 512
            if not self.check_valid(c):
                continue
            tiles = -(-m_hi // c.tile_size_m) * -(-N // c.tile_size_n)
            c.num_wave = -(-tiles // self.arch.num_sm)
            cost = c.num_wave * c.tile_size_m * c.tile_size_n / eff
            c.performance = 2.0 * m_hi * N / cost
            scored.append((cost, c))
        out += [c for _, c in sorted(scored, key=lambda t: t[0])]
        return out[:topk]

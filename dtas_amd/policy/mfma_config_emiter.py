"""Tile candidates for the dynamic-M GEMM on the MFMA matrix cores.

Plays the part of the reference's WMMAConfigEmiter (python/dtas/policy/wmma_config_emiter.py:15-353):
enumerate block tiles as i x j wavefronts of micro_x x micro_y matrix-core blocks (:72-115), drop
those that do not fit shared memory / registers (:46-70) and rank by a roofline estimate in which a
tile's throughput is min(matrix-core peak, bandwidth * flops-per-byte of the tile) and the job costs
ceil(tiles / SMs) rounds (:148-262).  The candidate set is what libdtas_gfx950.so has kernels for:
32x32x16 MFMA tiles from 64x64 to 256x256 with 2 to 4 LDS stages, plus, for M <= 64, the
weight-streaming 16x16x32 kernel whose wavefronts split K.  The order is the one on-GPU sweeps favoured;
with a GPU present the Engine times the top-k anyway.
"""
from typing import List, Tuple

from ..common.config import MFMAConfig, Range
from .base_config_emiter import BaseConfigEmiter

# (micro_x, micro_y) per wavefront of the 2x2-wavefront kernels (the 256x256 tile runs 2x4 wavefronts)
_TILES = [(4, 4), (4, 2), (2, 4), (2, 2), (1, 2), (2, 1), (1, 1)]
_LDS = 160 * 1024


class MFMAConfigEmiter(BaseConfigEmiter):
    def check_valid(self, c: MFMAConfig) -> bool:
        stages = c.stages or 2
        lds = stages * (c.tile_size_m + c.tile_size_n) * c.tile_size_k * 2  # fp16 stages of the load pipeline
        acc = c.micro_shape_x * c.micro_shape_y * 16                         # fp32 accumulators per lane
        return lds <= self.arch.max_smem_per_block and acc <= 256

    @staticmethod
    def max_stages(tile_m: int, tile_n: int) -> int:
        return 2 if tile_m + tile_n >= 512 else 3 if tile_m + tile_n >= 384 else 4

    def preferred(self, m_hi: int, N: int):
        """(tile_m, tile_n, stages) that sweeps on an MI355X favoured: 256x256 once it yields >= 150
        workgroups, else 128x128 from 256 workgroups, else 64x64; the deepest load pipeline with which all
        tiles stay co-resident (a margin when several workgroups share a CU), else 2 stages."""
        cdiv = lambda a, b: -(-a // b)
        if cdiv(m_hi, 256) * cdiv(N, 256) >= 150:
            return 256, 256, 2
        t = 128 if cdiv(m_hi, 128) * cdiv(N, 128) >= 256 else 64
        tiles = cdiv(m_hi, t) * cdiv(N, t)
        for ns in (4, 3):
            per_cu = _LDS // (ns * 2 * t * 128)
            if per_cu >= 1 and (tiles <= self.arch.num_sm if per_cu == 1 else tiles * 4 <= self.arch.num_sm * per_cu * 3):
                return t, t, ns
        return t, t, 2

    def emit_config(self, range_tuple: Tuple[Range, ...], topk: int = 20) -> List[MFMAConfig]:
        params = self.func_info.func.params
        N, K = params[1].shape
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
        pref = self.preferred(m_hi, N)
        scored = []
        for mx, my in _TILES:
            base = MFMAConfig()
            base.micro_shape_x, base.micro_shape_y = mx, my
            tm, tn = base.tile_size_m, base.tile_size_n
            for stages in range(2, self.max_stages(tm, tn) + 1):
                c = MFMAConfig()
                c.micro_shape_x, c.micro_shape_y, c.stages = mx, my, stages
                if (mx, my) == (4, 4):
                    # the 256x256 kernel runs 2x4 wavefronts of 128x64 (two per SIMD, alternating phases)
                    c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.block_threads = 2, 4, 4, 2, 512
                if not self.check_valid(c):
                    continue
                tiles = -(-m_hi // tm) * -(-N // tn)
                c.num_wave = -(-tiles // self.arch.num_sm)
                # rank: the measured preference first, then by distance in tile area and stage count
                rank = (0 if (tm, tn, stages) == pref else 1, abs(tm * tn - pref[0] * pref[1]), abs(stages - pref[2]))
                scored.append((rank, c))
        mfma = [c for _, c in sorted(scored, key=lambda t: t[0])]
        # M <= 32 streams W (skinny first); above that the MFMA tiles lead
        out = (out + mfma) if m_hi <= 32 else (mfma[:1] + out + mfma[1:])
        return out[:topk]

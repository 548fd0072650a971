"""Launch candidates for the decode GEMV.

The reference's GEMVConfigEmiter.emit_config is an unfinished stub that returns no candidates
(python/dtas/policy/gemv_config_emiter.py:26-30); its GEMV experiments used the GEMVConfig defaults
(block 32x16, grid N/16, python/dtas/common/config.py:339-356).  Here the candidates are rows of W per
workgroup x threads splitting K, ranked by what sweeps on an MI355X favoured.
"""
from typing import List, Tuple

from ..common.config import GEMVConfig, Range
from .base_config_emiter import BaseConfigEmiter


class GEMVConfigEmiter(BaseConfigEmiter):
    def emit_config(self, range_tuple: Tuple[Range, ...], topk: int = 20) -> List[GEMVConfig]:
        N, K = self.func_info.func.params[1].shape
        out = []
        for rows in (1, 2, 4, 8):
            for threads in (256, 128, 512, 64):
                if threads * 8 > max(K, 512):
                    continue
                c = GEMVConfig()
                c.TILE_S, c.TR = rows, threads
                out.append(c)
        # measured on MI355X: one row per 4-wavefront workgroup is best or within noise for K = 4096;
        # rows of K >= 8192 do better with 8 wavefronts on two rows, and rows that leave the last pass of 4 wavefronts
        # partly empty (K = 2560) with two rows on those 4
        # (short rows: up to 1024 elements one pass of 2 wavefronts, up to 2048 one pass of 4, several rows per workgroup)
        best = (2, 512) if K >= 8192 else (4, 64) if K <= 512 and N >= 12288 else (4 if N >= 12288 else 2, 128) if K <= 1024 else (2, 256) if K <= 2048 or K % 2048 != 0 else (1, 256)

        if not any((c.TILE_S, c.TR) == best for c in out):
            c = GEMVConfig()
            c.TILE_S, c.TR = best
            out.append(c)

        def score(c: GEMVConfig):
            return ((c.TILE_S, c.TR) != best, c.TILE_S, c.TR != 256)

        return sorted(out, key=score)[:topk]

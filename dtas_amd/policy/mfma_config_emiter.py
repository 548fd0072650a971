"""Tile candidates for the dynamic-M GEMM on the MFMA matrix cores.

Plays the part of the reference's WMMAConfigEmiter (python/dtas/policy/wmma_config_emiter.py:15-353):
enumerate block tiles as i x j wavefronts of micro_x x micro_y matrix-core blocks (:72-115), drop
those that do not fit shared memory / registers (:46-70) and rank by a roofline estimate in which a
tile's throughput is min(matrix-core peak, bandwidth * flops-per-byte of the tile) and the job costs
ceil(tiles / SMs) rounds (:148-262).  The candidate set is what libdtas_gfx950.so has kernels for:
MFMA tiles from 64x64 to 256x256 (16x16x32 on the largest, 32x32x16 below) with 2 to 4 LDS stages, with K split over up to 4 workgroups
per tile when M x N yields few tiles, plus, for M <= 64, the weight-streaming 16x16x32 kernel whose
wavefronts split K.  The order is the one on-GPU sweeps favoured;
with a GPU present the Engine times the top-k anyway.
"""
from typing import List, Tuple

from ..common.config import MFMAConfig, Range
from .base_config_emiter import BaseConfigEmiter

# (micro_x, micro_y) per wavefront of the 2x2-wavefront kernels (the 256x256 tile runs 2x4 wavefronts)
_TILES = [(4, 4), (3, 4), (4, 2), (3, 2), (2, 4), (2, 2), (1, 2), (2, 1), (1, 1)]
_LDS = 160 * 1024


class MFMAConfigEmiter(BaseConfigEmiter):
    def check_valid(self, c: MFMAConfig) -> bool:
        stages = c.stages or 2
        lds = stages * (c.tile_size_m + c.tile_size_n) * c.tile_size_k * 2  # fp16 stages of the load pipeline
        acc = c.micro_shape_x * c.micro_shape_y * 16                         # fp32 accumulators per lane
        return lds <= self.arch.max_smem_per_block and acc <= 256

    @staticmethod
    def max_stages(tile_m: int, tile_n: int) -> int:
        return 2 if tile_m + tile_n >= 512 or tile_m == 192 else 3 if tile_m + tile_n >= 384 else 4

    def preferred(self, m_hi: int, N: int, K: int = 4096):
        """(tile_m, tile_n, stages, split_k) under the cost model fitted to sweeps on an MI355X (the same
        one the library's built-in table uses): time = rounds of workgroups over the chip x time of one
        k tile x k tiles.  One k tile with every CU busy: 256x256 see below, 256x128 (8 wavefronts of 64x64) 1.00 us,
        128x128 0.665 us (4 stages, one workgroup per CU) or 1.14 us per round of two per CU (2 stages);
        a partly filled last round costs 0.55 + 0.45 * fill of a full one (0.8 + 0.2 * fill for 128x128 with 4 stages
        in a single round); 64x64 0.33 us per k tile up to
        one workgroup per CU, x 0.82 * (workgroups on the fullest CU) beyond; with few tiles K is split over up
        to 4 workgroups per tile at ~4 us (128x128) / ~1 us (64x64; 2.5 us with more than one per CU) per partial
        tile; 128x64 (4 stages, at most one workgroup per CU) 0.47 us per k tile whatever the fill and ~2.5 us
        per partial tile; 256x128 splits too while its workgroups fit one round and each keeps 32 k tiles or
        more (~4.5 us per partial tile: 512 x 5120 x 13824 in 3 parts 86.8 us against 98.2 for 256x256, 640 x 4096 x 8192 in 2 parts
        63.8 against 67.3).  No candidate is faster than W (2NK bytes) streams through it: 3.1 .. 4.3 TB/s
        by tile, measured with 64 rows against a 50280 x 2560 W."""
        cdiv = lambda a, b: -(-a // b)
        cus = self.arch.num_sm
        ktiles = cdiv(K, 64)

        def rounds(wgs, slots):
            full, rem = divmod(wgs, slots)
            return full + ((0.55 + 0.45 * rem / slots) if rem else 0.0)

        tiles = lambda bm, bn: cdiv(m_hi, bm) * cdiv(N, bn)
        w_mb = 2.0 * float(N) * float(K) * 1e-6
        # W streams at 3.1 .. 4.3 TB/s, by tile; candidates that all sit on that floor are told apart by their own estimates
        floored = lambda us, tbs: (us if us > w_mb / tbs else w_mb / tbs) + 1e-3 * us
        # 256x256 on 8 wavefronts: ~8 us per round of the chip plus 1.50 us per k tile with every CU busy, 0.63 of that
        # with half of the CUs or fewer busy (the card clocks higher), linear in between; split_k = 0: the tiles of
        # a partly filled last round are shared by 2..4 workgroups each (~15 / 18 / 21 us to combine)
        t256 = tiles(256, 256)
        full, rem = divmod(t256, cus)
        relief = lambda fill: 0.63 if fill <= 0.5 else 0.63 + 0.74 * (fill - 0.5)
        us256 = full * (8.0 + 1.50 * ktiles)
        if rem:
            split, _ = self.tail_split_256(m_hi, N, K)
            if split >= 2:
                us256 += 8.0 + 1.50 * cdiv(ktiles, split) * relief(rem * split / cus) + 12.0 + 3.0 * (split - 1)
            else:
                us256 += 8.0 + 1.50 * ktiles * relief(rem / cus)
        # 192x256 on 8 wavefronts (96x64 each): 1.18 us per k tile with every CU busy, the same relief
        full192, rem192 = divmod(tiles(192, 256), cus)
        us192 = full192 * (8.0 + 1.18 * ktiles) + ((8.0 + 1.18 * ktiles * relief(rem192 / cus)) if rem192 else 0.0)
        cands = [(floored(us256, 3.5), (256, 256, 2, 0)),
                 (floored(us192, 3.5), (192, 256, 2, 1)),
                 (floored(rounds(tiles(256, 128), cus) * 1.0 * ktiles, 3.5), (256, 128, 2, 1))]
        # 192x128 on 8 wavefronts (48x64 each), one round that fills three quarters of the chip or more: ~6 us plus
        # 0.66 us per k tile up to 64 of them
        if 3 * cus <= 4 * tiles(192, 128) <= 4 * cus and ktiles <= 64:
            cands.append((floored(6.0 + rounds(tiles(192, 128), cus) * 0.66 * ktiles, 3.5), (192, 128, 2, 1)))
        cands.append((floored(rounds(tiles(128, 128), 2 * cus) * 1.14 * ktiles, 3.1), (128, 128, 2, 1)))
        for split in (1, 2, 3, 4):
            if split > 1 and (ktiles // split < 8 or ktiles <= 16):    # (K <= 1024: a hand-over costs what the shorter loop saves)
                continue
            steps = cdiv(ktiles, split)
            t128, t64 = tiles(128, 128) * split, tiles(64, 64) * split
            if split == 1 or t128 <= cus:
                cands.append((floored((0.8 + 0.2 * t128 / cus if t128 <= cus else rounds(t128, cus)) * 0.665 * steps
                                      + (4.0 * split if split > 1 else 0.0), 4.1 if split == 1 else 3.5), (128, 128, 4, split)))
            cands.append((floored((1.0 if t64 <= cus else 0.82 * -(-int(t64) // cus)) * 0.33 * steps
                                  + ((1.0 if t64 <= cus else 2.5) * split if split > 1 else 0.0), 4.3),
                          (64, 64, 4, split)))
            t256128 = tiles(256, 128) * split
            if split > 1 and steps >= 32 and t256128 <= cus:
                cands.append((floored(rounds(t256128, cus) * 1.0 * steps + 4.5 * split, 3.5), (256, 128, 2, split)))
            t12864 = tiles(128, 64) * split
            if t12864 <= cus:
                cands.append((floored(0.47 * steps + (2.5 * split if split > 1 else 0.0), 3.8), (128, 64, 4, split)))
        best = cands[0]
        for c in cands[1:]:          # first strict minimum, in the library's order of evaluation
            if c[0] < best[0]:
                best = c
        self._model_us = best[0]
        return best[1]

    def tail_split_256(self, M: int, N: int, K: int):
        """(parts, tiles left whole) for split_k = 0 on the 8-wavefront 256x256 tile: whole rounds of the chip
        run one workgroup per tile, the tiles of a last, partly filled round are shared by 2..4 workgroups each
        (as many as still fit the chip at once, each keeping 8 k tiles or more) -- unless the parts would fill more
        than three quarters of the chip and K is short (a partly filled round clocks higher; libdtas: tail_split_256)."""
        cdiv = lambda a, b: -(-a // b)
        cus = self.arch.num_sm
        tiles, ktiles = cdiv(M, 256) * cdiv(N, 256), cdiv(K, 64)
        rem = tiles % cus
        if rem == 0:
            return 1, 0
        split = min(cus // rem, 4)
        while split >= 2 and ktiles // split < 8:
            split -= 1
        if split >= 2 and rem * split > 3 * cus // 4 and ktiles < 128:
            return 1, 0
        if split < 2:
            return 1, 0
        return split, tiles - rem

    def prefers_stream(self, m_hi: int, N: int, K: int) -> bool:
        """M <= 32 and at most one workgroup per CU of the W-streaming kernel (M <= 16: 64 columns x 1024 of K each):
        measured 10.9 against 12.8 us at 4096 x 4096, 7.2 against 10.2 at 2560 x 2560; beyond one round of
        workgroups the tiles win again (libdtas: gemm_policy)."""
        if m_hi <= 16:
            return -(-N // 64) * -(-K // 1024) <= self.arch.num_sm
        # 17 .. 32 rows: 32 rows of A and 512 of K per workgroup, between a quarter of a round and one round of them
        # (8.4 against 9.8 us at 2560 x 2560, 11.4 / 13.9 at 1024 x 8192)
        # (from K = 2048 on: at 4096 x 1024 the 64x64 tiles take 7.4 us, this form 8.2)
        return m_hi <= 32 and K >= 2048 and self.arch.num_sm // 4 <= -(-N // 64) * -(-K // 512) <= self.arch.num_sm

    def prefers_stream_loop(self, m_hi: int, N: int, K: int) -> int:
        """Columns per workgroup (16 or 64) of the looping W-streaming kernel where it leads, else 0: M <= 16, K <= 4096
        and its workgroups fill one round of the chip -- two one-wavefront workgroups per CU for 4096 < N <= 8192, one
        4-wavefront workgroup per CU for 8192 <= N <= 16384 (15.9 against 20.2 us at 8192 x 4096, 20.4 / 24.5 at
        11008 x 4096; libdtas: gemm_policy)."""
        if m_hi > 16 or K > 4096 or self.prefers_stream(m_hi, N, K):
            return 0
        cu = self.arch.num_sm
        if cu < -(-N // 16) <= 2 * cu:
            return 16
        if cu // 2 <= -(-N // 64) <= cu:
            return 64
        return 0

    def prefers_skinny(self, m_hi: int, N: int, K: int) -> bool:
        """M <= 32: the W-streaming kernel (about 3.5 TB/s of W, slower as M grows) against the model's
        best MFMA candidate; call after preferred()."""
        if m_hi > 32:
            return False
        us = N * K * 2.0 / 3.5e6 * (0.9 if m_hi <= 8 else 0.95 if m_hi <= 16 else 1.35)
        wgs = -(-N // 16)               # one workgroup per 16 rows of W: fewer than one per CU leave CUs idle
        if wgs < self.arch.num_sm:
            us *= self.arch.num_sm / wgs
        return us <= self._model_us

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
        stream: List[MFMAConfig] = []
        if m_hi <= 64:
            # the W-streaming kernel: rows of A x columns x K slice, (rows + columns) * slice * 2 bytes of LDS
            for cols, kslice in ((64, 1024), (64, 512), (128, 512)):
                rows = 16 if m_hi <= 16 else 32 if m_hi <= 32 else 64
                if (rows + cols) * kslice * 2 > _LDS or (rows == 64 and cols == 128):
                    continue
                c = MFMAConfig()
                c.stream, c.block_threads = True, 4 * cols
                c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.micro_shape_k = 1, cols // 16, rows // 16, 1, kslice // 32
                c.mfma_m, c.mfma_n, c.mfma_k = 16, 16, 32
                stream.append(c)
        loop: List[MFMAConfig] = []
        if m_hi <= 16:
            # its looping form (K slice 256 = the segment of the LDS ring; the whole of K per workgroup)
            for cols in (64, 16):
                c = MFMAConfig()
                c.stream, c.block_threads = True, 4 * cols
                c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.micro_shape_k = 1, cols // 16, 1, 1, 8
                c.mfma_m, c.mfma_n, c.mfma_k = 16, 16, 32
                loop.append(c)
            lead = self.prefers_stream_loop(m_hi, N, K)
            loop.sort(key=lambda c: c.tile_size_n != lead)
        if m_hi <= 64:
            for threads in (512, 256):
                c = MFMAConfig()
                c.skinny, c.block_threads = True, threads
                c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.micro_shape_k = 1, 1, -(-m_hi // 16), 1, 1
                c.mfma_m, c.mfma_n, c.mfma_k = 16, 16, 32
                out.append(c)
        pref = self.preferred(m_hi, N, K)
        scored = []
        for mx, my in _TILES:
            base = MFMAConfig()
            base.micro_shape_x, base.micro_shape_y = mx, my
            tm, tn = base.tile_size_m, base.tile_size_n
            for stages in range(2, self.max_stages(tm, tn) + 1):
                c = MFMAConfig()
                c.micro_shape_x, c.micro_shape_y, c.stages = mx, my, stages
                if (mx, my) == (4, 4):
                    # the 256x256 kernel runs 2x4 wavefronts of 128x64 (two per SIMD)
                    c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.block_threads = 2, 4, 4, 2, 512
                if (mx, my) == (3, 4):
                    # 192x256: 2x4 wavefronts of 96x64 on the same ring loop
                    c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.block_threads = 2, 4, 3, 2, 512
                if (mx, my) == (3, 2):
                    # 192x128: 4x2 wavefronts of 48x64 (16x16x32 blocks) on the ring loop; the vocabulary's 32-wide micro
                    # blocks do not express 48 rows, so the 2x2 shape stands for the tile's extents
                    c.block_threads = 512
                if (mx, my) == (4, 2) and stages == 2:
                    # 256x128 with two "stages": 4x2 wavefronts of 64x64 on the ring loop of the 256x256 kernel
                    c.i, c.j, c.micro_shape_x, c.micro_shape_y, c.block_threads = 4, 2, 2, 2, 512
                if not self.check_valid(c):
                    continue
                tiles = -(-m_hi // tm) * -(-N // tn)
                c.num_wave = -(-tiles // self.arch.num_sm)
                splits = [1] + [sk for sk in (2, 3, 4) if tiles * sk <= 4 * self.arch.num_sm and -(-K // 64) // sk >= 8]
                if c.block_threads == 512 and (tm, tn) == (256, 256):
                    splits = [0] + splits   # 0: only the tiles of a partly filled last round are split
                for sk in splits:
                    cs = MFMAConfig().from_dict(c.to_dict())
                    cs.split_k, cs.num_wave = sk, -(-tiles * sk // self.arch.num_sm)
                    # rank: the measured preference first, then by distance in tile area, split and stage count
                    rank = (0 if (tm, tn, stages, sk) == pref else 1, abs(tm * tn - pref[0] * pref[1]),
                            abs(sk - pref[3]), abs(stages - pref[2]))
                    scored.append((rank, cs))
        mfma = [c for _, c in sorted(scored, key=lambda t: t[0])]
        # the W-streaming kernel leads only where it beats the best MFMA candidate under the model
        out = (out + mfma) if self.prefers_skinny(m_hi, N, K) else (mfma[:1] + out + mfma[1:])
        out = (stream + out) if self.prefers_stream(m_hi, N, K) else (out[:1] + stream + out[1:])
        out = (loop + out) if m_hi <= 16 and self.prefers_stream_loop(m_hi, N, K) else (out[:2] + loop + out[2:])
        return out[:topk]

"""Launch candidates for row reductions (layer norm, RMS norm, softmax).

The occupancy arithmetic is the reference's ReductionConfigEmiter (python/dtas/policy/
reduction_config_emiter.py:39-158): workgroup sizes warp*partition, +warp, ... while <= 1024 and <=
row length; ``max_active = min(tpm // tx, [smem_sm // smem_row,] max_blocks)``; rows map 1:1 to
workgroups unless there are more rows than ``num_sm * max_active * 32``; candidates sorted by
(max_active, tx, vec) descending.  For ROCm the candidate set is the three gfx950 kernels instead:
"local" (one wavefront per row, row in registers), "shared.dyn" (one workgroup per row) and "cache"
(row re-read per pass), each only where its register budget holds the row.
"""
from typing import List, Optional, Tuple

from ..common.config import Range, ReductionConfig, Var
from .base_config_emiter import BaseConfigEmiter, dtype_bits


class ReductionConfigEmiter(BaseConfigEmiter):
    # the reference hard-wires "cache" (:85); its layer-norm artefacts came from "shared.dyn"
    cuda_temp_storage = "cache"
    # bytes of shared memory one row needs in "shared.dyn" mode; None = (row + 2) * bytes (:79)
    cuda_smem_usage: Optional[int] = None

    def plan_vectorize(self, re_range: Range, in_bytes: int, is_dynamic_reduction: bool = False):
        def allowed(vec: int) -> bool:
            bits = in_bytes * 8 * vec
            if in_bytes == 2:
                return vec % 2 == 0 and 32 <= bits <= 128
            return 32 <= bits <= 128

        valid = [v for v in (16, 8, 4, 3, 2, 1) if allowed(v)]
        if is_dynamic_reduction:
            return valid[0]
        for vec in valid:
            if re_range.end % vec == 0:
                return vec
        return None

    def get_unroll_depth(self):
        return 256

    def get_num_blocks(self, config: ReductionConfig, row_range: Range, max_smem_usage: int, use_shared: bool = True,
                       waves: int = 32) -> None:
        limits = [self.arch.max_resident_threads_per_sm // config.len_tx, self.arch.max_resident_blocks_per_sm]
        if use_shared:
            limits.append(self.arch.max_smem_per_sm // max_smem_usage)
        config.max_active_blocks_per_sm = min(limits)
        max_blocks = self.arch.num_sm * config.max_active_blocks_per_sm * waves
        if max_blocks >= row_range.start:
            config.bx_factor, config.bx = 1, None
        else:
            config.bx, config.bx_factor = max(1, max_blocks), None

    def generate_config_candidates(self, re_range: Range, row_range: Range, in_bytes: int,
                                   is_dynamic_reduction: bool = False, topk: int = 20) -> List[ReductionConfig]:
        if self.arch.platform != "CUDA":
            return self._gfx950_candidates(re_range, row_range, in_bytes, topk)
        max_smem_usage = self.cuda_smem_usage or (re_range.end + 2) * in_bytes
        temp_storage = self.cuda_temp_storage
        vec = self.plan_vectorize(re_range, in_bytes) if temp_storage == "shared.dyn" else None
        configs = []
        block = self.arch.warp_size * self.arch.sm_partition
        while block <= self.arch.max_threads_per_block and block <= re_range.end:
            c = ReductionConfig()
            c.unroll_depth = self.get_unroll_depth()
            c.temp_storage = temp_storage
            c.len_tx = block
            self.get_num_blocks(c, row_range, max_smem_usage, temp_storage == "shared.dyn", 32)
            if vec is not None:
                c.vector_size = vec
            configs.append(c)
            block += self.arch.warp_size
        if len(configs) >= topk:
            return sorted(configs, key=lambda c: (c.max_active_blocks_per_sm, c.len_tx, c.vector_size), reverse=True)[:topk]
        return configs

    @staticmethod
    def _norm_choice(rms: bool, n_hi: int, nvec: int, num_cu: int) -> Optional[Tuple[int, int]]:
        """(threads, rows per trip) of the library's built-in choice for a norm over rows of ``nvec`` 128-bit
        vectors, where it was fitted to sweeps (dispatch.hip:norm_policy, the same rule): up to 4 rows per CU one
        row per workgroup at ~2 vectors per thread; up to 16 .. 24 rows per CU the forms that keep every row
        resident in one round and fetch the per-column parameters once for several rows; beyond, RMSNorm one row
        at ~3 vectors per thread and LayerNorm two rows at ~2.  None outside the fitted row lengths."""
        def round64(v: int) -> int:
            return min(1024, max(64, -(-v // 64) * 64))

        pref, narrow = round64(-(-nvec // 2)), round64(-(-nvec // 5))
        n4, n8, n12, n16, n24 = (k * num_cu for k in (4, 8, 12, 16, 24))
        if rms and 256 <= nvec <= 1024:
            if n_hi <= n4:
                return pref, 1
            if n_hi < n8 or (n_hi == n8 and nvec < 1024):
                return min(pref, 256), 2
            if n_hi <= n24 and nvec < 512:
                return pref, 2 if n_hi <= n12 else 4
            if n_hi <= n16:
                return (256 if nvec >= 512 else pref), 4
            return round64(-(-nvec // 3)), 1
        if not rms and 512 <= nvec <= 2048:
            if n_hi < n4:
                return pref, 1
            if n_hi < n8:
                if nvec <= 640:
                    return pref, 1 if n_hi <= n4 else 2
                return (320 if nvec <= 1024 else 256), 2
            if n_hi <= n16:
                if nvec <= 640:
                    return narrow, 2
                if nvec <= 1024:
                    return (128, 2) if n_hi <= n12 else (256, 4)
                if n_hi <= n8:
                    return (256, 2) if nvec < 2048 else (512, 4)
                return 768, 2
            return pref, 2
        return None

    def _gfx950_candidates(self, re_range: Range, row_range: Range, in_bytes: int, topk: int) -> List[ReductionConfig]:
        """Candidates for libdtas_gfx950.so's row kernels, the library's own built-in choice first:
        a workgroup per row with about two 128-bit vectors per thread (sized in multiples of 64 threads
        so that no lane idles), several rows per trip once there are >= 8 rows per CU; for dynamic rows
        (softmax: 32 rows per unit of row length) a wavefront per row up to 512 vectors, four
        wavefronts per row up to 2048."""
        vec = 16 // in_bytes
        nvec = -(-re_range.end // vec)
        rows = row_range.end
        many_rows = rows >= 8 * self.arch.num_sm
        out: List[ReductionConfig] = []

        def cand(storage: str, tx: int, rpt: int = 1) -> Optional[ReductionConfig]:
            width = 64 if storage == "local" else tx
            iters = -(-nvec // width)
            if storage != "cache" and (iters > 16 or iters * rpt > 16 or (rpt == 2 and iters > 8) or (rpt == 4 and iters > 4)
                                       or (iters * rpt > 8 and tx > 512)):
                return None
            c = ReductionConfig()
            c.temp_storage, c.len_tx, c.vector_size, c.unroll_depth, c.rows_per_trip = storage, tx, vec, 1, rpt
            self.get_num_blocks(c, row_range, 64, storage == "shared.dyn", 32)
            c.bx = None  # rows map 1:1 to wavefronts / workgroups; the kernels stride if capped
            return c

        def round64(v: int) -> int:
            return min(1024, max(64, -(-v // 64) * 64))

        pref = round64(-(-nvec // 2))                       # ~2 vectors per thread
        narrow = round64(-(-nvec // 5))                     # ~5 vectors per thread
        two_params = self.func_info.in_dtype == "float32" and not self.func_info.dyn_red   # layer norm: gamma and beta
        multi = (2 if two_params else 4) if many_rows and not self.func_info.dyn_red else 1   # softmax: one row per trip
        if self.func_info.dyn_red and 512 <= nvec <= 2048:
            # softmax rows of 512 .. 2048 vectors: 4 wavefronts up to 32 rows per CU, ~3 vectors per thread in 256 .. 512
            # threads beyond
            pref = 256 if rows <= 32 * self.arch.num_sm else min(512, max(256, round64(-(-nvec // 3))))
        block_sizes = [pref, narrow] + [t for t in (64, 128, 256, 320, 512, 1024) if t not in (pref, narrow)]
        if two_params and many_rows and rows <= 16 * self.arch.num_sm and -(-nvec // narrow) <= 5 and narrow <= 512:
            block_sizes = [narrow, pref] + block_sizes[2:]
        block_rows = []
        for tx in block_sizes:
            for rpt in dict.fromkeys((multi, 1, 2, 4)):
                if tx <= max(64, round64(nvec)):
                    block_rows.append(cand("shared.dyn", tx, rpt))
        wave_order = (64, 128, 256, 512) if nvec <= 64 else (256, 128, 512, 64)
        wave_rows = [cand("local", tx, rpt) for rpt in (1, 2) for tx in wave_order]
        wave_first = self.func_info.dyn_red and (nvec < 64 * 8 or (nvec == 64 * 8 and rows <= 32 * self.arch.num_sm)) and rows > 2 * self.arch.num_sm
        ordered = (wave_rows + block_rows) if wave_first else (block_rows[:2] + wave_rows[:2] + block_rows[2:] + wave_rows[2:])
        fitted = None if self.func_info.dyn_red else self._norm_choice(not two_params, rows, nvec, self.arch.num_sm)
        if fitted is not None and cand("shared.dyn", *fitted) is not None:
            ordered = [cand("shared.dyn", *fitted)] + [c for c in ordered if c is not None and
                                                         (c.temp_storage, c.len_tx, c.rows_per_trip) != ("shared.dyn",) + fitted]
        out = [c for c in ordered if c is not None]
        stream = cand("cache", 1024 if re_range.end >= 4096 else 256)
        stream.vector_size = 1
        return out[:max(1, topk - 1)] + [stream]

    def emit_config(self, range_tuple: Tuple[Range, ...], topk: int = 20) -> List[ReductionConfig]:
        re_len = self.func_info.red_len
        rows = self.func_info.rows
        re_range = None
        row_range = None
        if self.func_info.dyn_red:
            for r in range_tuple:
                if re_range is None and r.var.name == re_len.name:
                    re_range = r
                    # an extent that is both a row factor and the row length ([heads*n, n])
                    if self._also_row_factor(r):
                        row_range = self._scale(row_range, r, rows)
                else:
                    row_range = self._scale(row_range, r, rows)
            if re_range is None:
                raise ValueError("reduction_len is dynamic, but can't find reduction range info in range_tuple")
        else:
            re_range = Range(Var("re_len"), re_len, re_len)
            for r in range_tuple:
                row_range = self._scale(row_range, r, rows)
        if row_range is None:
            row_range = Range("row_range", rows, rows)
        in_bytes = (dtype_bits(self.func_info.in_dtype) + 7) // 8
        return self.generate_config_candidates(re_range, row_range, in_bytes, self.func_info.dyn_red, topk)

    def _also_row_factor(self, r: Range) -> bool:
        shape = self.func_info.func.params[0].shape
        return any(e == r.var.name for e in shape[:-1])

    @staticmethod
    def _scale(row_range: Optional[Range], r: Range, rows: int) -> Range:
        if row_range is None:
            return Range("row_range", r.start * rows, r.end * rows)
        return Range("row_range", row_range.start * r.start, row_range.end * r.end)

"""Launch candidates for elementwise PrimFuncs.

Follows the reference's ElementwiseConfigEmiter (python/dtas/policy/elementwise_config_emiter.py:
9-88): vector widths of 128 / 64 / 32 bit that the dtype allows, 256-thread workgroups and
``grid = max(1, min(ceil(N / (256 * vec)), num_sm * tpm / 256 * 32))`` with N taken at the bucket's
upper end.  For ROCm architectures each width is additionally offered with 1, 2, 4 or 8 accesses in
flight per thread (the tile a workgroup walks is 256 * vec * unroll elements), ranked by width (128 bit on the
wider side first) and then by the deepest unroll that still leaves a few workgroups per CU.
"""
from typing import List, Tuple

from ..common.config import ElementwiseConfig, Range
from .base_config_emiter import BaseConfigEmiter, dtype_bits


class ElementwiseConfigEmiter(BaseConfigEmiter):
    def plan_vectorize(self, num_elements: int, in_dtype: str, is_dynamic: bool = False) -> List[int]:
        bits = dtype_bits(in_dtype)

        def allowed(vec: int) -> bool:
            if bits == 16:
                return (vec % 2 == 0 or vec == 1) and 32 <= bits * vec <= 128
            if bits == 8:
                return 32 <= bits * vec <= 128
            return bits * vec <= 128

        valid = [v for v in (16, 8, 4, 3, 2, 1) if allowed(v)]
        if is_dynamic:
            return valid
        # static shape: keep widths that need no predicate
        return [v for v in valid if num_elements % v == 0]

    def get_num_blocks(self, n: int, vector_size: int, num_sm: int, tpm: int) -> int:
        k_num_waves, k_block = 32, 256
        return max(1, min((n + k_block * vector_size - 1) // (k_block * vector_size), num_sm * tpm // k_block * k_num_waves))

    def get_unroll_depth(self):
        return 256 if self.arch.platform == "CUDA" else None

    def emit_config(self, range_tuple: Tuple[Range, ...], topk: int = 20) -> List[ElementwiseConfig]:
        num_elements = self.func_info.num_elements
        is_dynamic = len(range_tuple) > 0
        for r in range_tuple:
            num_elements *= r.end
        # the narrower side of a cast bounds the width: 128 bit there, at most 256 on the other
        dtypes = [self.func_info.in_dtype, self.func_info.out_dtype]
        narrow = min(dtypes, key=dtype_bits)
        vecs = self.plan_vectorize(num_elements, narrow, is_dynamic)
        configs: List[ElementwiseConfig] = []
        if self.arch.platform == "CUDA":
            for vec in vecs:
                c = ElementwiseConfig()
                c.vector_size = vec
                c.unroll_depth = self.get_unroll_depth()
                c.grid_size = self.get_num_blocks(num_elements, vec, self.arch.num_sm, self.arch.max_resident_threads_per_sm)
                configs.append(c)
            return configs[:topk]
        vecs = [v for v in vecs if v != 3]  # the reference also offers 96-bit fp32 accesses; no such kernel here
        target = 8 * self.arch.num_sm  # workgroups that give every CU a few wavefronts of loads in flight
        for vec in vecs:
            for unroll in (1, 2, 4, 8):
                c = ElementwiseConfig()
                c.vector_size = vec
                c.unroll_depth = unroll
                c.grid_size = self.get_num_blocks(num_elements, vec * unroll, self.arch.num_sm,
                                                  self.arch.max_resident_threads_per_sm)
                configs.append(c)
        # 128 bit on the wider side of a cast (256-bit accesses on it measured ~40 % slower)
        preferred = max(1, 128 // max(dtype_bits(d) for d in dtypes))

        def score(c: ElementwiseConfig):
            # preferred width first; then the deepest unroll that still leaves >= 4 workgroups per CU
            short = c.grid_size < target // 2
            return (c.vector_size != preferred, short and c.unroll_depth > 1, -c.unroll_depth if not short else c.unroll_depth)

        ranked = sorted(configs, key=score)
        # eight accesses per thread only while all workgroups are resident at once (8 per CU, 6 for the two-input
        # ops); beyond one round many short workgroups are ahead (dispatch.hip:elementwise_policy, the same rule)
        two_inputs = len(self.func_info.func.params) > 2
        first = ranked[0]
        if first.unroll_depth == 8 and num_elements // first.vector_size // (256 * 8) > (6 if two_inputs else 8) * self.arch.num_sm:
            want = 2 if (self.func_info.in_dtype, self.func_info.out_dtype) == ("float32", "float16") else 1
            ranked.sort(key=lambda c: (c.vector_size != first.vector_size, c.unroll_depth != want))
        return ranked[:topk]

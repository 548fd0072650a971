#!/usr/bin/env python3
"""Benchmark of the DTAS hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-sweep] [--no-cpu]

A "step" is one pass of the workload's kernel over its whole pool of synthetic, seeded inputs, all
resident in device memory: one call through the C ABI per buffer set of the pool (`launches_per_step` in
`config`).  The headline workload is the elementwise fp32 -> fp16 cast over [4096, 4096] (the largest n
of the elementwise sweep); the pool is larger than 3x the 256 MiB Infinity Cache so that every launch
streams from HBM.  W warm-up steps, then exactly K timed steps between two device synchronisations;
`value` = algorithmic bytes of those launches / that time.

The same JSON line also carries
  roofline     : the workload's kernel against MI355X's published peak (HBM 8 TB/s, or dense fp16
                 MFMA 2.5 PFLOP/s for the GEMM workloads); `achieved` uses the average per-launch
                 duration measured with HIP events on the launch stream inside the timed region;
  cpu_baseline : the CPU oracle (a port of the PrimFunc loop nest, oracle/cpu_ref.c) on a bounded
                 sample of the same workload, on this machine's host cores;
  roofline.fam_* : the other families of the metric as flat scalar keys (nested values do not survive every
                 consumer of the line) -- `fam_<op>_<shape>_frac` = fraction of the op's roof (HBM for add / copy /
                 casts / RMSNorm / layer norm / softmax / GEMV and for GEMM while its bytes bound it, MFMA otherwise)
                 and `fam_<op>_<shape>_us` = the launch; every GEMM point of the M sweep at the three (N, K), and the
                 reference's own GEMM shapes (N, K) = (2560, 10240), (10240, 2560), (7680, 10240) at n = 256 / 1024 / 4096;
  cpu_baseline.* : beside the headline sample, the oracle on all host cores and on bounded samples of a GEMV and a
                 GEMM point, flat as well (`all_cores_value`, `gemv_f16_4096x4096_gbs_1core`, ...);
  the sweep    : every op family over the dynamic extent n (GB/s or TFLOP/s and roofline fraction), all of them
                 HBM-streaming (rotating buffer sets, the GEMM's W included), printed as one `sweep {...}` text line per
                 row *before* the JSON line, which is the last line of stdout (`--out` writes the rows to a file).
For the gemm_f16 workload two more switches: `--operands zeros|ones|ints` runs the same launches on operands whose
bits hardly toggle (how far the card's power limit sets the rate on the benchmark's random operands), and
`--beside-library` times torch.matmul -- the vendor's GEMM library -- on the same operand pool and reports it as
`library_gemm`, a yardstick that is never part of `value`.
For the two attention workloads `--keys m` sets the key count apart from `--n` (the decode step: `--n 1 --keys 2048`).
One GPU only: `--gpus N` with N > 1 exits with a message.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_FP16_PEAK_TFLOPS = 2500.0  # dense fp16 -> fp32 MFMA
INFINITY_CACHE_BYTES = 256 << 20
METRIC = "achieved HBM GB/s (eltwise/reduce/GEMV) + GEMM TFLOP/s, swept over dynamic n"
OPERANDS = "normal"            # --operands: what the gemm_f16 workload multiplies


# ---------------------------------------------------------------------------------------------
# workloads: name -> (make_buffers(seed) -> tuple of tensors, bind(buffers) -> zero-argument call of
# the C-ABI entry point with the arguments already marshalled, algorithmic bytes, flops)
# ---------------------------------------------------------------------------------------------
def _workload(name: str, n: int, extra=None):
    import torch

    from dtas_amd import _lib

    L = _lib.lib()
    H = 4096
    g = torch.Generator(device="cuda")
    stream = torch.cuda.current_stream().cuda_stream or None

    def uniform(shape, seed, lo=-1.0, hi=1.0, dtype=torch.float16):
        g.manual_seed(seed)
        return (torch.rand(shape, device="cuda", generator=g) * (hi - lo) + lo).to(dtype)

    def normal(shape, seed, std=1.0, dtype=torch.float16):
        g.manual_seed(seed)
        return (torch.randn(shape, device="cuda", generator=g) * std).to(dtype)

    def empty(shape, dtype=torch.float16):
        return torch.empty(shape, dtype=dtype, device="cuda")

    def call(fn, *args):
        def run():
            if fn(*args) != 0:
                raise RuntimeError(_lib.last_error())
        return run

    P = lambda t: t.data_ptr()
    if name == "add_f16":
        make = lambda s: (uniform((n, H), 2 * s), uniform((n, H), 2 * s + 1), empty((n, H)))
        return make, lambda b: call(L.dtas_add_f16, P(b[0]), P(b[1]), P(b[2]), n, H, None, stream), 3 * 2 * n * H, 0
    if name == "copy_f16":
        make = lambda s: (normal((n, H), s, 100.0), empty((n, H)))
        return make, lambda b: call(L.dtas_copy_f16, P(b[0]), P(b[1]), n, H, None, stream), 2 * 2 * n * H, 0
    if name == "cast_f32_f16":
        make = lambda s: (normal((n, H), s, 100.0, torch.float32), empty((n, H)))
        return make, lambda b: call(L.dtas_cast_f32_f16, P(b[0]), P(b[1]), n, H, None, stream), (4 + 2) * n * H, 0
    if name == "cast_f16_f32":
        make = lambda s: (normal((n, H), s, 100.0), empty((n, H), torch.float32))
        return make, lambda b: call(L.dtas_cast_f16_f32, P(b[0]), P(b[1]), n, H, None, stream), (4 + 2) * n * H, 0
    if name == "rms_norm_f16":
        w = uniform((H,), 3, 0.5, 1.5)
        make = lambda s: (normal((n, H), s), w, empty((n, H)))
        return (make, lambda b: call(L.dtas_rms_norm_f16, P(b[0]), P(b[1]), P(b[2]), n, H, 1e-5, None, stream),
                2 * 2 * n * H + 2 * H, 0)
    if name == "layer_norm_f32_f16":
        Hr = 2560
        gm, bt = uniform((Hr,), 3, 0.5, 1.5, torch.float32), uniform((Hr,), 4, -1, 1, torch.float32)
        make = lambda s: (normal((n, Hr), s, 1.0, torch.float32), gm, bt, empty((n, Hr)))
        return (make, lambda b: call(L.dtas_layer_norm_f32_f16, P(b[0]), P(b[1]), P(b[2]), P(b[3]), n, Hr, 1e-5, None, stream),
                (4 + 2) * n * Hr + 8 * Hr, 0)
    if name == "layer_norm_f32":
        # layer_norm: the graph's last layer norm, fp32 in and out
        Hr = 2560
        gm, bt = uniform((Hr,), 3, 0.5, 1.5, torch.float32), uniform((Hr,), 4, -1, 1, torch.float32)
        make = lambda s: (normal((n, Hr), s, 1.0, torch.float32), gm, bt, empty((n, Hr), torch.float32))
        return (make, lambda b: call(L.dtas_layer_norm_f32, P(b[0]), P(b[1]), P(b[2]), P(b[3]), n, Hr, 1e-5, stream),
                8 * n * Hr + 8 * Hr, 0)
    if name == "softmax_f16":
        R = 32 * n
        make = lambda s: (normal((R, n), s, 2.0), empty((R, n)))
        return make, lambda b: call(L.dtas_softmax_f16, P(b[0]), P(b[1]), R, n, None, stream), 2 * 2 * R * n, 0
    if name == "softmax_f32_f16":
        # the reference's published softmax sweep: fp32 in, fp16 out, 12800 rows x n
        # (experiment/dtas_tuned/general_reduction/softmax/row_12800/top10_256_10_nounroll/latency.json)
        R = 12800
        make = lambda s: (normal((R, n), s, 2.0, torch.float32), empty((R, n)))
        return make, lambda b: call(L.dtas_softmax_f32_f16, P(b[0]), P(b[1]), R, n, None, stream), (4 + 2) * R * n, 0
    if name == "gemv_f16":
        N, K = extra
        make = lambda s: (normal((1, K), s), normal((N, K), s + 100, 0.02), empty((1, N)))
        return (make, lambda b: call(L.dtas_gemv_f16, P(b[0]), P(b[1]), None, P(b[2]), N, K, None, stream),
                2 * N * K + 2 * K + 2 * N, 2 * N * K)
    if name == "gemv_f32":
        # NT_matmul5: the fp32 vocabulary projection of the decode graph (50280 x 2560)
        N, K = extra
        make = lambda s: (normal((1, K), s, 1.0, torch.float32), normal((N, K), s + 100, 0.02, torch.float32), empty((1, N), torch.float32))
        return (make, lambda b: call(L.dtas_gemv_f32, P(b[0]), P(b[1]), P(b[2]), N, K, None, stream),
                4 * N * K + 4 * K + 4 * N, 2 * N * K)
    if name == "gemv_q8_f16":
        # fused_fused_decode2_fused_NT_matmul_add: 8-bit weights (4 to a word) with an fp16 scale per 32, dequantised in registers
        N, K = extra
        def make(s):
            g = torch.Generator(device="cuda").manual_seed(s + 200)
            wq = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 4), dtype=torch.int32, device="cuda", generator=g)
            return normal((1, K), s), wq, uniform((N, K // 32), s + 100, 0.001, 0.02), empty((1, N))
        return (make, lambda b: call(L.dtas_gemv_q8_f16, P(b[0]), P(b[1]), P(b[2]), None, P(b[3]), N, K, 0, None, stream),
                N * K + 2 * N * (K // 32) + 2 * K + 2 * N, 2 * N * K)
    if name == "gemv_q8_f32":
        # fused_fused_decode6_NT_matmul5: the 8-bit model's vocabulary projection (fp32 x, y and group scales)
        N, K = extra
        def make(s):
            g = torch.Generator(device="cuda").manual_seed(s + 200)
            wq = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 4), dtype=torch.int32, device="cuda", generator=g)
            return (normal((1, K), s, 1.0, torch.float32), wq, uniform((N, K // 32), s + 100, 0.001, 0.02).float(),
                    empty((1, N), torch.float32))
        return (make, lambda b: call(L.dtas_gemv_q8_f32, P(b[0]), P(b[1]), P(b[2]), P(b[3]), N, K, None, stream),
                N * K + 4 * N * (K // 32) + 4 * K + 4 * N, 2 * N * K)
    if name == "take_q8_f16":
        # fused_fused_decode1_take1: n rows of the 50280 x 2560 embedding table, dequantised (1.0625 bytes in, 2 out per element)
        V, K = extra
        def make(s):
            g = torch.Generator(device="cuda").manual_seed(s + 200)
            wq = torch.randint(-2 ** 31, 2 ** 31 - 1, (V, K // 4), dtype=torch.int32, device="cuda", generator=g)
            ids = torch.randint(0, V, (n,), dtype=torch.int32, device="cuda", generator=g)
            return wq, uniform((V, K // 32), s + 100, 0.001, 0.02), ids, empty((n, K))
        return (make, lambda b: call(L.dtas_take_q8_f16, P(b[0]), P(b[1]), P(b[2]), P(b[3]), n, V, K, None, stream),
                n * K + 2 * n * (K // 32) + 4 * n + 2 * n * K, 0)
    if name == "take_f16":
        # take: n rows of the 50280 x 2560 fp16 embedding table
        V, K = extra
        def make(s):
            g = torch.Generator(device="cuda").manual_seed(s + 200)
            return normal((V, K), s), torch.randint(0, V, (n,), dtype=torch.int32, device="cuda", generator=g), empty((n, K))
        return (make, lambda b: call(L.dtas_take_f16, P(b[0]), P(b[1]), P(b[2]), n, V, K, None, stream), 4 * n * K + 4 * n, 0)
    if name == "rotary_f16":
        # rotary_embedding: [n, 32, 80] with the first 20 of every 80 rotated, tables [4096, 20]
        make = lambda s: (normal((n, 32, 80), s), uniform((4096, 20), s + 1), uniform((4096, 20), s + 2), empty((n, 32, 80)))
        return (make, lambda b: call(L.dtas_rotary_f16, P(b[0]), P(b[1]), P(b[2]), P(b[3]), n, n, 32, 80, 20, 4096, None, stream),
                4 * n * 2560 + 2 * 2 * n * 20, 0)
    if name == "attn_mask_f16":
        # fused_min_max_triu_te_broadcast_to + extend_te: the [n, n] causal mask, written only
        make = lambda s: (empty((n, n)),)
        return make, lambda b: call(L.dtas_attn_mask_f16, P(b[0]), n, n, stream), 2 * n * n, 0
    if name == "swap_axes_f16":
        # transpose6: [n, 32, 80] -> [32, n, 80]
        make = lambda s: (normal((n, 32, 80), s), empty((32, n, 80)))
        return make, lambda b: call(L.dtas_swap_axes_f16, P(b[0]), P(b[1]), n, 32, 80, stream), 4 * n * 2560, 0
    if name == "split3_f16":
        # split: the fused projection [n, 32, 240] into queries, keys and values [n, 32, 80]
        make = lambda s: (normal((n * 32, 240), s), empty((n * 32, 80)), empty((n * 32, 80)), empty((n * 32, 80)))
        return (make, lambda b: call(L.dtas_split3_f16, P(b[0]), P(b[1]), P(b[2]), P(b[3]), n * 32, 80, stream),
                4 * n * 7680, 0)
    if name == "softmax_temperature_f32":
        # softmax_with_temperature: n rows (the model has 1) of 50280 fp32 logits
        V = 50280
        temp = torch.tensor(0.7, dtype=torch.float32, device="cuda")
        make = lambda s: (normal((n, V), s, 4.0, torch.float32), temp, empty((n, V), torch.float32))
        return (make, lambda b: call(L.dtas_softmax_temperature_f32, P(b[0]), P(b[1]), P(b[2]), n, V, stream),
                8 * n * V + 4, 0)
    if name == "gemm_f16":
        N, K = extra
        # OPERANDS != "normal" (--operands): the same launches on operands whose bits hardly toggle -- how far the
        # card's power limit, not the kernel, sets the rate on the benchmark's random operands
        def operand(shape, s, std):
            if OPERANDS == "zeros":
                return torch.zeros(shape, dtype=torch.float16, device="cuda")
            if OPERANDS == "ones":
                return torch.ones(shape, dtype=torch.float16, device="cuda")
            if OPERANDS == "ints":
                g.manual_seed(s)
                return torch.randint(-2, 3, shape, device="cuda", generator=g).to(torch.float16)
            return normal(shape, s, std)
        make = lambda s: (operand((n, K), s, 1.0), operand((N, K), 100 + s, 0.02), empty((n, N)))
        return (make, lambda b: call(L.dtas_gemm_f16, P(b[0]), P(b[1]), None, P(b[2]), n, N, K, None, stream),
                2 * (n * K + N * K + n * N), 2 * n * N * K)
    if name == "attn_scores_f16_f32":
        # fused_NT_matmul1_divide_maximum_minimum_cast2: 32 heads of 80, n = m; the fp32 scores dominate the bytes
        # (extra = (rows, m): a handful of query rows against m keys, the decode step's form; what it moves is K)
        heads, d = 32, 80
        rows, m = (extra if extra else (n, n))
        if extra:
            mask = torch.zeros((rows, m), dtype=torch.float16, device="cuda")
        else:
            mask = torch.full((n, n), 65504.0, dtype=torch.float16, device="cuda").tril_().add_(
                torch.full((n, n), -65504.0, dtype=torch.float16, device="cuda").triu_(1))
        make = lambda s: (normal((heads, rows, d), s), normal((heads, m, d), s + 50), mask, empty((heads, rows, m), torch.float32))
        return (make, lambda b: call(L.dtas_attn_scores_f16_f32, P(b[0]), P(b[1]), P(b[2]), P(b[3]), heads, rows, m, d,
                                     0.11179039301310044, None, stream),
                2 * heads * (rows + m) * d + 2 * rows * m + 4 * heads * rows * m, 2 * heads * rows * m * d)
    if name == "attn_pv_f16":
        # matmul8 (n = m) / matmul10 (extra = (1, m): one query row): 32 heads of 80; the probabilities dominate the bytes
        heads, d = 32, 80
        rows, m = (extra if extra else (n, n))
        make = lambda s: (uniform((heads, rows, m), s), normal((heads, m, d), s + 50), empty((heads, rows, d)))
        return (make, lambda b: call(L.dtas_attn_pv_f16, P(b[0]), P(b[1]), P(b[2]), heads, rows, m, d, None, stream),
                2 * heads * (rows * m + m * d + rows * d), 2 * heads * rows * m * d)
    if name == "gemm_q8_f16":
        # fused_fused_decode2_fused_NT_matmul6_add4: 8-bit weights + fp16 group scales, bias epilogue, n rows
        N, K = extra
        bias = uniform((N,), 302)

        def make(s):
            # the weights rotate with the rest: with few rows the launch is a read of them
            g.manual_seed(300 + s)
            wq = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 4), dtype=torch.int32, device="cuda", generator=g)
            return (normal((n, K), s), wq, uniform((N, K // 32), 301 + s, 0.001, 0.02), bias, empty((n, N)))
        return (make, lambda b: call(L.dtas_gemm_q8_f16_fused, P(b[0]), P(b[1]), P(b[2]), P(b[3]), None, None, P(b[4]), n, N, K, 0,
                                     None, stream),
                2 * n * K + N * K + 2 * N * (K // 32) + 2 * n * N + 2 * N, 2 * n * N * K)
    if name in ("gemm_add2_f16", "gemm_gelu_f16"):
        # fused_NT_matmul2_add1_add3_add3 at (N, K) = (2560, 2560); fused_NT_matmul3_add2_gelu at (10240, 2560)
        N, K = extra
        bias = uniform((N,), 101)
        if name == "gemm_add2_f16":
            make = lambda s: (normal((n, K), s), normal((N, K), 100 + s, 0.02), bias, normal((n, N), s + 1), normal((n, N), s + 2), empty((n, N)))
            return (make, lambda b: call(L.dtas_gemm_f16_fused, P(b[0]), P(b[1]), P(b[2]), P(b[3]), P(b[4]), P(b[5]), n, N, K,
                                         _lib.EPI_BIAS_ADD2, None, stream),
                    2 * (n * K + N * K + 3 * n * N + N), 2 * n * N * K)
        make = lambda s: (normal((n, K), s), normal((N, K), 100 + s, 0.02), bias, empty((n, N)))
        return (make, lambda b: call(L.dtas_gemm_f16_fused, P(b[0]), P(b[1]), P(b[2]), None, None, P(b[3]), n, N, K,
                                     _lib.EPI_BIAS_GELU, None, stream),
                2 * (n * K + N * K + n * N + N), 2 * n * N * K)
    raise ValueError(f"unknown workload {name}")


def _pool_bytes(bufs) -> int:
    seen, total = set(), 0
    for t in bufs:
        if t.data_ptr() not in seen:
            seen.add(t.data_ptr())
            total += t.numel() * t.element_size()
    return total


def make_pool(make, streaming: bool, max_bytes: int = 6 << 30):
    """Buffer sets to rotate through: enough distinct sets that a set has left the Infinity Cache
    before it is used again (>= 3x its capacity), one set when cache-resident timing is wanted."""
    first = make(0)
    if not streaming:
        return [first]
    per = max(1, _pool_bytes(first))
    count = max(2, min(64, -(-3 * INFINITY_CACHE_BYTES // per)))
    count = max(2, min(count, max_bytes // per))
    return [first] + [make(i) for i in range(1, count)]


def time_kernel(calls, steps: int, warmup: int, min_warm_s: float = 0.2):
    """(wall seconds for `steps` steps between two synchronisations, device seconds per launch from a
    pair of HIP events recorded on the launch stream before the first and after the last call).
    A step is one pass over the pool: len(calls) launches, issued back to back, so device seconds / launches
    is the average launch duration (kernel time plus the inter-kernel gap, which is what a caller sees).
    Warm-up runs at least `warmup` steps and at least `min_warm_s`: clocks take a moment to settle."""
    import torch

    t0, i = time.perf_counter(), 0
    while i < warmup * len(calls) or time.perf_counter() - t0 < min_warm_s:
        calls[i % len(calls)]()
        i += 1
        if i % 64 == 0:
            torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        for c in calls:
            c()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, start.elapsed_time(stop) * 1e-3 / (steps * len(calls))


def measure(name: str, n: int, extra, steps: int, warmup: int, streaming: bool = True, min_region_s: float = 2e-3,
            library: bool = False) -> dict:
    """`library` (gemm_f16 only): the same pool, same order, same timing, through torch.matmul -- the vendor's GEMM
    library -- instead of the C-ABI entry point: a yardstick measured on the same card, never part of `value`."""
    make, bind, nbytes, flops = _workload(name, n, extra)
    pool = make_pool(make, streaming)
    if library:
        import torch
        assert name == "gemm_f16"
        calls = [(lambda b: (lambda: torch.matmul(b[0], b[1].t(), out=b[2])))(b) for b in pool]
    else:
        calls = [bind(b) for b in pool]
    wall, per_launch = time_kernel(calls, steps, warmup)
    # short regions: lengthen the timed region so that event and synchronisation costs vanish
    if per_launch * steps * len(calls) < min_region_s:
        steps2 = min(20000, int(min_region_s / max(per_launch * len(calls), 1e-7)) + 1)
        _, per_launch = time_kernel(calls, steps2, 0, 0.0)
    out = {"op": name, "n": n, "us": round(per_launch * 1e6, 3), "ms_per_step": wall * 1e3 / steps,
           "bytes": nbytes, "flops": flops, "pool": len(pool), "gbs": nbytes / per_launch / 1e9}
    if extra:
        out["NK"] = list(extra)
    if flops and name in ("gemm_f16", "gemm_q8_f16", "gemm_add2_f16", "gemm_gelu_f16", "attn_scores_f16_f32", "attn_pv_f16"):
        out["tflops"] = flops / per_launch / 1e12
        hbm_bound_s = nbytes / (HBM_PEAK_GBS * 1e9)
        mfma_bound_s = flops / (MFMA_FP16_PEAK_TFLOPS * 1e12)
        out["bound"] = "mfma" if mfma_bound_s >= hbm_bound_s else "hbm"
        out["frac"] = (out["tflops"] / MFMA_FP16_PEAK_TFLOPS) if out["bound"] == "mfma" else out["gbs"] / HBM_PEAK_GBS
    else:
        out["bound"] = "hbm"
        out["frac"] = out["gbs"] / HBM_PEAK_GBS
    del pool, calls
    return out


# ---------------------------------------------------------------------------------------------
def cpu_baseline(name: str, n: int, budget_s: float = 12.0) -> dict:
    """The CPU oracle on a bounded sample of the headline workload (1 thread = what an unscheduled
    PrimFunc built for an llvm CPU target executes; all host cores reported beside it)."""
    import numpy as np

    import oracle

    oracle.build()
    H = 4096
    rng = np.random.default_rng(2)
    if name == "cast_f32_f16":
        x = (rng.standard_normal((n, H)) * 100).astype(np.float32)
        fn = lambda th: oracle.c.cast(x, "float16", threads=th)
        nbytes = 6 * n * H
    elif name == "add_f16":
        a = rng.uniform(-1, 1, (n, H)).astype(np.float16)
        b = rng.uniform(-1, 1, (n, H)).astype(np.float16)
        fn = lambda th: oracle.c.add(a, b, threads=th)
        nbytes = 6 * n * H
    elif name == "copy_f16":
        a = rng.standard_normal((n, H)).astype(np.float16)
        fn = lambda th: oracle.c.copy(a, threads=th)
        nbytes = 4 * n * H
    else:
        x = rng.standard_normal((n, H)).astype(np.float16)
        w = rng.uniform(0.5, 1.5, H).astype(np.float16)
        fn = lambda th: oracle.c.rms_norm(x, w, threads=th)
        nbytes = 4 * n * H + 2 * H

    def run(threads: int, budget: float):
        fn(threads)  # page in
        reps, t0 = 0, time.perf_counter()
        while True:
            fn(threads)
            reps += 1
            el = time.perf_counter() - t0
            if el > budget or reps >= 200:
                return nbytes * reps / el / 1e9, reps

    cores = min(oracle.c.max_threads(), len(os.sched_getaffinity(0)))
    one, reps1 = run(1, budget_s * 0.6)
    many, repsn = run(cores, budget_s * 0.4)
    return {"value": round(one, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{name} n={n} H={H}, {reps1} full passes of the oracle (oracle/cpu_ref.c), 1 thread",
            "all_cores_value": round(many, 3), "all_cores": cores, "all_cores_passes": repsn}


# ---------------------------------------------------------------------------------------------
SWEEP_N = [1, 16, 128, 1024, 4096]
SWEEP_M = [1, 16, 64, 256, 1024, 2048, 4096, 8192]
GEMV_SHAPES = [(4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)]
GEMM_NK = [(4096, 4096), (11008, 4096), (4096, 11008)]
# the reference's own GEMM sweeps (experiment/testIR/GEMM/m_n2560_k10240, m_n10240_k2560, m_n7680_k10240: data/*.json)
GEMM_NK_REFERENCE = [(2560, 10240), (10240, 2560), (7680, 10240)]


def sweep(steps: int, warmup: int) -> list:
    rows = []
    for op in ("add_f16", "copy_f16", "cast_f32_f16", "cast_f16_f32", "rms_norm_f16", "layer_norm_f32_f16", "softmax_f16"):
        for n in SWEEP_N:
            rows.append(measure(op, n, None, steps, warmup))
    rows.append(measure("softmax_f16", 8192, None, steps, warmup))   # the far end of the dynamic range: [262144, 8192]
    for n in (1024, 2048, 4096):   # the reference's published softmax form: fp32 in, 12800 rows x n
        rows.append(measure("softmax_f32_f16", n, None, steps, warmup))
    for nk in GEMV_SHAPES:
        rows.append(measure("gemv_f16", 1, nk, steps, warmup))
    for nk in GEMV_SHAPES:
        rows.append(measure("gemv_q8_f16", 1, nk, steps, warmup))
    rows.append(measure("gemv_f32", 1, (50280, 2560), steps, warmup))
    rows.append(measure("gemv_q8_f32", 1, (50280, 2560), steps, warmup))
    for n in (1, 1024, 4096):
        rows.append(measure("take_q8_f16", n, (50280, 2560), steps, warmup))
        rows.append(measure("take_f16", n, (50280, 2560), steps, warmup))
        rows.append(measure("rotary_f16", n, None, steps, warmup))
        rows.append(measure("split3_f16", n, None, steps, warmup))
        rows.append(measure("swap_axes_f16", n, None, steps, warmup))
        rows.append(measure("attn_mask_f16", n, None, steps, warmup))
    rows.append(measure("softmax_temperature_f32", 1, None, steps, warmup))
    for n in (1, 4096):
        rows.append(measure("layer_norm_f32", n, None, steps, warmup))
    for nk in GEMM_NK:
        for m in SWEEP_M:
            rows.append(measure("gemm_f16", m, nk, steps, warmup))
    for nk in GEMM_NK_REFERENCE:
        for m in (256, 1024, 4096):
            rows.append(measure("gemm_f16", m, nk, steps, warmup))
    # the model's own fused shapes (dolly-v2-3b: hidden 2560, 32 heads of 80)
    for m in (1, 16, 256, 2048):   # m = 1: the decode forms (fused_NT_matmul8_add5_add7_add7, ..9_add6_gelu1) on the GEMV kernel
        rows.append(measure("gemm_add2_f16", m, (2560, 2560), steps, warmup))
        rows.append(measure("gemm_gelu_f16", m, (10240, 2560), steps, warmup))
        if m == 1:
            continue
        rows.append(measure("gemm_q8_f16", m, (7680, 2560), steps, warmup))
    for n in (128, 1024, 2048):
        rows.append(measure("attn_scores_f16_f32", n, None, steps, warmup))
        rows.append(measure("attn_pv_f16", n, None, steps, warmup))
    rows.append(measure("attn_pv_f16", 1, (1, 2048), steps, warmup))      # matmul10: decoding against 2048 keys
    rows.append(measure("attn_pv_f16", 1, (1, 8192), steps, warmup))      # ... against 8192 (the keys shared by workgroups)
    rows.append(measure("attn_scores_f16_f32", 1, (1, 2048), steps, warmup))  # the decode step's scores
    rows.append(measure("attn_scores_f16_f32", 1, (1, 8192), steps, warmup))
    # a sequence length off every vector width: rows that start at any element
    for op in ("softmax_f16", "attn_scores_f16_f32", "attn_pv_f16"):
        rows.append(measure(op, 1025, None, steps, warmup))
    return rows


def families(rows: list) -> dict:
    """The metric's families as flat scalar keys, from the sweep rows: `fam_<op>_<shape>_frac` is the fraction of the
    op's roof (HBM at the largest n of the memory-bound ops and for every GEMM point whose bytes bound it, MFMA for
    the other GEMM points); GEMM points also carry `_us`, and `_tflops` where the MFMA roof applies."""
    out = {}
    for op in ("add_f16", "copy_f16", "cast_f32_f16", "cast_f16_f32", "rms_norm_f16", "layer_norm_f32_f16", "softmax_f16"):
        for r in rows:
            if r["op"] == op and "NK" not in r and r["n"] in (4096, 8192):
                out[f"fam_{op}_n{r['n']}_frac"] = round(r["frac"], 3)
    for r in rows:
        if r["op"] == "softmax_f32_f16":
            out[f"fam_softmax_f32_f16_12800x{r['n']}_frac"] = round(r["frac"], 3)
        if r["op"] == "gemv_f16":
            out[f"fam_gemv_f16_{r['NK'][0]}x{r['NK'][1]}_frac"] = round(r["frac"], 3)
    for r in rows:
        if r["op"] == "gemm_f16":
            key = f"fam_gemm_f16_M{r['n']}_{r['NK'][0]}x{r['NK'][1]}"
            out[key + "_us"] = round(r["us"], 2)
            if r["bound"] == "mfma":
                out[key + "_tflops"] = round(r["tflops"], 1)
            out[key + ("_frac" if r["bound"] == "mfma" else "_frac_hbm")] = round(r["frac"], 3)
    # the graph's other PrimFuncs (attention matmuls, fused epilogues, 8-bit weights, index-only ops), at their larger points
    for r in rows:
        op, n = r["op"], r["n"]
        frac = "_frac" if r["bound"] == "mfma" else "_frac_hbm"
        if op in ("attn_scores_f16_f32", "attn_pv_f16") and n >= 1024:
            out[f"fam_{op}_n{n}_us"] = round(r["us"], 2)
            out[f"fam_{op}_n{n}_frac_hbm"] = round(r["frac"], 3)
        elif op in ("gemm_q8_f16", "gemm_add2_f16", "gemm_gelu_f16") and n >= 16:
            key = f"fam_{op}_M{n}_{r['NK'][0]}x{r['NK'][1]}"
            out[key + "_us"] = round(r["us"], 2)
            out[key + frac] = round(r["frac"], 3)
        elif op in ("gemv_q8_f16", "gemv_q8_f32", "gemv_f32"):
            out[f"fam_{op}_{r['NK'][0]}x{r['NK'][1]}_frac_hbm"] = round(r["frac"], 3)
        elif op in ("layer_norm_f32", "take_q8_f16", "take_f16", "rotary_f16", "split3_f16", "swap_axes_f16", "attn_mask_f16",
                    "softmax_temperature_f32") and n >= 4096:
            out[f"fam_{op}_n{n}_frac_hbm"] = round(r["frac"], 3)
    return out


def cpu_families(budget_s: float = 6.0) -> dict:
    """The oracle on bounded samples of a GEMV and a GEMM point (one thread and all host cores), as flat keys."""
    import numpy as np

    import oracle

    oracle.build()
    rng = np.random.default_rng(5)
    cores = min(oracle.c.max_threads(), len(os.sched_getaffinity(0)))

    def rate(fn, work, budget):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            el = time.perf_counter() - t0
            if el > budget or reps >= 50:
                return work * reps / el, reps

    N, K = 4096, 4096
    x = rng.standard_normal((1, K)).astype(np.float16)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    gemv_bytes = 2 * N * K + 2 * K + 2 * N
    g1, r1 = rate(lambda: oracle.c.gemm(x, w, threads=1), gemv_bytes, budget_s * 0.2)
    gn, rn = rate(lambda: oracle.c.gemm(x, w, threads=cores), gemv_bytes, budget_s * 0.1)
    M = 64   # 64 of the rows of the M-sweep's problems against the whole W
    a = rng.standard_normal((M, K)).astype(np.float16)
    flops = 2.0 * M * N * K
    f1, q1 = rate(lambda: oracle.c.gemm(a, w, threads=1), flops, budget_s * 0.4)
    fn_, qn = rate(lambda: oracle.c.gemm(a, w, threads=cores), flops, budget_s * 0.3)
    return {"gemv_f16_4096x4096_gbs_1core": round(g1 / 1e9, 3), "gemv_f16_4096x4096_gbs_all_cores": round(gn / 1e9, 3),
            "gemv_f16_4096x4096_passes": r1 + rn,
            "gemm_f16_4096x4096_tflops_1core": round(f1 / 1e12, 5), "gemm_f16_4096x4096_tflops_all_cores": round(fn_ / 1e12, 5),
            "gemm_f16_sample": f"{M} rows of A against the whole W, {q1 + qn} passes (the oracle is row-parallel: the rate does not depend on M)"}


def recorded_traffic(workload_key: str):
    """HBM bytes per launch of this workload's kernel as measured with rocprofv3 --pmc (FETCH_SIZE and
    WRITE_SIZE runs, calibrated on the copy kernel) and committed under profiles/; None when no
    counter run was recorded for it.  Counters cannot be read from inside this process."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(workload_key, {}).get("traffic_bytes")
    except (OSError, ValueError):
        return None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cast_f32_f16",
                    help="cast_f32_f16 | cast_f16_f32 | add_f16 | copy_f16 | rms_norm_f16 | layer_norm_f32_f16 | layer_norm_f32 | softmax_f16 | softmax_f32_f16 (12800 rows x n) | attn_scores_f16_f32 | attn_pv_f16 | "
                         "gemv_f16 | gemv_f32 | gemv_q8_f16 | gemv_q8_f32 | take_q8_f16 | take_f16 | rotary_f16 | split3_f16 | swap_axes_f16 | attn_mask_f16 | softmax_temperature_f32 | gemm_f16 | gemm_q8_f16 | gemm_add2_f16 | gemm_gelu_f16 (the last five take --nk; attn_scores n = m)")
    ap.add_argument("--n", type=int, default=4096, help="dynamic extent of the workload (rows n, or GEMM M)")
    ap.add_argument("--nk", default="4096x4096", help="N x K of the gemv/gemm workloads")
    ap.add_argument("--keys", type=int, default=0,
                    help="attn_scores_f16_f32 / attn_pv_f16: n query rows against this many keys (the decode step's form with --n 1); 0: n = m")
    ap.add_argument("--operands", default="normal", choices=["normal", "zeros", "ones", "ints"],
                    help="gemm_f16 only: normal = the benchmark's A ~ N(0,1), W ~ N(0,0.02); zeros / ones / ints (-2..2) "
                         "run the same launches on operands that draw less power")
    ap.add_argument("--beside-library", action="store_true",
                    help="gemm_f16 only: also time torch.matmul (the vendor GEMM library) on the same operand pool and "
                         "report it as `library_gemm`")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cache-resident", action="store_true", help="time on one buffer set (no rotation)")
    ap.add_argument("--out", default=None, help="also write the sweep rows to this JSON file")
    args = ap.parse_args()
    global OPERANDS
    OPERANDS = args.operands
    if args.gpus != 1:
        print(f"bench.py measures one GPU: every kernel here runs on a single device and no collective exists "
              f"(--gpus {args.gpus} is not supported)", file=sys.stderr)
        return 2

    import torch

    from dtas_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the kernels have no CPU path)", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    if _lib.lib().dtas_init() != 0:
        print(_lib.last_error(), file=sys.stderr)
        return 2

    extra = tuple(int(v) for v in args.nk.split("x")) if args.workload in ("gemv_f16", "gemv_f32", "gemv_q8_f16", "gemv_q8_f32", "take_q8_f16", "take_f16", "gemm_f16", "gemm_q8_f16", "gemm_add2_f16", "gemm_gelu_f16") else None
    if args.workload in ("attn_scores_f16_f32", "attn_pv_f16") and args.keys > 0:
        extra = (args.n, args.keys)
    head = measure(args.workload, args.n, extra, args.steps, args.warmup, streaming=not args.cache_resident)
    is_gemm = args.workload in ("gemm_f16", "gemm_q8_f16", "gemm_add2_f16", "gemm_gelu_f16") and head["bound"] == "mfma"
    info = None
    try:
        op = {"cast_f32_f16": _lib.OP_CAST_F32_F16, "add_f16": _lib.OP_ADD_F16, "copy_f16": _lib.OP_COPY_F16,
              "rms_norm_f16": _lib.OP_RMS_NORM_F16}.get(args.workload)
        if op is not None:
            info = _lib.select_bucket(op, args.n, 4096, 0)
    except _lib.DtasError:
        info = None

    if args.workload == "layer_norm_f32_f16":
        workload_key = f"{args.workload} [n={args.n}, 2560]"
    elif args.workload == "softmax_f16":
        workload_key = f"{args.workload} [{32 * args.n}, n={args.n}]"
    elif args.workload == "softmax_f32_f16":
        workload_key = f"{args.workload} [12800, n={args.n}]"
    elif args.workload in ("attn_scores_f16_f32", "attn_pv_f16"):
        workload_key = f"{args.workload} [32 heads of 80, n=m={args.n}]" if args.keys <= 0 else f"{args.workload} [32 heads of 80, n={args.n}, m={args.keys}]"
    elif extra is None:
        workload_key = f"{args.workload} [n={args.n}, 4096]"
    elif args.workload in ("gemv_f16", "gemv_f32", "gemv_q8_f16", "gemv_q8_f32"):
        workload_key = f"{args.workload} M=1 NxK={args.nk}"
    else:
        workload_key = f"{args.workload} M={args.n} NxK={args.nk}"
    line = {
        "metric": METRIC,
        # one step = one launch per buffer set of the pool
        "value": round(head["flops"] * head["pool"] / (head["ms_per_step"] * 1e-3) / 1e12, 3) if is_gemm
        else round(head["bytes"] * head["pool"] / (head["ms_per_step"] * 1e-3) / 1e9, 3),
        "unit": "TFLOP/s" if is_gemm else "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic" if OPERANDS == "normal" else f"synthetic ({OPERANDS}: not the benchmark's operands)",
        "config": {"workload": workload_key,
                   "buffers": "rotating pool > 3x Infinity Cache" if not args.cache_resident else "single set (cache-resident)",
                   "pool_sets": head["pool"], "launches_per_step": head["pool"],
                   "kernel": info.name.decode() if info is not None else args.workload,
                   "launch": list(info.launch_args)[:5] if info is not None else None},
        "roofline": {
            "bound": "mfma" if is_gemm else "hbm",
            "achieved": round(head["tflops"], 3) if is_gemm else round(head["gbs"], 3),
            "peak": MFMA_FP16_PEAK_TFLOPS if is_gemm else HBM_PEAK_GBS,
            "unit": "TFLOP/s" if is_gemm else "GB/s",
            "frac": round((head["tflops"] / MFMA_FP16_PEAK_TFLOPS) if is_gemm else head["gbs"] / HBM_PEAK_GBS, 4),
            "traffic": recorded_traffic(workload_key),
            "launch_us_mean": head["us"],
            "algorithmic_bytes_per_launch": head["bytes"],
        },
    }
    if args.beside_library and args.workload == "gemm_f16":
        lib_row = measure(args.workload, args.n, extra, args.steps, args.warmup, streaming=not args.cache_resident, library=True)
        again = measure(args.workload, args.n, extra, args.steps, args.warmup, streaming=not args.cache_resident)
        line["library_gemm"] = {"call": "torch.matmul(A, W.t(), out=C), fp16", "launch_us_mean": lib_row["us"],
                                "tflops": round(lib_row["tflops"], 3), "frac": round(lib_row["tflops"] / MFMA_FP16_PEAK_TFLOPS, 4),
                                "this_kernel_after_it_us": again["us"]}
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args.workload if args.workload in ("cast_f32_f16", "add_f16", "copy_f16") else "rms_norm_f16",
                                            min(args.n, 4096))
    else:
        line["cpu_baseline"] = None
    if not args.no_sweep:
        rows = sweep(max(3, args.steps // 40), 1)
        line["roofline"].update(families(rows))
        if line["cpu_baseline"] is not None:
            line["cpu_baseline"].update(cpu_families())
        # the sweep rows go out as text lines ahead of the JSON line, which stays short enough to be read whole
        for r in rows:
            print("sweep " + json.dumps({k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()
                                         if k in ("op", "n", "NK", "us", "gbs", "tflops", "bound", "frac")}))
        line["config"]["sweep_rows"] = len(rows)
        if args.out:
            with open(args.out, "w") as f:
                json.dump(rows, f, indent=1)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

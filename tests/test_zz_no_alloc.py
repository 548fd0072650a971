"""dtas_gemm_f16_static, the GEMM entry point that allocates nothing: its K-split partial tiles and arrival counters
live in a static device array of the library.  Called through the C ABI and compared bit for bit with
dtas_gemm_f16, which runs the same kernels on the workspace it allocates -- twice in a row, the second time on
a smaller problem that finds the first one's leftovers in the array."""
import ctypes

import numpy as np
import pytest
import torch

from dtas_amd import _lib
from gpu_util import Guarded, assert_bits_equal, cfg

pytestmark = pytest.mark.gpu


def _problem(M, N, K, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    a = torch.randn(M, K, device="cuda", generator=g).half()
    w = (torch.randn(N, K, device="cuda", generator=g) * 0.02).half()
    bias = (torch.rand(N, device="cuda", generator=g) * 2 - 1).half()
    return a, w, bias


def _run(fn, a, w, bias, c, stream=None):
    M, K = a.shape
    N = w.shape[0]
    out = Guarded((M, N), torch.float16)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    rc = fn(a.data_ptr(), w.data_ptr(), bias.data_ptr(), out.t.data_ptr(), M, N, K, ctypes.byref(c) if c is not None else None, s or None)
    assert rc == 0, _lib.last_error()
    return out.check()


def test_static_scratch_gemm_equals_the_allocating_entry_point_twice_in_a_row():
    L = _lib.lib()
    assert L.dtas_init() == 0, _lib.last_error()
    # the first problem splits K four ways over 64x64 tiles (built-in row), the second -- smaller, other tile -- three ways
    first = _problem(96, 4096, 4096, 1)
    assert _lib.select_bucket(_lib.OP_GEMM_F16, 96, 4096, 4096).config.split_k > 1
    got1 = _run(L.dtas_gemm_f16_static, *first, None)
    second = _problem(40, 1000, 2048, 2)
    c2 = cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=3, tile=[128, 128, 64], split_k=3)
    got2 = _run(L.dtas_gemm_f16_static, *second, c2)
    assert_bits_equal(got1, _run(L.dtas_gemm_f16, *first, None))
    assert_bits_equal(got2, _run(L.dtas_gemm_f16, *second, c2))
    ref = (second[0].float() @ second[1].float().T + second[2].float()).cpu().numpy()
    assert float(np.abs(got2.astype(np.float32) - ref).max()) < 2e-2
    # and once more, the larger one again over the smaller one's leftovers
    assert_bits_equal(_run(L.dtas_gemm_f16_static, *first, None), got1)


def test_static_scratch_gemm_tail_split_and_unsplit_launches():
    L = _lib.lib()
    # the 8-wavefront tile with only its last round split (2 tiles x 4 parts), and a launch that needs no scratch at all
    big = _problem(512, 256, 4096, 3)
    c0 = cfg(variant=_lib.GEMM_MFMA, block=512, vec=8, unroll=2, tile=[256, 256, 64], split_k=0)
    assert_bits_equal(_run(L.dtas_gemm_f16_static, *big, c0), _run(L.dtas_gemm_f16, *big, c0))
    c1 = cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=4, tile=[64, 64, 64], split_k=1)
    assert_bits_equal(_run(L.dtas_gemm_f16_static, *big, c1), _run(L.dtas_gemm_f16, *big, c1))


def test_static_scratch_gemm_refuses_what_the_array_cannot_hold():
    L = _lib.lib()
    # 16 x 16 tiles of 256x256, each in 2 parts: 2 * 256 * 256 KiB of partial tiles > 32 MiB
    a, w, bias = _problem(256, 256, 1024, 4)
    M = N = 4096
    c = cfg(variant=_lib.GEMM_MFMA, block=512, vec=8, unroll=2, tile=[256, 256, 64], split_k=2)
    big_a = torch.zeros(M, 1024, dtype=torch.float16, device="cuda")
    big_w = torch.zeros(N, 1024, dtype=torch.float16, device="cuda")
    out = torch.empty(M, N, dtype=torch.float16, device="cuda")
    rc = L.dtas_gemm_f16_static(big_a.data_ptr(), big_w.data_ptr(), None, out.data_ptr(), M, N, 1024, ctypes.byref(c), None)
    assert rc == -1 and "static scratch holds" in _lib.last_error()
    # more split tiles than counters
    c64 = cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=2, tile=[64, 64, 64], split_k=2)
    out2 = torch.empty(M, 8192, dtype=torch.float16, device="cuda")
    wide_w = torch.zeros(8192, 1024, dtype=torch.float16, device="cuda")
    rc = L.dtas_gemm_f16_static(big_a.data_ptr(), wide_w.data_ptr(), None, out2.data_ptr(), M, 8192, 1024, ctypes.byref(c64), None)
    assert rc == -1 and "counters" in _lib.last_error()


def test_static_scratch_gemm_on_the_w_streaming_kernel():
    L = _lib.lib()
    # 16 rows against 4096 x 4096: the built-in row is the W-streaming kernel, whose K slices meet in the scratch as well
    small = _problem(16, 4096, 4096, 5)
    assert _lib.select_bucket(_lib.OP_GEMM_F16, 16, 4096, 4096).config.variant == _lib.GEMM_STREAM
    assert_bits_equal(_run(L.dtas_gemm_f16_static, *small, None), _run(L.dtas_gemm_f16, *small, None))


def test_static_scratch_gemm_allocates_no_device_memory():
    L = _lib.lib()
    assert L.dtas_init() == 0, _lib.last_error()
    a, w, bias = _problem(96, 4096, 4096, 6)
    out = torch.empty(96, 4096, dtype=torch.float16, device="cuda")
    fresh = torch.cuda.Stream()          # a stream that owns no workspace yet
    with torch.cuda.stream(fresh):       # (the runtime sets a stream's queue up at its first launch, which takes device memory: not ours)
        out.zero_()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    rc = L.dtas_gemm_f16_static(a.data_ptr(), w.data_ptr(), bias.data_ptr(), out.data_ptr(), 96, 4096, 4096, None, fresh.cuda_stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "the static entry point changed the device's free memory"
    # the same launch through the allocating entry point on that stream takes its 32 MiB workspace: the check above can see one
    rc = L.dtas_gemm_f16(a.data_ptr(), w.data_ptr(), bias.data_ptr(), out.data_ptr(), 96, 4096, 4096, None, fresh.cuda_stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert free0 - torch.cuda.mem_get_info()[0] >= 32 << 20


def test_static_scratch_gemm_under_stream_capture_replays_the_same_bits():
    L = _lib.lib()
    assert L.dtas_init() == 0, _lib.last_error()   # resolves the scratch address: required before a captured call
    a, w, bias = _problem(96, 4096, 4096, 7)
    eager = _run(L.dtas_gemm_f16_static, a, w, bias, None)
    out = torch.zeros(96, 4096, dtype=torch.float16, device="cuda")
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        rc = L.dtas_gemm_f16_static(a.data_ptr(), w.data_ptr(), bias.data_ptr(), out.data_ptr(), 96, 4096, 4096, None,
                                    torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.last_error()
    other = _problem(40, 1000, 2048, 8)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert_bits_equal(out.cpu().numpy(), eager)
        # eager work on the same scratch between the replays
        _run(L.dtas_gemm_f16_static, *other, cfg(variant=_lib.GEMM_MFMA, block=256, vec=8, unroll=3, tile=[128, 128, 64], split_k=3))

"""CPU oracle for the DTAS hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Two independent restatements of the PrimFunc math:

* ``oracle.c``   -- ctypes bindings of ``cpu_ref.c`` (literal loop nests, fp32 / fp16
  arithmetic as the PrimFunc text states; also timed as the CPU baseline);
* ``oracle.np64`` -- closed forms in numpy float64 (the tolerance anchor that pins
  ``cpu_ref.c`` and the GPU kernels alike).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
import this package.  The product (``dtas_amd``) never does.

The reference holds no numerical tests or golden vectors for this path, so each
function is pinned by closed forms, library routines, exhaustive enumeration and
invariants (``tests/test_oracle_*.py``).  ``rms_norm`` has no counterpart in the
reference at all: parity unpinned by the reference, closed form only.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libdtas_oracle.so")


def build(force: bool = False) -> str:
    """Compile cpu_ref.c into libdtas_oracle.so (gcc, a second or two)."""
    src = os.path.join(_HERE, "cpu_ref.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libdtas_oracle.so"])
    return _SO


def _ptr(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"], "oracle takes C-contiguous arrays"
    return a.ctypes.data_as(ctypes.c_void_p)


class _C:
    """Lazy ctypes view of libdtas_oracle.so."""

    _lib = None

    @classmethod
    def lib(cls):
        if cls._lib is None:
            if not os.path.exists(_SO):
                build()
            lib = ctypes.CDLL(_SO)
            vp, i64, ci, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
            sig = {
                "oracle_add_f16": [vp, vp, vp, i64, ci],
                "oracle_add_f32": [vp, vp, vp, i64, ci],
                "oracle_add_i8": [vp, vp, vp, i64, ci],
                "oracle_copy_bytes": [vp, vp, i64, ci],
                "oracle_cast_f16_f32": [vp, vp, i64, ci],
                "oracle_cast_f32_f16": [vp, vp, i64, ci],
                "oracle_layer_norm_f32_f16": [vp, vp, vp, vp, i64, i64, f32, ci],
                "oracle_rms_norm_f16": [vp, vp, vp, i64, i64, f32, ci],
                "oracle_softmax_f32_f16": [vp, vp, i64, i64, ci],
                "oracle_softmax_f16_f16": [vp, vp, i64, i64, ci],
                "oracle_softmax_temperature_f32": [vp, vp, vp, i64, i64, ci],
                "oracle_divide_f32": [vp, vp, vp, i64],
                "oracle_layer_norm_f32": [vp, vp, vp, vp, i64, i64, ctypes.c_float, ci],
                "oracle_gemm_f16": [vp, vp, vp, vp, i64, i64, i64, ci, ci],
                "oracle_gemm_f16_f32out": [vp, vp, vp, i64, i64, i64, ci],
                "oracle_gemv_f16_rf": [vp, vp, vp, vp, i64, i64, ci],
                "oracle_gemm_f16_fused": [vp, vp, vp, vp, vp, vp, i64, i64, i64, ci, ci, ci],
                "oracle_attn_scores_f16_f32": [vp, vp, vp, vp, i64, i64, i64, i64, f32, ci, ci],
                "oracle_attn_pv_f16": [vp, vp, vp, i64, i64, i64, i64, ci, ci],
                "oracle_gemv_f32": [vp, vp, vp, i64, i64, ci],
                "oracle_take_f16": [vp, vp, vp, i64, i64, ci],
                "oracle_rotary_f16": [vp, vp, vp, vp, i64, i64, i64, i64, i64, ci],
                "oracle_take_q8_f16": [vp, vp, vp, vp, i64, i64, ci],
                "oracle_gemv_q8_f32": [vp, vp, vp, vp, i64, i64, ci],
                "oracle_decode_q8_f16": [vp, vp, vp, i64, i64, ci],
                "oracle_gemv_q8_f16": [vp, vp, vp, vp, vp, i64, i64, ci, ci, ci],
            }
            for name, argtypes in sig.items():
                fn = getattr(lib, name)
                fn.argtypes = argtypes
                fn.restype = None
            lib.oracle_soft_h2f.argtypes = [ctypes.c_uint16]
            lib.oracle_soft_h2f.restype = ctypes.c_float
            lib.oracle_soft_f2h.argtypes = [ctypes.c_float]
            lib.oracle_soft_f2h.restype = ctypes.c_uint16
            lib.oracle_max_threads.argtypes = []
            lib.oracle_max_threads.restype = ctypes.c_int
            cls._lib = lib
        return cls._lib


class c:  # noqa: N801  (namespace, mirrors the C file)
    """cpu_ref.c through ctypes.  Arrays in, new array out; ``threads`` splits rows."""

    @staticmethod
    def max_threads() -> int:
        return int(_C.lib().oracle_max_threads())

    @staticmethod
    def add(a: np.ndarray, b: np.ndarray, threads: int = 1) -> np.ndarray:
        assert a.dtype == b.dtype and a.shape == b.shape
        out = np.empty_like(a)
        fn = {"float16": "oracle_add_f16", "float32": "oracle_add_f32", "int8": "oracle_add_i8"}[a.dtype.name]
        getattr(_C.lib(), fn)(_ptr(a), _ptr(b), _ptr(out), a.size, threads)
        return out

    @staticmethod
    def copy(a: np.ndarray, threads: int = 1) -> np.ndarray:
        out = np.empty_like(a)
        _C.lib().oracle_copy_bytes(_ptr(a), _ptr(out), a.nbytes, threads)
        return out

    @staticmethod
    def cast(a: np.ndarray, dtype: str, threads: int = 1) -> np.ndarray:
        out = np.empty(a.shape, dtype=dtype)
        key = (a.dtype.name, np.dtype(dtype).name)
        fn = {("float16", "float32"): "oracle_cast_f16_f32", ("float32", "float16"): "oracle_cast_f32_f16"}[key]
        getattr(_C.lib(), fn)(_ptr(a), _ptr(out), a.size, threads)
        return out

    @staticmethod
    def layer_norm(x, gamma, beta, eps: float = 1e-5, threads: int = 1) -> np.ndarray:
        assert x.dtype == np.float32 and gamma.dtype == np.float32 and beta.dtype == np.float32
        H = x.shape[-1]
        out = np.empty(x.shape, dtype=np.float16)
        _C.lib().oracle_layer_norm_f32_f16(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(out), x.size // H, H, eps, threads)
        return out

    @staticmethod
    def layer_norm_f32(x, gamma, beta, eps: float = 1e-5, threads: int = 1) -> np.ndarray:
        assert x.dtype == gamma.dtype == beta.dtype == np.float32
        H = x.shape[-1]
        out = np.empty(x.shape, dtype=np.float32)
        _C.lib().oracle_layer_norm_f32(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(out), x.size // max(H, 1), H, eps, threads)
        return out

    @staticmethod
    def rms_norm(x, w, eps: float = 1e-5, threads: int = 1) -> np.ndarray:
        assert x.dtype == np.float16 and w.dtype == np.float16
        H = x.shape[-1]
        out = np.empty_like(x)
        _C.lib().oracle_rms_norm_f16(_ptr(x), _ptr(w), _ptr(out), x.size // H, H, eps, threads)
        return out

    @staticmethod
    def softmax(x, threads: int = 1) -> np.ndarray:
        cols = x.shape[-1]
        out = np.empty(x.shape, dtype=np.float16)
        fn = {"float16": "oracle_softmax_f16_f16", "float32": "oracle_softmax_f32_f16"}[x.dtype.name]
        getattr(_C.lib(), fn)(_ptr(x), _ptr(out), x.size // max(cols, 1), cols, threads)
        return out

    @staticmethod
    def divide(a, b: float) -> np.ndarray:
        assert a.dtype == np.float32
        bb = np.array([b], dtype=np.float32)
        out = np.empty_like(a)
        _C.lib().oracle_divide_f32(_ptr(a), _ptr(bb), _ptr(out), a.size)
        return out

    @staticmethod
    def softmax_f32(x, threads: int = 1) -> np.ndarray:
        """softmax2 (before_dl.py:1062-1096): the fp32 pipeline of softmax_temperature with nothing divided (x / 1 is x)."""
        return c.softmax_temperature(x, 1.0, threads)

    @staticmethod
    def softmax_temperature(x, temperature: float, threads: int = 1) -> np.ndarray:
        assert x.dtype == np.float32
        cols = x.shape[-1]
        t = np.array([temperature], dtype=np.float32)
        out = np.empty(x.shape, dtype=np.float32)
        _C.lib().oracle_softmax_temperature_f32(_ptr(x), _ptr(t), _ptr(out), x.size // max(cols, 1), cols, threads)
        return out

    @staticmethod
    def gemm(a, w, bias=None, acc_f16: bool = False, threads: int = 1) -> np.ndarray:
        """C[M,N] = A[M,K] . W[N,K]^T (+ bias[N]); GEMV is M == 1."""
        assert a.dtype == np.float16 and w.dtype == np.float16
        K = a.shape[-1]
        M, N = a.size // K, w.shape[0]
        assert w.shape == (N, K)
        out = np.empty(a.shape[:-1] + (N,), dtype=np.float16)
        bp = _ptr(bias) if bias is not None else None
        _C.lib().oracle_gemm_f16(_ptr(a), _ptr(w), bp, _ptr(out), M, N, K, int(acc_f16), threads)
        return out

    @staticmethod
    def gemv_rf(x, w, bias=None, threads: int = 1) -> np.ndarray:
        """y[N] = W[N,K] . x[K] (+ bias), every sum in fp16 in the order of the reference's scheduled GEMV kernel
        (256 strided partial sums per row, folded 8 at a time, then the 32-lane shuffle tree)."""
        assert x.dtype == np.float16 and w.dtype == np.float16 and x.size == w.shape[1]
        N, K = w.shape
        out = np.empty(N, dtype=np.float16)
        _C.lib().oracle_gemv_f16_rf(_ptr(x), _ptr(w), _ptr(bias) if bias is not None else None, _ptr(out), N, K, threads)
        return out

    @staticmethod
    def gemm_fused(a, w, bias, res1, res2, kind: int, acc_f16: bool = False, threads: int = 1) -> np.ndarray:
        """GEMM + fused epilogue (0 bias, 1 bias+add+add, 2 the same widened to fp32, 3 bias+gelu)."""
        assert a.dtype == np.float16 and w.dtype == np.float16
        K = a.shape[-1]
        M, N = a.size // K, w.shape[0]
        out = np.empty(a.shape[:-1] + (N,), dtype=np.float32 if kind == 2 else np.float16)
        opt = lambda t: _ptr(t) if t is not None else None
        _C.lib().oracle_gemm_f16_fused(_ptr(a), _ptr(w), opt(bias), opt(res1), opt(res2), _ptr(out), M, N, K, kind,
                                       int(acc_f16), threads)
        return out

    @staticmethod
    def attn_scores(q, k, mask, scale: float, acc_f16: bool = False, threads: int = 1) -> np.ndarray:
        """fp32 scores[h,n,m] of fp16 q[h,n,d], k[h,m,d], mask[n,m]: scale, clamp at -65504, min with the mask."""
        heads, n, d = q.shape
        m = k.shape[1]
        assert k.shape == (heads, m, d) and mask.shape == (n, m)
        out = np.empty((heads, n, m), dtype=np.float32)
        _C.lib().oracle_attn_scores_f16_f32(_ptr(q), _ptr(k), _ptr(mask), _ptr(out), heads, n, m, d, scale, int(acc_f16), threads)
        return out

    @staticmethod
    def attn_pv(p, v, acc_f16: bool = False, threads: int = 1) -> np.ndarray:
        """fp16 out[h,n,d] = p[h,n,m] . v[h,m,d]."""
        heads, n, m = p.shape
        d = v.shape[2]
        assert v.shape == (heads, m, d) and p.dtype == np.float16 and v.dtype == np.float16
        out = np.empty((heads, n, d), dtype=np.float16)
        _C.lib().oracle_attn_pv_f16(_ptr(p), _ptr(v), _ptr(out), heads, n, m, d, int(acc_f16), threads)
        return out

    @staticmethod
    def gemv_f32(x, w, threads: int = 1) -> np.ndarray:
        """fp32 y[N] = x[K] . w[N,K]^T, fp32 running sum with k ascending."""
        assert x.dtype == np.float32 and w.dtype == np.float32 and x.size == w.shape[1]
        out = np.empty(x.shape[:-1] + (w.shape[0],), dtype=np.float32)
        _C.lib().oracle_gemv_f32(_ptr(x), _ptr(w), _ptr(out), w.shape[0], w.shape[1], threads)
        return out

    @staticmethod
    def decode_q8(wq, scale, threads: int = 1) -> np.ndarray:
        """fp16 W[N,K] of uint32 wq[N,K/4] (byte j % 4 of word j / 4) and fp16 scale[N,K/32]."""
        N, K = wq.shape[0], wq.shape[1] * 4
        assert wq.dtype == np.uint32 and scale.dtype == np.float16 and scale.shape == (N, K // 32)
        out = np.empty((N, K), dtype=np.float16)
        _C.lib().oracle_decode_q8_f16(_ptr(wq), _ptr(scale), _ptr(out), N, K, threads)
        return out

    @staticmethod
    def gemv_q8(x, wq, scale, bias=None, kind: int = 0, acc_f16: bool = False, threads: int = 1) -> np.ndarray:
        """fp16 y[N] = x[K] . decode_q8(wq, scale)^T (+ bias; kind 3: GELU)."""
        N, K = wq.shape[0], wq.shape[1] * 4
        assert x.dtype == np.float16 and x.size == K and scale.shape == (N, K // 32)
        out = np.empty(x.shape[:-1] + (N,), dtype=np.float16)
        bp = _ptr(bias) if bias is not None else None
        _C.lib().oracle_gemv_q8_f16(_ptr(x), _ptr(wq), _ptr(scale), bp, _ptr(out), N, K, kind, int(acc_f16), threads)
        return out

    @staticmethod
    def rotary(a, cos, sin, m: int, threads: int = 1) -> np.ndarray:
        """fp16 rotary embedding of a[n, heads, d] with tables cos/sin[max_pos, rot] at positions m - n .. m - 1."""
        n, heads, d = a.shape[-3:]
        rot = cos.shape[1]
        assert a.dtype == cos.dtype == sin.dtype == np.float16 and cos.shape == sin.shape and n <= m <= cos.shape[0]
        out = np.empty_like(a)
        _C.lib().oracle_rotary_f16(_ptr(a), _ptr(cos), _ptr(sin), _ptr(out), n, m, heads, d, rot, threads)
        return out

    @staticmethod
    def take(a, ids, threads: int = 1) -> np.ndarray:
        """fp16 out[n,H]: rows ids[i] of a[V,H]."""
        assert a.dtype == np.float16 and a.ndim == 2 and ids.dtype == np.int32
        assert ids.size == 0 or (0 <= ids.min() and ids.max() < a.shape[0])
        out = np.empty((ids.size, a.shape[1]), dtype=np.float16)
        _C.lib().oracle_take_f16(_ptr(a), _ptr(ids), _ptr(out), ids.size, a.shape[1], threads)
        return out

    @staticmethod
    def take_q8(wq, scale, ids, threads: int = 1) -> np.ndarray:
        """fp16 out[n,K]: rows ids[i] of decode_q8(wq, scale)."""
        V, K = wq.shape[0], wq.shape[1] * 4
        assert wq.dtype == np.uint32 and scale.dtype == np.float16 and scale.shape == (V, K // 32) and ids.dtype == np.int32
        assert ids.size == 0 or (0 <= ids.min() and ids.max() < V)
        out = np.empty((ids.size, K), dtype=np.float16)
        _C.lib().oracle_take_q8_f16(_ptr(wq), _ptr(scale), _ptr(ids), _ptr(out), ids.size, K, threads)
        return out

    @staticmethod
    def gemv_q8_f32(x, wq, scale, threads: int = 1) -> np.ndarray:
        """fp32 y[N] = x[K] . W^T with W = float32(byte - 127) * fp32 scale[N,K/32]."""
        N, K = wq.shape[0], wq.shape[1] * 4
        assert x.dtype == np.float32 and x.size == K and wq.dtype == np.uint32
        assert scale.dtype == np.float32 and scale.shape == (N, K // 32)
        out = np.empty(x.shape[:-1] + (N,), dtype=np.float32)
        _C.lib().oracle_gemv_q8_f32(_ptr(x), _ptr(wq), _ptr(scale), _ptr(out), N, K, threads)
        return out

    @staticmethod
    def gemm_f32out(a, w, threads: int = 1) -> np.ndarray:
        K = a.shape[-1]
        M, N = a.size // K, w.shape[0]
        out = np.empty(a.shape[:-1] + (N,), dtype=np.float32)
        _C.lib().oracle_gemm_f16_f32out(_ptr(a), _ptr(w), _ptr(out), M, N, K, threads)
        return out

    @staticmethod
    def soft_h2f(bits: int) -> float:
        return float(_C.lib().oracle_soft_h2f(bits))

    @staticmethod
    def soft_f2h(v: float) -> int:
        return int(_C.lib().oracle_soft_f2h(ctypes.c_float(v)))


class layout:
    """The index-only PrimFuncs around attention, in numpy (bit-exact by construction)."""

    @staticmethod
    def attn_mask(n: int, m: int) -> np.ndarray:
        """fused_min_max_triu_te_broadcast_to (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:642-658) followed by
        extend_te (:68-80), in one expression: -65504 where key j lies after query i (of the last n positions), 65504
        elsewhere; n = 1 is full (:83-93)."""
        i, j = np.arange(n)[:, None], np.arange(m)[None, :]
        return np.where(j - (m - n) > i, np.float16(-65504), np.float16(65504)).astype(np.float16)

    @staticmethod
    def split3(a: np.ndarray):
        """split (before_dl.py:1099-1125) / fused_reshape7_split1 (:661-688): section s of the last axis is
        A[..., s d : (s + 1) d]."""
        d = a.shape[-1] // 3
        return tuple(np.ascontiguousarray(a[..., s_ * d:(s_ + 1) * d]) for s_ in range(3))

    @staticmethod
    def swap_axes(a: np.ndarray) -> np.ndarray:
        """transpose6 / transpose7 (before_dl.py:1177-1203): T[.., i1, i2, :] = A[.., i2, i1, :]."""
        return np.ascontiguousarray(np.swapaxes(a, -3, -2))


class np64:  # noqa: N801
    """Closed forms in float64 -- independent of cpu_ref.c; the tolerance anchor."""

    @staticmethod
    def layer_norm(x, gamma, beta, eps=1e-5):
        x = x.astype(np.float64)
        mean = x.mean(-1, keepdims=True)
        var = (x * x).mean(-1, keepdims=True) - mean * mean
        return (x - mean) / np.sqrt(var + eps) * gamma.astype(np.float64) + beta.astype(np.float64)

    @staticmethod
    def rms_norm(x, w, eps=1e-5):
        x = x.astype(np.float64)
        return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w.astype(np.float64)

    @staticmethod
    def softmax(x):
        x = x.astype(np.float64)
        e = np.exp(x - x.max(-1, keepdims=True))
        return e / e.sum(-1, keepdims=True)

    @staticmethod
    def gemm(a, w, bias=None):
        r = a.astype(np.float64) @ w.astype(np.float64).T
        if bias is not None:
            r = r + bias.astype(np.float64)
        return r

    @staticmethod
    def attn_scores(q, k, mask, scale):
        s_ = np.einsum("hnd,hmd->hnm", q.astype(np.float64), k.astype(np.float64)) * float(np.float16(scale))
        return np.minimum(np.maximum(s_, -65504.0), mask.astype(np.float64)[None])

    @staticmethod
    def decode_q8(wq, scale):
        q = wq.view(np.uint8).reshape(wq.shape[0], -1).astype(np.float64) - 127.0      # little endian: byte j of the row
        return q * np.repeat(scale.astype(np.float64), 32, axis=1)

    @staticmethod
    def attn_pv(p, v):
        return np.einsum("hnm,hmd->hnd", p.astype(np.float64), v.astype(np.float64))

    @staticmethod
    def gemm_fused(a, w, bias, res1, res2, kind):
        """The fused epilogues in float64, no intermediate rounding (the tolerance anchor)."""
        from scipy.special import erf
        r = np64.gemm(a, w, bias)
        if kind in (1, 2):
            r = res1.astype(np.float64) + r + res2.astype(np.float64)
        elif kind == 3:
            r = r * (0.5 + 0.5 * erf(r * 0.70710678118654757))
        return r

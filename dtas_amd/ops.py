"""Entry points on torch tensors: each function enqueues one kernel of libdtas_gfx950.so.

Destination passing, as in the reference (``rt_mod["add"](x, y, out)``,
experiment/dtas_tuned/elementwise/add/profile_add.py:26): the caller allocates every buffer, outputs
included; nothing is allocated or synchronised here.  Tensors must be contiguous device tensors; the
kernel goes on torch's current stream.  ``cfg`` (a ``_lib.DtasConfig``) overrides the built-in bucket
table.  torch is used for device memory and streams only.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib
from ._lib import DtasConfig, check, lib

_ELT = {
    ("add", torch.float16): ("dtas_add_f16", _lib.OP_ADD_F16),
    ("add", torch.float32): ("dtas_add_f32", _lib.OP_ADD_F32),
    ("add", torch.int8): ("dtas_add_i8", _lib.OP_ADD_I8),
    ("copy", torch.float16): ("dtas_copy_f16", _lib.OP_COPY_F16),
    ("copy", torch.float32): ("dtas_copy_f32", _lib.OP_COPY_F32),
    ("copy", torch.int8): ("dtas_copy_i8", _lib.OP_COPY_I8),
}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """torch's current stream on the current device as a raw hipStream_t (0 = the default stream)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device()) or None
    return torch.cuda.current_stream().cuda_stream or None


def _dev(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("dtas_amd kernels take device tensors; got a CPU tensor (there is no CPU path)")
        if not t.is_contiguous():
            raise ValueError("dtas_amd kernels take compact row-major buffers (strides == NULL in the reference)")


def _p(t: Optional[torch.Tensor]):
    # ints convert to void* through the argtypes; 0 (an empty tensor) becomes NULL
    return None if t is None else (t.data_ptr() or None)


def _cfg(cfg: Optional[DtasConfig]):
    return ctypes.byref(cfg) if cfg is not None else None


def _rows_cols(t: torch.Tensor):
    cols = t.shape[-1] if t.dim() > 0 else 1
    rows = t.numel() // cols if cols else 0
    return rows, cols


def add(A: torch.Tensor, B: torch.Tensor, T_add: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """T_add = A + B, elementwise, fp16 / fp32 / int8 (int8 wraps)."""
    _dev(A, B, T_add)
    if not (A.dtype == B.dtype == T_add.dtype) or not (A.shape == B.shape == T_add.shape):
        raise ValueError("add: A, B, T_add must agree in dtype and shape")
    name, _ = _ELT[("add", A.dtype)]
    n, H = _rows_cols(A)
    check(getattr(lib(), name)(_p(A), _p(B), _p(T_add), n, H, _cfg(cfg), _stream()), name)


def copy(A: torch.Tensor, B: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """B = A, bit for bit."""
    _dev(A, B)
    if A.dtype != B.dtype or A.shape != B.shape:
        raise ValueError("copy: A and B must agree in dtype and shape")
    name, _ = _ELT[("copy", A.dtype)]
    n, H = _rows_cols(A)
    check(getattr(lib(), name)(_p(A), _p(B), n, H, _cfg(cfg), _stream()), name)


def cast(A: torch.Tensor, compute: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """compute = Cast(A): fp16 -> fp32 (exact) or fp32 -> fp16 (round to nearest even, overflow to inf)."""
    _dev(A, compute)
    if A.shape != compute.shape:
        raise ValueError("cast: shapes differ")
    key = (A.dtype, compute.dtype)
    if key == (torch.float16, torch.float32):
        name = "dtas_cast_f16_f32"
    elif key == (torch.float32, torch.float16):
        name = "dtas_cast_f32_f16"
    else:
        raise ValueError(f"cast: no kernel for {A.dtype} -> {compute.dtype}")
    n, H = _rows_cols(A)
    check(getattr(lib(), name)(_p(A), _p(compute), n, H, _cfg(cfg), _stream()), name)


def layer_norm(x: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor, out: torch.Tensor, eps: float = 1e-5,
               cfg: Optional[DtasConfig] = None) -> None:
    """fused_layer_norm_cast1: fp32 x, gamma, beta -> fp16 out, over the last axis."""
    _dev(x, gamma, beta, out)
    n, H = _rows_cols(x)
    if x.dtype != torch.float32 or gamma.dtype != torch.float32 or beta.dtype != torch.float32 or out.dtype != torch.float16:
        raise ValueError("layer_norm: expects fp32 x/gamma/beta and fp16 out")
    if out.shape != x.shape or gamma.numel() != H or beta.numel() != H:
        raise ValueError("layer_norm: shape mismatch")
    check(lib().dtas_layer_norm_f32_f16(_p(x), _p(gamma), _p(beta), _p(out), n, H, eps, _cfg(cfg), _stream()),
          "dtas_layer_norm_f32_f16")


def layer_norm_f32(x: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor, out: torch.Tensor, eps: float = 1e-5) -> None:
    """layer_norm / layer_norm1 (dolly-v2-3b-q0f16/before_dl.py:846-896): layer norm over the last axis, fp32 in and out."""
    _dev(x, gamma, beta, out)
    if any(t.dtype != torch.float32 for t in (x, gamma, beta, out)) or out.shape != x.shape:
        raise ValueError("layer_norm_f32: expects fp32 tensors and an output of x's shape")
    n, H = _rows_cols(x)
    if gamma.numel() != H or beta.numel() != H:
        raise ValueError("layer_norm_f32: gamma and beta hold one value per column")
    check(lib().dtas_layer_norm_f32(_p(x), _p(gamma), _p(beta), _p(out), n, H, eps, _stream()), "dtas_layer_norm_f32")


def rms_norm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, eps: float = 1e-5,
             cfg: Optional[DtasConfig] = None) -> None:
    """out = x * rsqrt(mean(x^2) + eps) * w over the last axis; fp16 in/out, fp32 arithmetic."""
    _dev(x, w, out)
    n, H = _rows_cols(x)
    if x.dtype != torch.float16 or w.dtype != torch.float16 or out.dtype != torch.float16:
        raise ValueError("rms_norm: expects fp16 x, w, out")
    if out.shape != x.shape or w.numel() != H:
        raise ValueError("rms_norm: shape mismatch")
    check(lib().dtas_rms_norm_f16(_p(x), _p(w), _p(out), n, H, eps, _cfg(cfg), _stream()), "dtas_rms_norm_f16")


def softmax(A: torch.Tensor, out: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """fused_softmax_cast: softmax over the last axis, fp32 or fp16 in, fp16 out."""
    _dev(A, out)
    if out.dtype != torch.float16 or out.shape != A.shape:
        raise ValueError("softmax: out must be fp16 with A's shape")
    rows, cols = _rows_cols(A)
    if A.dtype == torch.float32:
        name = "dtas_softmax_f32_f16"
    elif A.dtype == torch.float16:
        name = "dtas_softmax_f16"
    else:
        raise ValueError(f"softmax: no kernel for {A.dtype}")
    check(getattr(lib(), name)(_p(A), _p(out), rows, cols, _cfg(cfg), _stream()), name)


def gemv(x: torch.Tensor, W: torch.Tensor, bias: Optional[torch.Tensor], y: torch.Tensor,
         cfg: Optional[DtasConfig] = None, epilogue: int = 0, res1: Optional[torch.Tensor] = None,
         res2: Optional[torch.Tensor] = None) -> None:
    """y[N] = epilogue(W[N,K] . x[K]); fp16, fp32 accumulate.  epilogue (``_lib.EPI_*``) as for gemm: 0 ``+ bias``
    (fused_NT_matmul10_add5); 1 ``(res1 + (mm + bias)) + res2`` (fused_NT_matmul8_add5_add7_add7,
    before_dl.py:408-439); 2 the same into an fp32 y (.._cast5, :442-480); 3 ``gelu(mm + bias)``
    (fused_NT_matmul9_add6_gelu1, :483-549)."""
    _dev(x, W, bias, y, res1, res2)
    N, K = W.shape
    if x.numel() != K or y.numel() != N or any(t is not None and t.numel() != N for t in (bias, res1, res2)):
        raise ValueError("gemv: shape mismatch")
    want_out = torch.float32 if epilogue == _lib.EPI_BIAS_ADD2_CAST_F32 else torch.float16
    if any(t.dtype != torch.float16 for t in (x, W)) or y.dtype != want_out or \
            any(t is not None and t.dtype != torch.float16 for t in (bias, res1, res2)):
        raise ValueError("gemv: expects fp16 tensors (and an fp32 y for the cast epilogue)")
    if epilogue == _lib.EPI_BIAS and res1 is None and res2 is None:
        check(lib().dtas_gemv_f16(_p(x), _p(W), _p(bias), _p(y), N, K, _cfg(cfg), _stream()), "dtas_gemv_f16")
    else:
        check(lib().dtas_gemv_f16_fused(_p(x), _p(W), _p(bias), _p(res1), _p(res2), _p(y), N, K, epilogue, _cfg(cfg),
                                        _stream()), "dtas_gemv_f16_fused")


def gemv_f32(x: torch.Tensor, W: torch.Tensor, y: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """y[N] = W[N,K] . x[K], all fp32: NT_matmul5 (dolly-v2-3b-q0f16/before_dl.py:8-19)."""
    _dev(x, W, y)
    N, K = W.shape
    if x.numel() != K or y.numel() != N:
        raise ValueError("gemv_f32: shape mismatch")
    if any(t.dtype != torch.float32 for t in (x, W, y)):
        raise ValueError("gemv_f32: expects fp32 tensors")
    check(lib().dtas_gemv_f32(_p(x), _p(W), _p(y), N, K, _cfg(cfg), _stream()), "dtas_gemv_f32")


def gemm(A: torch.Tensor, W: torch.Tensor, bias: Optional[torch.Tensor], C: torch.Tensor,
         cfg: Optional[DtasConfig] = None, epilogue: int = 0, res1: Optional[torch.Tensor] = None,
         res2: Optional[torch.Tensor] = None) -> None:
    """C[M,N] = epilogue(A[M,K] . W[N,K]^T); fp16 operands, fp32 accumulate on MFMA.  M is every leading
    extent of A flattened.  epilogue (``_lib.EPI_*``): 0 ``+ bias``; 1 ``(res1 + (mm + bias)) + res2``;
    2 the same into an fp32 C; 3 ``gelu(mm + bias)`` -- each step rounded to fp16 as in the fused
    PrimFuncs (before_dl.py:163-318)."""
    _dev(A, W, bias, C, res1, res2)
    N, K = W.shape
    if A.shape[-1] != K or C.shape[-1] != N:
        raise ValueError("gemm: inner extents differ")
    M = A.numel() // K if K else C.numel() // max(N, 1)
    if C.numel() != M * N or (bias is not None and bias.numel() != N):
        raise ValueError("gemm: shape mismatch")
    want_out = torch.float32 if epilogue == _lib.EPI_BIAS_ADD2_CAST_F32 else torch.float16
    if any(t.dtype != torch.float16 for t in (A, W)) or C.dtype != want_out or \
            any(t is not None and t.dtype != torch.float16 for t in (bias, res1, res2)):
        raise ValueError("gemm: expects fp16 operands (and an fp32 C for the cast epilogue)")
    if any(t is not None and t.numel() != M * N for t in (res1, res2)):
        raise ValueError("gemm: residual shape mismatch")
    if epilogue == _lib.EPI_BIAS and res1 is None and res2 is None:
        check(lib().dtas_gemm_f16(_p(A), _p(W), _p(bias), _p(C), M, N, K, _cfg(cfg), _stream()), "dtas_gemm_f16")
    else:
        check(lib().dtas_gemm_f16_fused(_p(A), _p(W), _p(bias), _p(res1), _p(res2), _p(C), M, N, K, epilogue, _cfg(cfg),
                                        _stream()), "dtas_gemm_f16_fused")


def attn_scores(Q: torch.Tensor, K: torch.Tensor, mask: torch.Tensor, out: torch.Tensor, scale: float = 0.11179039301310044,
                cfg: Optional[DtasConfig] = None) -> None:
    """out[h,n,m] (fp32) = min(max(fp16(Q[h,n,:] . K[h,m,:]) * fp16(scale), -65504), mask[n,m]), each step an fp16
    value: fused_NT_matmul1_divide_maximum_minimum_cast2 (before_dl.py:116-160).  Q (..., heads, n, d),
    K (..., heads, m, d), mask (..., n, m) with leading extents of 1."""
    _dev(Q, K, mask, out)
    heads, n, d = Q.shape[-3:]
    m = K.shape[-2]
    if K.shape[-3:] != (heads, m, d) or mask.shape[-2:] != (n, m) or out.shape[-3:] != (heads, n, m):
        raise ValueError("attn_scores: shape mismatch")
    if Q.numel() != heads * n * d or K.numel() != heads * m * d or mask.numel() != n * m or out.numel() != heads * n * m:
        raise ValueError("attn_scores: leading extents must be 1")
    if any(t.dtype != torch.float16 for t in (Q, K, mask)) or out.dtype != torch.float32:
        raise ValueError("attn_scores: expects fp16 inputs and an fp32 output")
    check(lib().dtas_attn_scores_f16_f32(_p(Q), _p(K), _p(mask), _p(out), heads, n, m, d, scale, _cfg(cfg), _stream()),
          "dtas_attn_scores_f16_f32")


def attn_pv(P: torch.Tensor, V: torch.Tensor, out: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """out[h,n,:] = sum_k P[h,n,k] * V[h,k,:], fp16 with fp32 accumulation: matmul8 (before_dl.py:915-929) and,
    with n = 1, matmul10 (:899-912).  P (..., heads, n, m), V (..., heads, m, d), out (..., heads, n, d) with
    leading extents of 1."""
    _dev(P, V, out)
    heads, n, m = P.shape[-3:]
    d = V.shape[-1]
    if V.shape[-3:] != (heads, m, d) or out.shape[-3:] != (heads, n, d):
        raise ValueError("attn_pv: shape mismatch")
    if P.numel() != heads * n * m or V.numel() != heads * m * d or out.numel() != heads * n * d:
        raise ValueError("attn_pv: leading extents must be 1")
    if any(t.dtype != torch.float16 for t in (P, V, out)):
        raise ValueError("attn_pv: expects fp16 buffers")
    check(lib().dtas_attn_pv_f16(_p(P), _p(V), _p(out), heads, n, m, d, _cfg(cfg), _stream()), "dtas_attn_pv_f16")


def _q8_shapes(what: str, Wq: torch.Tensor, scale: torch.Tensor, scale_dtype=torch.float16):
    if Wq.dim() != 2 or Wq.dtype not in (torch.int32, torch.uint32) or scale.dtype != scale_dtype:
        raise ValueError(f"{what}: expects 32-bit words [N, K/4] and {str(scale_dtype).split('.')[-1]} scales [N, K/32]")
    N, K = Wq.shape[0], Wq.shape[1] * 4
    if K % 32 != 0 or tuple(scale.shape) != (N, K // 32):
        raise ValueError(f"{what}: K = {K} and scales {tuple(scale.shape)} do not form groups of 32")
    return N, K


def decode_q8(Wq: torch.Tensor, scale: torch.Tensor, W: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """W[N,K] (fp16) = (fp16(byte) - 127) * scale[N, K/32]; element j of a row is byte j % 4 of word j / 4 of
    Wq[N, K/4]: fused_decode3 (dolly-v2-3b-q8f16_1/before_dl.py:335-343)."""
    _dev(Wq, scale, W)
    N, K = _q8_shapes("decode_q8", Wq, scale)
    if W.dtype != torch.float16 or W.numel() != N * K:
        raise ValueError("decode_q8: expects an fp16 output of N * K elements")
    check(lib().dtas_decode_q8_f16(_p(Wq), _p(scale), _p(W), N, K, _cfg(cfg), _stream()), "dtas_decode_q8_f16")


def attn_mask(out: torch.Tensor) -> None:
    """out (..., n, m) fp16 = the causal mask of n query positions against m >= n key positions (65504 where a key
    may be seen, -65504 where not): fused_min_max_triu_te_broadcast_to + extend_te, and full for n = 1
    (dolly-v2-3b-q0f16/before_dl.py:642-658, :68-80, :83-93)."""
    _dev(out)
    n, m = out.shape[-2:]
    if out.dtype != torch.float16 or out.numel() != n * m:
        raise ValueError("attn_mask: expects an fp16 output (..., n, m) with leading extents of 1")
    check(lib().dtas_attn_mask_f16(_p(out), n, m, _stream()), "dtas_attn_mask_f16")


def softmax_temperature(logits: torch.Tensor, temperature: torch.Tensor, out: torch.Tensor) -> None:
    """softmax_with_temperature (dolly-v2-3b-q0f16/before_dl.py:4154-4161): out = softmax(logits / temperature) over
    the last axis, fp32 in and out; `temperature` is a 0-d (or one-element) fp32 device tensor."""
    _dev(logits, temperature, out)
    if logits.dtype != torch.float32 or out.dtype != torch.float32 or temperature.dtype != torch.float32:
        raise ValueError("softmax_temperature: logits, temperature and out must be fp32")
    if out.shape != logits.shape or temperature.numel() != 1:
        raise ValueError("softmax_temperature: out must have the logits' shape and temperature one element")
    rows, cols = _rows_cols(logits)
    check(lib().dtas_softmax_temperature_f32(_p(logits), _p(temperature), _p(out), rows, cols, _stream()),
          "dtas_softmax_temperature_f32")


def divide(A: torch.Tensor, B: torch.Tensor, out: torch.Tensor) -> None:
    """divide2 (dolly-v2-3b-q0f16/before_dl.py:57-65): out = A / B, fp32, B a 0-d (one-element) device tensor."""
    _dev(A, B, out)
    if any(t.dtype != torch.float32 for t in (A, B, out)) or out.shape != A.shape or B.numel() != 1:
        raise ValueError("divide: expects fp32 A and out of one shape and a one-element fp32 B")
    check(lib().dtas_divide_f32(_p(A), _p(B), _p(out), A.numel(), _stream()), "dtas_divide_f32")


def softmax_f32(A: torch.Tensor, out: torch.Tensor) -> None:
    """softmax2 (dolly-v2-3b-q0f16/before_dl.py:1062-1096): softmax over the last axis, fp32 in and out."""
    _dev(A, out)
    if A.dtype != torch.float32 or out.dtype != torch.float32 or out.shape != A.shape:
        raise ValueError("softmax_f32: expects fp32 A and out of one shape")
    rows, cols = _rows_cols(A)
    check(lib().dtas_softmax_f32(_p(A), _p(out), rows, cols, _stream()), "dtas_softmax_f32")


def split3(A: torch.Tensor, out0: torch.Tensor, out1: torch.Tensor, out2: torch.Tensor) -> None:
    """split / fused_reshape7_split1 (dolly-v2-3b-q0f16/before_dl.py:1099-1125, :661-688): A (..., 3 d) fp16 cut into
    three (..., d) buffers along the last axis."""
    _dev(A, out0, out1, out2)
    d3 = A.shape[-1]
    if d3 % 3 != 0:
        raise ValueError("split3: the last extent must be a multiple of 3")
    d = d3 // 3
    rows = A.numel() // d3 if d3 else 0
    for o in (out0, out1, out2):
        if o.dtype != torch.float16 or o.shape[-1] != d or o.numel() != rows * d:
            raise ValueError("split3: each output must be fp16 (..., d) with A's leading extents")
    if A.dtype != torch.float16:
        raise ValueError("split3: A must be fp16")
    check(lib().dtas_split3_f16(_p(A), _p(out0), _p(out1), _p(out2), rows, d, _stream()), "dtas_split3_f16")


def swap_axes(A: torch.Tensor, out: torch.Tensor) -> None:
    """out (..., b, a, d) = A (..., a, b, d) with leading extents of 1, fp16: transpose6 / transpose7
    (dolly-v2-3b-q0f16/before_dl.py:1177-1203)."""
    _dev(A, out)
    a, b, d = A.shape[-3:]
    if A.dtype != torch.float16 or out.dtype != torch.float16 or A.numel() != a * b * d or tuple(out.shape[-3:]) != (b, a, d) \
            or out.numel() != a * b * d:
        raise ValueError("swap_axes: expects fp16 A (..., a, b, d) and out (..., b, a, d) with leading extents of 1")
    check(lib().dtas_swap_axes_f16(_p(A), _p(out), a, b, d, _stream()), "dtas_swap_axes_f16")


def rotary(A: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, out: torch.Tensor, m: int,
           cfg: Optional[DtasConfig] = None) -> None:
    """rotary_embedding (dolly-v2-3b-q0f16/before_dl.py:1023-1035; rotary_embedding1 :1038-1047): A and out
    (..., n, heads, d) fp16 with leading extents of 1, cos / sin [max_pos, rot] fp16; position s of A takes the
    tables' row m + s - n (m = length of the whole sequence)."""
    _dev(A, cos, sin, out)
    if any(t.dtype != torch.float16 for t in (A, cos, sin, out)) or cos.dim() != 2 or cos.shape != sin.shape or A.dim() < 3:
        raise ValueError("rotary: expects fp16 A (..., n, heads, d) and fp16 tables [max_pos, rot]")
    n, heads, d = A.shape[-3:]
    if A.numel() != n * heads * d or out.shape != A.shape:
        raise ValueError("rotary: leading extents must be 1 and out must have A's shape")
    check(lib().dtas_rotary_f16(_p(A), _p(cos), _p(sin), _p(out), n, int(m), heads, d, cos.shape[1], cos.shape[0], _cfg(cfg),
                                _stream()), "dtas_rotary_f16")


def take(A: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """out[n,H] = A[ids[i], :], the fp16 embedding lookup: take (dolly-v2-3b-q0f16/before_dl.py:1151-1163) and, one row,
    take1 (:1166-1174).  ids int32; values outside [0, V) are clipped to the nearest row."""
    _dev(A, ids, out)
    if A.dim() != 2 or A.dtype != torch.float16 or ids.dtype != torch.int32 or out.dtype != torch.float16:
        raise ValueError("take: expects an fp16 table [V, H], int32 ids[n] and an fp16 output")
    V, H = A.shape
    n = ids.numel()
    if out.numel() != n * H:
        raise ValueError("take: the output holds n * H elements")
    check(lib().dtas_take_f16(_p(A), _p(ids), _p(out), n, V, H, _cfg(cfg), _stream()), "dtas_take_f16")


def take_q8(Wq: torch.Tensor, scale: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """out[n,K] (fp16) = rows ids[i] of decode_q8(Wq, scale), the embedding lookup of the 8-bit model:
    fused_fused_decode1_take1 (dolly-v2-3b-q8f16_1/before_dl.py:357-369) and, one row, fused_fused_decode1_take
    (:346-355).  ids int32; values outside [0, V) are clipped to the nearest row."""
    _dev(Wq, scale, ids, out)
    V, K = _q8_shapes("take_q8", Wq, scale)
    n = ids.numel()
    if ids.dtype != torch.int32 or out.dtype != torch.float16 or out.numel() != n * K:
        raise ValueError("take_q8: expects int32 ids[n] and an fp16 output of n * K elements")
    check(lib().dtas_take_q8_f16(_p(Wq), _p(scale), _p(ids), _p(out), n, V, K, _cfg(cfg), _stream()), "dtas_take_q8_f16")


def gemv_q8_f32(x: torch.Tensor, Wq: torch.Tensor, scale: torch.Tensor, y: torch.Tensor, cfg: Optional[DtasConfig] = None) -> None:
    """fp32 y[N] = x[K] . W^T with W = float32(byte - 127) * scale[N, K/32] (fp32 scales), never written: the vocabulary
    projection of the 8-bit model, fused_fused_decode6_NT_matmul5 (dolly-v2-3b-q8f16_1/before_dl.py:640-657)."""
    _dev(x, Wq, scale, y)
    N, K = _q8_shapes("gemv_q8_f32", Wq, scale, torch.float32)
    if x.numel() != K or y.numel() != N:
        raise ValueError("gemv_q8_f32: shape mismatch")
    if x.dtype != torch.float32 or y.dtype != torch.float32:
        raise ValueError("gemv_q8_f32: expects fp32 x and y")
    check(lib().dtas_gemv_q8_f32(_p(x), _p(Wq), _p(scale), _p(y), N, K, _cfg(cfg), _stream()), "dtas_gemv_q8_f32")


def gemv_q8(x: torch.Tensor, Wq: torch.Tensor, scale: torch.Tensor, bias: Optional[torch.Tensor], y: torch.Tensor,
            cfg: Optional[DtasConfig] = None, epilogue: int = 0) -> None:
    """y[N] = x[K] . decode_q8(Wq, scale)^T (+ bias[N]; ``_lib.EPI_BIAS_GELU``: then GELU), the weights dequantised
    in registers: fused_fused_decode2_fused_NT_matmul_add / fused_fused_decode4_fused_NT_matmul3_add2_gelu
    (dolly-v2-3b-q8f16_1/before_dl.py:401-426, :428-502)."""
    _dev(x, Wq, scale, bias, y)
    N, K = _q8_shapes("gemv_q8", Wq, scale)
    if x.numel() != K or y.numel() != N or (bias is not None and bias.numel() != N):
        raise ValueError("gemv_q8: shape mismatch")
    if any(t.dtype != torch.float16 for t in (x, y)) or (bias is not None and bias.dtype != torch.float16):
        raise ValueError("gemv_q8: expects fp16 x, bias and y")
    check(lib().dtas_gemv_q8_f16(_p(x), _p(Wq), _p(scale), _p(bias), _p(y), N, K, epilogue, _cfg(cfg), _stream()),
          "dtas_gemv_q8_f16")


def gemm_q8(A: torch.Tensor, Wq: torch.Tensor, scale: torch.Tensor, bias: Optional[torch.Tensor], C: torch.Tensor,
            cfg: Optional[DtasConfig] = None, epilogue: int = 0, res1: Optional[torch.Tensor] = None,
            res2: Optional[torch.Tensor] = None) -> None:
    """C[M,N] = epilogue(A[M,K] . decode_q8(Wq, scale)^T), the weights dequantised on their way into the LDS: the
    dynamic-n q8f16_1 PrimFuncs (dolly-v2-3b-q8f16_1/before_dl.py:371-399, :504-581); epilogues as ``gemm``."""
    _dev(A, Wq, scale, bias, C, res1, res2)
    N, K = _q8_shapes("gemm_q8", Wq, scale)
    if A.shape[-1] != K or C.shape[-1] != N:
        raise ValueError("gemm_q8: inner extents differ")
    M = A.numel() // K if K else C.numel() // max(N, 1)
    want_out = torch.float32 if epilogue == _lib.EPI_BIAS_ADD2_CAST_F32 else torch.float16
    if A.dtype != torch.float16 or C.dtype != want_out or any(t is not None and t.dtype != torch.float16 for t in (bias, res1, res2)):
        raise ValueError("gemm_q8: expects fp16 A, bias and residuals (and an fp32 C for the cast epilogue)")
    if C.numel() != M * N or (bias is not None and bias.numel() != N) or any(t is not None and t.numel() != M * N for t in (res1, res2)):
        raise ValueError("gemm_q8: shape mismatch")
    check(lib().dtas_gemm_q8_f16_fused(_p(A), _p(Wq), _p(scale), _p(bias), _p(res1), _p(res2), _p(C), M, N, K, epilogue,
                                       _cfg(cfg), _stream()), "dtas_gemm_q8_f16_fused")

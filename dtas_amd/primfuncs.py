"""The PrimFunc signatures the kernels stand behind, as ``PrimFunc`` descriptors.

Each constructor cites the TVMScript it restates (paths relative to the reference checkout).
Parameter order and the destination-passing convention (output buffer last) are the reference's;
the hidden size and the static matmul extents are arguments because the benchmark configs use
4096-wide shapes where the reference's model uses 2560.
"""
from __future__ import annotations

from typing import Optional

from .common.analisys import Block, Buffer, IRModule, PrimFunc


def add(dtype: str = "float16", hidden: int = 2560) -> PrimFunc:
    """T_add = A + B over (1, n, hidden): tuning_test/tune_ele_add.py:10-22 (committed as int8;
    fp16 / fp32 artefacts under experiment/dtas_tuned/elementwise/add/)."""
    shape = (1, "n", hidden)
    return PrimFunc("add", [Buffer("A", shape, dtype), Buffer("B", shape, dtype), Buffer("T_add", shape, dtype)],
                    [Block("T_add", "SSS", ["A", "B"], ["T_add"])], op="add",
                    attrs={"op_pattern": 0, "tir.noalias": True})


def copy(dtype: str = "float32", hidden: int = 2560) -> PrimFunc:
    """B = A over (1, n, hidden): tuning_test/tune_ele_copy.py:10-21."""
    shape = (1, "n", hidden)
    return PrimFunc("copy", [Buffer("A", shape, dtype), Buffer("B", shape, dtype)],
                    [Block("B", "SSS", ["A"], ["B"])], op="copy", attrs={"tir.noalias": True})


def cast(src: str = "float16", dst: str = "float32", hidden: int = 2560) -> PrimFunc:
    """compute = Cast(dst, A) over (1, n, hidden): tuning_test/tune_cast.py:10-21 (fp16 -> fp32)."""
    shape = (1, "n", hidden)
    return PrimFunc("cast", [Buffer("A", shape, src), Buffer("compute", shape, dst)],
                    [Block("compute", "SSS", ["A"], ["compute"])], op="cast", attrs={"tir.noalias": True})


def fused_layer_norm_cast1(hidden: int = 2560) -> PrimFunc:
    """LayerNorm fp32 -> fp16 with gamma/beta: experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:607-636."""
    return PrimFunc(
        "fused_layer_norm_cast1",
        [Buffer("lv6", (1, "n", hidden), "float32"), Buffer("param_1", (hidden,), "float32"),
         Buffer("param_2", (hidden,), "float32"), Buffer("compute_intermediate", (1, "n", hidden), "float16")],
        [Block("A_red_temp", "SSR", ["lv6"], ["A_red_temp_v0", "A_red_temp_v1"]),
         Block("T_layer_norm", "SSS", ["lv6", "A_red_temp_v0", "A_red_temp_v1", "param_1", "param_2"],
               ["T_layer_norm_intermediate"]),
         Block("compute", "SSS", ["T_layer_norm_intermediate"], ["compute_intermediate"])],
        op="layer_norm", attrs={"tir.noalias": True, "eps": 1e-5})


def layer_norm(hidden: int = 2560, decode: bool = False) -> PrimFunc:
    """LayerNorm fp32 -> fp32 (the graph's last one): layer_norm (dolly-v2-3b-q0f16/before_dl.py:846-872; n dynamic) or,
    with ``decode``, layer_norm1 (:874-896; one row).  Parameters: A, B (gamma), C (beta), T_layer_norm."""
    n = 1 if decode else "n"
    return PrimFunc(
        "layer_norm1" if decode else "layer_norm",
        [Buffer("A", (1, n, hidden), "float32"), Buffer("B", (hidden,), "float32"), Buffer("C", (hidden,), "float32"),
         Buffer("T_layer_norm", (1, n, hidden), "float32")],
        [Block("A_red_temp", "SSR", ["A"], ["A_red_temp_v0", "A_red_temp_v1"]),
         Block("T_layer_norm", "SSS", ["A", "A_red_temp_v0", "A_red_temp_v1", "B", "C"], ["T_layer_norm"])],
        op="layer_norm_f32", attrs={"tir.noalias": True, "eps": 1e-5})


def rms_norm(hidden: int = 4096, eps: float = 1e-5) -> PrimFunc:
    """RMSNorm fp16 with fp16 weight; no counterpart in the reference (the benchmark's norm)."""
    return PrimFunc(
        "rms_norm",
        [Buffer("x", ("n", hidden), "float16"), Buffer("weight", (hidden,), "float16"),
         Buffer("out", ("n", hidden), "float16")],
        [Block("sum_sq", "SR", ["x"], ["sum_sq"]), Block("norm", "SS", ["x", "sum_sq", "weight"], ["out"])],
        op="rms_norm", attrs={"tir.noalias": True, "eps": eps})


def fused_softmax_cast(rows: int = 1000, dtype: str = "float32") -> PrimFunc:
    """Softmax over the dynamic last axis of (1, rows, n), fp16 out:
    experiment/dtas_tuned/general_reduction/softmax/profile_dlight.py:8-52."""
    return PrimFunc(
        "fused_softmax_cast",
        [Buffer("A", (1, rows, "n"), dtype), Buffer("compute_intermediate", (1, rows, "n"), "float16")],
        _softmax_blocks("A"), op="softmax", attrs={"tir.noalias": True})


def fused_softmax_cast3(heads: int = 32, dtype: str = "float32") -> PrimFunc:
    """Softmax over m of (1, heads, n, m), fp16 out: before_dl.py:756-800 (two dynamic extents)."""
    return PrimFunc(
        "fused_softmax_cast3",
        [Buffer("lv38", (1, heads, "n", "m"), dtype), Buffer("compute_intermediate", (1, heads, "n", "m"), "float16")],
        _softmax_blocks("lv38"), op="softmax", attrs={"tir.noalias": True})


def softmax_scores(heads: int = 32) -> PrimFunc:
    """The benchmark's attention-score softmax: fp16 [heads*n, n] -> fp16, one dynamic extent n
    that is both the row count factor and the row length."""
    return PrimFunc(
        "softmax_scores",
        [Buffer("scores", (heads, "n", "n"), "float16"), Buffer("out", (heads, "n", "n"), "float16")],
        _softmax_blocks("scores"), op="softmax", attrs={"tir.noalias": True})


def _softmax_blocks(src: str):
    return [Block("T_softmax_maxelem", "SSR", [src], ["T_softmax_maxelem"]),
            Block("T_softmax_exp", "SSS", [src, "T_softmax_maxelem"], ["T_softmax_exp"]),
            Block("T_softmax_expsum", "SSR", ["T_softmax_exp"], ["T_softmax_expsum"]),
            Block("T_softmax_norm", "SSS", ["T_softmax_exp", "T_softmax_expsum"], ["T_softmax_norm"]),
            Block("compute", "SSS", ["T_softmax_norm"], ["compute_intermediate"])]


def fused_NT_matmul_add_gemv(N: int = 2560, K: int = 10240, bias: bool = True,
                             name: Optional[str] = None) -> PrimFunc:
    """y(1,1,N) = x(1,1,K) . W(N,K)^T (+ bias): fused_NT_matmul10_add5, before_dl.py:96-113."""
    params = [Buffer("lv1825", (1, 1, K), "float16"), Buffer("param_1110", (N, K), "float16")]
    blocks = [Block("NT_matmul", "SSSR", ["lv1825", "param_1110"], ["NT_matmul_intermediate"])]
    if bias:
        params.append(Buffer("param_1210", (N,), "float16"))
        blocks.append(Block("T_add", "SSS", ["NT_matmul_intermediate", "param_1210"], ["T_add_intermediate"]))
    params.append(Buffer("T_add_intermediate", (1, 1, N), "float16"))
    return PrimFunc(name or ("fused_NT_matmul10_add5" if bias else "NT_matmul10"), params, blocks, op="matmul",
                    attrs={"tir.noalias": True})


def NT_matmul_f32(N: int = 50280, K: int = 2560, name: Optional[str] = None) -> PrimFunc:
    """y(1,1,N) = x(1,1,K) . W(N,K)^T, all fp32: NT_matmul5 (the vocabulary projection), before_dl.py:8-19."""
    params = [Buffer("A", (1, 1, K), "float32"), Buffer("B", (N, K), "float32"), Buffer("NT_matmul", (1, 1, N), "float32")]
    blocks = [Block("NT_matmul", "SSSR", ["A", "B"], ["NT_matmul"])]
    return PrimFunc(name or "NT_matmul5", params, blocks, op="gemv_f32", attrs={"tir.noalias": True})


def fused_NT_matmul_add_gemm(N: int = 2560, K: int = 10240, bias: bool = True,
                             name: Optional[str] = None) -> PrimFunc:
    """C(1,n,N) = A(1,n,K) . W(N,K)^T (+ bias), n dynamic: fused_NT_matmul4_add1, before_dl.py:320-341."""
    params = [Buffer("lv55", (1, "n", K), "float16"), Buffer("param_11", (N, K), "float16")]
    blocks = [Block("NT_matmul", "SSSR", ["lv55", "param_11"], ["NT_matmul_intermediate"])]
    if bias:
        params.append(Buffer("param_12", (N,), "float16"))
        blocks.append(Block("T_add", "SSS", ["NT_matmul_intermediate", "param_12"], ["T_add_intermediate"]))
    params.append(Buffer("T_add_intermediate", (1, "n", N), "float16"))
    return PrimFunc(name or ("fused_NT_matmul4_add1" if bias else "NT_matmul4"), params, blocks, op="matmul",
                    attrs={"tir.noalias": True})


def fused_NT_matmul_add_add_add(N: int = 2560, K: int = 2560, cast: bool = False,
                                name: Optional[str] = None, decode: bool = False) -> PrimFunc:
    """out(1,n,N) = (lv58 + (A(1,n,K) . W(N,K)^T + bias)) + lv2, every step an fp16 tensor; with ``cast`` the
    result is widened to fp32: fused_NT_matmul2_add1_add3_add3, before_dl.py:163-200, and
    fused_NT_matmul2_add1_add3_add3_cast, :202-246.  Parameter order as there: A, W, bias, res1, res2, out.
    ``decode``: the static one-row forms of the decode graph, fused_NT_matmul8_add5_add7_add7 (:408-439) and
    fused_NT_matmul8_add5_add7_add7_cast5 (:442-480)."""
    n = 1 if decode else "n"
    params = [Buffer("lv43", (1, n, K), "float16"), Buffer("param_7", (N, K), "float16"),
              Buffer("param_8", (N,), "float16"), Buffer("lv58", (1, n, N), "float16"),
              Buffer("lv2", (1, n, N), "float16")]
    blocks = [Block("NT_matmul", "SSSR", ["lv43", "param_7"], ["NT_matmul_intermediate"]),
              Block("T_add", "SSS", ["NT_matmul_intermediate", "param_8"], ["T_add_intermediate"]),
              Block("T_add_1", "SSS", ["lv58", "T_add_intermediate"], ["T_add_intermediate_1"]),
              Block("T_add_2", "SSS", ["T_add_intermediate_1", "lv2"], ["T_add_intermediate_1_2"])]
    if cast:
        blocks.append(Block("compute", "SSS", ["T_add_intermediate_1_2"], ["compute_intermediate"]))
        params.append(Buffer("compute_intermediate", (1, n, N), "float32"))
    else:
        params.append(Buffer("T_add_intermediate_1_2", (1, n, N), "float16"))
    stem = "fused_NT_matmul8_add5_add7_add7" if decode else "fused_NT_matmul2_add1_add3_add3"
    return PrimFunc(name or (stem + (("_cast5" if decode else "_cast") if cast else "")),
                    params, blocks, op="matmul", attrs={"tir.noalias": True, "epilogue": 2 if cast else 1})


def fused_NT_matmul_add_gelu(N: int = 10240, K: int = 2560, name: Optional[str] = None, decode: bool = False) -> PrimFunc:
    """out(1,n,N) = gelu(A(1,n,K) . W(N,K)^T + bias) with the erf form and an fp16 tensor after every step:
    fused_NT_matmul3_add2_gelu, before_dl.py:248-318.  Parameters: A, W, bias, out.  ``decode``: the static
    one-row form of the decode graph, fused_NT_matmul9_add6_gelu1 (:483-549)."""
    n = 1 if decode else "n"
    params = [Buffer("lv50", (1, n, K), "float16"), Buffer("param_9", (N, K), "float16"),
              Buffer("param_10", (N,), "float16"), Buffer("T_multiply_intermediate", (1, n, N), "float16")]
    blocks = [Block("NT_matmul", "SSSR", ["lv50", "param_9"], ["NT_matmul_intermediate"]),
              Block("T_add", "SSS", ["NT_matmul_intermediate", "param_10"], ["T_add_intermediate"]),
              Block("T_multiply", "SSS", ["T_add_intermediate"], ["T_multiply"]),
              Block("compute", "SSS", ["T_multiply"], ["compute"]),
              Block("compute_1", "SSS", ["compute"], ["compute_1"]),
              Block("compute_2", "SSS", ["compute_1"], ["compute_2"]),
              Block("T_multiply_1", "SSS", ["compute_2"], ["T_multiply_1"]),
              Block("T_add_1", "SSS", ["T_multiply_1"], ["T_add"]),
              Block("T_multiply_2", "SSS", ["T_add_intermediate", "T_add"], ["T_multiply_intermediate"])]
    return PrimFunc(name or ("fused_NT_matmul9_add6_gelu1" if decode else "fused_NT_matmul3_add2_gelu"), params, blocks,
                    op="matmul", attrs={"tir.noalias": True, "epilogue": 3})


def fused_NT_matmul_divide_maximum_minimum_cast(heads: int = 32, head_dim: int = 80,
                                                scale: float = 0.11179039301310044, name: Optional[str] = None) -> PrimFunc:
    """scores(1,heads,n,m) fp32 = min(max(fp16(Q(1,heads,n,d) . K(1,heads,m,d)^T) * fp16(scale), -65504), mask(1,1,n,m)):
    fused_NT_matmul1_divide_maximum_minimum_cast2, before_dl.py:116-160; n and m dynamic."""
    params = [Buffer("lv30", (1, heads, "n", head_dim), "float16"), Buffer("lv31", (1, heads, "m", head_dim), "float16"),
              Buffer("lv5", (1, 1, "n", "m"), "float16"), Buffer("compute_intermediate", (1, heads, "n", "m"), "float32")]
    blocks = [Block("NT_matmul", "SSSSR", ["lv30", "lv31"], ["NT_matmul_intermediate"]),
              Block("T_divide", "SSSS", ["NT_matmul_intermediate"], ["T_divide_intermediate"]),
              Block("T_maximum", "SSSS", ["T_divide_intermediate"], ["T_maximum_intermediate"]),
              Block("T_minimum", "SSSS", ["T_maximum_intermediate", "lv5"], ["T_minimum_intermediate"]),
              Block("compute", "SSSS", ["T_minimum_intermediate"], ["compute_intermediate"])]
    return PrimFunc(name or "fused_NT_matmul1_divide_maximum_minimum_cast2", params, blocks, op="attn_scores",
                    attrs={"tir.noalias": True, "scale": scale})


def matmul_pv(heads: int = 32, head_dim: int = 80, decode: bool = False, name: Optional[str] = None) -> PrimFunc:
    """out(1,heads,n,d) = P(1,heads,n,m) . V(1,heads,m,d), the attention output: matmul8 (before_dl.py:915-929;
    n and m dynamic) or, with ``decode``, matmul10 (:899-912; n = 1, m dynamic)."""
    n = 1 if decode else "n"
    params = [Buffer("A", (1, heads, n, "m"), "float16"), Buffer("B", (1, heads, "m", head_dim), "float16"),
              Buffer("matmul", (1, heads, n, head_dim), "float16")]
    blocks = [Block("matmul", "SSSSR", ["A", "B"], ["matmul"])]
    return PrimFunc(name or ("matmul10" if decode else "matmul8"), params, blocks, op="attn_pv", attrs={"tir.noalias": True})


def fused_decode(N: int = 2560, K: int = 2560, name: Optional[str] = None) -> PrimFunc:
    """W(N,K) fp16 = (fp16(byte) - 127) * scale(N, K/32) of 8-bit weights packed four to a uint32 word:
    fused_decode3, dolly-v2-3b-q8f16_1/before_dl.py:335-343."""
    params = [Buffer("model_params_9", (N, K // 4), "uint32"), Buffer("model_params_10", (N, K // 32), "float16"),
              Buffer("decode_intermediate", (N, K), "float16")]
    blocks = [Block("decode", "SS", ["model_params_9", "model_params_10"], ["decode_intermediate"])]
    return PrimFunc(name or "fused_decode3", params, blocks, op="decode_q8", attrs={"tir.noalias": True})


def take(V: int = 50280, H: int = 2560, decode: bool = False, name: Optional[str] = None) -> PrimFunc:
    """T_take(n,H) = A(V,H)[B(n), :], the fp16 embedding lookup: take (dolly-v2-3b-q0f16/before_dl.py:1151-1163; n dynamic)
    or, with ``decode``, take1 (:1166-1174; one row).  Parameters: A, B, T_take."""
    n = 1 if decode else "n"
    params = [Buffer("A", (V, H), "float16"), Buffer("B", (n,), "int32"), Buffer("T_take", (n, H), "float16")]
    blocks = [Block("T_take", "SS", ["A", "B"], ["T_take"])]
    return PrimFunc(name or ("take1" if decode else "take"), params, blocks, op="take", attrs={"tir.noalias": True})


def split(heads: int = 32, d: int = 80, decode: bool = False, name: Optional[str] = None) -> PrimFunc:
    """The fused projection cut into queries, keys and values, section s = columns [s d, (s + 1) d) of every head:
    split (dolly-v2-3b-q0f16/before_dl.py:1099-1125; A (1, n, heads, 3 d), n dynamic) or, with ``decode``,
    fused_reshape7_split1 (:661-688; A (1, 1, heads * 3 d), reshaped first).  Parameters: A and the three sections."""
    n = 1 if decode else "n"
    a_shape = (1, 1, heads * 3 * d) if decode else (1, n, heads, 3 * d)
    outs = ["T_split_sections", "T_split_sections_1", "T_split_sections_2"]
    params = [Buffer("A", a_shape, "float16")] + [Buffer(o, (1, n, heads, d), "float16") for o in outs]
    blocks = [Block(o, "SSSS", ["A"], [o]) for o in outs]
    return PrimFunc(name or ("fused_reshape7_split1" if decode else "split"), params, blocks, op="split3",
                    attrs={"tir.noalias": True, "heads": heads, "d": d})


def transpose(heads: int = 32, d: int = 80, back: bool = False, decode: bool = False, name: Optional[str] = None) -> PrimFunc:
    """T_transpose(1, heads, n, d) = A(1, n, heads, d): transpose6 (dolly-v2-3b-q0f16/before_dl.py:1177-1189) or, with
    ``back``, transpose7 (:1191-1203; (1, heads, n, d) -> (1, n, heads, d)); ``decode``: transpose8 (:1205-1213, n = 1)."""
    n = 1 if decode else "n"
    src, dst = ((1, heads, n, d), (1, n, heads, d)) if back else ((1, n, heads, d), (1, heads, n, d))
    params = [Buffer("A", src, "float16"), Buffer("T_transpose", dst, "float16")]
    blocks = [Block("T_transpose", "SSSS", ["A"], ["T_transpose"])]
    return PrimFunc(name or ("transpose8" if decode else "transpose7" if back else "transpose6"), params, blocks, op="swap_axes",
                    attrs={"tir.noalias": True})


def divide(V: int = 50280, name: Optional[str] = None) -> PrimFunc:
    """T_divide(1, 1, V) = A(1, 1, V) / B(), fp32: divide2 (dolly-v2-3b-q0f16/before_dl.py:57-65)."""
    params = [Buffer("A", (1, 1, V), "float32"), Buffer("B", (), "float32"), Buffer("T_divide", (1, 1, V), "float32")]
    return PrimFunc(name or "divide2", params, [Block("T_divide", "SSS", ["A", "B"], ["T_divide"])], op="divide",
                    attrs={"tir.noalias": True})


def softmax2(V: int = 50280, name: Optional[str] = None) -> PrimFunc:
    """T_softmax_norm(1, 1, V) = softmax(A(1, 1, V)), fp32 in and out: softmax2 (dolly-v2-3b-q0f16/before_dl.py:1062-1096)."""
    params = [Buffer("A", (1, 1, V), "float32"), Buffer("T_softmax_norm", (1, 1, V), "float32")]
    blocks = [Block("T_softmax_maxelem", "SSR", ["A"], ["T_softmax_maxelem"]),
              Block("T_softmax_exp", "SSS", ["A", "T_softmax_maxelem"], ["T_softmax_exp"]),
              Block("T_softmax_expsum", "SSR", ["T_softmax_exp"], ["T_softmax_expsum"]),
              Block("T_softmax_norm", "SSS", ["T_softmax_exp", "T_softmax_expsum"], ["T_softmax_norm"])]
    return PrimFunc(name or "softmax2", params, blocks, op="softmax_f32", attrs={"tir.noalias": True})


def softmax_with_temperature(V: int = 50280, name: Optional[str] = None) -> PrimFunc:
    """T_softmax_norm(1, 1, V) = softmax(A(1, 1, V) / B()), fp32: divide2 (dolly-v2-3b-q0f16/before_dl.py:57-65) and
    softmax2 (:1062-1096) as the graph's softmax_with_temperature chains them (:4154-4161).  Parameters: A (the
    logits), B (the temperature, a 0-d buffer), T_softmax_norm."""
    params = [Buffer("A", (1, 1, V), "float32"), Buffer("B", (), "float32"), Buffer("T_softmax_norm", (1, 1, V), "float32")]
    blocks = [Block("T_divide", "SSS", ["A", "B"], ["T_divide"]), Block("T_softmax_maxelem", "SSR", ["T_divide"], ["T_softmax_maxelem"]),
              Block("T_softmax_exp", "SSS", ["T_divide", "T_softmax_maxelem"], ["T_softmax_exp"]),
              Block("T_softmax_expsum", "SSR", ["T_softmax_exp"], ["T_softmax_expsum"]),
              Block("T_softmax_norm", "SSS", ["T_softmax_exp", "T_softmax_expsum"], ["T_softmax_norm"])]
    return PrimFunc(name or "softmax_with_temperature", params, blocks, op="softmax_temperature", attrs={"tir.noalias": True})


def fused_decode_take(V: int = 50280, K: int = 2560, decode: bool = False, name: Optional[str] = None) -> PrimFunc:
    """out(n,K) fp16 = rows ids(n) of the dequantised table: fused_fused_decode1_take1
    (dolly-v2-3b-q8f16_1/before_dl.py:357-369; n dynamic) or, with ``decode``, fused_fused_decode1_take (:346-355;
    one row).  Parameters: Wq, scale, ids, out."""
    n = 1 if decode else "n"
    params = [Buffer("lv775", (V, K // 4), "uint32"), Buffer("lv776", (V, K // 32), "float16"), Buffer("lv", (n,), "int32"),
              Buffer("T_take_intermediate", (n, K), "float16")]
    blocks = [Block("T_take", "SS", ["lv", "lv775", "lv776"], ["T_take_intermediate"])]
    return PrimFunc(name or ("fused_fused_decode1_take" if decode else "fused_fused_decode1_take1"), params, blocks,
                    op="take_q8", attrs={"tir.noalias": True})


def fused_decode_NT_matmul_f32(N: int = 50280, K: int = 2560, name: Optional[str] = None) -> PrimFunc:
    """y(1,1,N) fp32 = x(1,1,K) fp32 . W^T with W = float32(byte - 127) * scale(N, K/32) fp32:
    fused_fused_decode6_NT_matmul5, dolly-v2-3b-q8f16_1/before_dl.py:640-657.  Parameters: Wq, scale, x, out."""
    params = [Buffer("lv772", (N, K // 4), "uint32"), Buffer("lv773", (N, K // 32), "float32"), Buffer("lv771", (1, 1, K), "float32"),
              Buffer("NT_matmul_intermediate", (1, 1, N), "float32")]
    blocks = [Block("decode", "SS", ["lv772", "lv773"], ["decode_intermediate_intermediate"]),
              Block("NT_matmul", "SSSR", ["lv771", "decode_intermediate_intermediate"], ["NT_matmul_intermediate"])]
    return PrimFunc(name or "fused_fused_decode6_NT_matmul5", params, blocks, op="gemv_q8_f32", attrs={"tir.noalias": True})


def fused_decode_NT_matmul_add(N: int = 7680, K: int = 2560, gelu: bool = False, name: Optional[str] = None) -> PrimFunc:
    """y(1,1,N) = x(1,1,K) . decode(Wq, scale)^T + bias (then GELU): fused_fused_decode2_fused_NT_matmul_add
    (dolly-v2-3b-q8f16_1/before_dl.py:401-426) or, with ``gelu``, fused_fused_decode4_fused_NT_matmul3_add2_gelu
    (:428-502; N = 10240).  Parameters: Wq, scale, x, bias, out."""
    out = "T_multiply_intermediate_intermediate" if gelu else "T_add_intermediate_intermediate"
    params = [Buffer("lv4", (N, K // 4), "uint32"), Buffer("lv5", (N, K // 32), "float16"), Buffer("lv3", (1, 1, K), "float16"),
              Buffer("param_8", (N,), "float16"), Buffer(out, (1, 1, N), "float16")]
    blocks = [Block("decode", "SS", ["lv4", "lv5"], ["decode_intermediate_intermediate"]),
              Block("NT_matmul", "SSSR", ["lv3", "decode_intermediate_intermediate"], ["NT_matmul_intermediate"]),
              Block("T_add", "SSS", ["NT_matmul_intermediate", "param_8"], [out if not gelu else "T_add_intermediate"])]
    if gelu:
        blocks.append(Block("T_multiply_2", "SSS", ["T_add_intermediate"], [out]))
    return PrimFunc(name or ("fused_fused_decode4_fused_NT_matmul3_add2_gelu" if gelu else "fused_fused_decode2_fused_NT_matmul_add"),
                    params, blocks, op="gemv_q8", attrs={"tir.noalias": True, "epilogue": 3 if gelu else 0})


def fused_decode_NT_matmul_add_dyn(N: int = 7680, K: int = 2560, gelu: bool = False, name: Optional[str] = None) -> PrimFunc:
    """out(1,n,N) = A(1,n,K) . decode(Wq, scale)^T + bias (then GELU), n dynamic: fused_fused_decode2_fused_NT_matmul6_add4
    (dolly-v2-3b-q8f16_1/before_dl.py:371-399) or, with ``gelu``, fused_fused_decode4_fused_NT_matmul9_add6_gelu1
    (:504-581).  Parameters: Wq, scale, A, bias, out."""
    out = "T_multiply_intermediate_intermediate" if gelu else "T_add_intermediate_intermediate"
    params = [Buffer("lv780", (N, K // 4), "uint32"), Buffer("lv781", (N, K // 32), "float16"), Buffer("lv779", (1, "n", K), "float16"),
              Buffer("param_810", (N,), "float16"), Buffer(out, (1, "n", N), "float16")]
    blocks = [Block("decode", "SS", ["lv780", "lv781"], ["decode_intermediate_intermediate"]),
              Block("NT_matmul", "SSSR", ["lv779", "decode_intermediate_intermediate"], ["NT_matmul_intermediate"]),
              Block("T_add", "SSS", ["NT_matmul_intermediate", "param_810"], [out if not gelu else "T_add_intermediate"])]
    if gelu:
        blocks.append(Block("T_multiply_2", "SSS", ["T_add_intermediate"], [out]))
    return PrimFunc(name or ("fused_fused_decode4_fused_NT_matmul9_add6_gelu1" if gelu else "fused_fused_decode2_fused_NT_matmul6_add4"),
                    params, blocks, op="gemm_q8", attrs={"tir.noalias": True, "epilogue": 3 if gelu else 0})


def module(*funcs: PrimFunc, upper_bound: Optional[dict] = None) -> IRModule:
    """An IRModule of the given PrimFuncs; ``upper_bound`` is the ``tir_var_upper_bound`` attribute
    (tuning_test/tune_cast.py:26 uses {"m": 512, "n": 4096})."""
    attrs = {"tir_var_upper_bound": dict(upper_bound)} if upper_bound else {}
    for f in funcs:
        if upper_bound:
            f.attrs.setdefault("tir_var_upper_bound", dict(upper_bound))
    return IRModule(list(funcs), attrs)

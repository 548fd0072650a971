// libdtas_packed.so: the TVM PackedFunc C signature of the reference's generated host functions
// (experiment/dtas_tuned/elementwise/add/float16/top1_256/host.cc:38-145) over the dtas_* entry points.
// Each function unpacks DLTensor handles in PrimFunc parameter order, checks what the generated code takes for
// granted (argument count and kinds, element types, compact strides, matching shapes), makes the tensors' device
// current as host.cc:70-83 does through __tvm_set_device, and calls the entry point for the element types.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../../include/dtas_abi.h"
#include "../../include/dtas_packed.h"

extern "C" void* __tvm_module_ctx = nullptr;

namespace {

thread_local char t_error[512];
thread_local bool t_own_error = false;
thread_local void* t_stream = nullptr;

int bad(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(t_error, sizeof(t_error), fmt, ap);
  va_end(ap);
  t_own_error = true;
  return -1;
}

enum Kind { kF16, kF32, kI8, kU32, kOther };
Kind kind_of(const DLDataType& t) {
  if (t.lanes != 1) return kOther;
  if (t.code == 2 && t.bits == 16) return kF16;
  if (t.code == 2 && t.bits == 32) return kF32;
  if (t.code == 0 && t.bits == 8) return kI8;
  if (t.code == 1 && t.bits == 32) return kU32;
  return kOther;
}
const char* kind_name(Kind k) {
  return k == kF16 ? "float16" : k == kF32 ? "float32" : k == kI8 ? "int8" : k == kU32 ? "uint32" : "an unsupported type";
}

struct Arg {
  const DLTensor* t;
  char* data;
  int64_t count;  // elements
};

// DLTensor handles 0 .. want-1 of `args`, each checked on its own.
int unpack(const char* fn, void* args, const int32_t* codes, int32_t num_args, int want, Arg* out) {
  t_own_error = false;
  if (num_args != want) return bad("%s: takes %d buffers, got %d arguments", fn, want, num_args);
  if (!args || !codes) return bad("%s: NULL argument array", fn);
  const TVMValue* v = static_cast<const TVMValue*>(args);
  for (int i = 0; i < want; ++i) {
    if (codes[i] == DTAS_TCODE_NULLPTR || !v[i].v_handle) return bad("%s: argument %d is a null handle", fn, i);
    if (codes[i] != DTAS_TCODE_DLTENSOR_HANDLE && codes[i] != DTAS_TCODE_NDARRAY_HANDLE && codes[i] != DTAS_TCODE_OPAQUE_HANDLE)
      return bad("%s: argument %d has type code %d, not a tensor handle", fn, i, codes[i]);
    const DLTensor* t = static_cast<const DLTensor*>(v[i].v_handle);
    if (t->ndim < 1 || t->ndim > 8 || !t->shape) return bad("%s: argument %d has %d dimensions", fn, i, t->ndim);
    int64_t count = 1;
    for (int d = 0; d < t->ndim; ++d) {
      if (t->shape[d] < 0) return bad("%s: argument %d has a negative extent", fn, i);
      count *= t->shape[d];
    }
    if (t->strides) {  // NULL or compact (host.cc:64-69 reads them and goes on: the kernels index compactly)
      int64_t expect = 1;
      for (int d = t->ndim - 1; d >= 0; --d) {
        if (t->shape[d] != 1 && t->strides[d] != expect) return bad("%s: argument %d is not compact (stride %lld of axis %d)", fn, i, (long long)t->strides[d], d);
        expect *= t->shape[d];
      }
    }
    if (t->device.device_type != 2 && t->device.device_type != 10)
      return bad("%s: argument %d lives on device type %d, not on a GPU", fn, i, t->device.device_type);
    if (t->device.device_id != static_cast<const DLTensor*>(v[0].v_handle)->device.device_id)
      return bad("%s: argument %d is on device %d, argument 0 on device %d", fn, i, t->device.device_id,
                 static_cast<const DLTensor*>(v[0].v_handle)->device.device_id);
    out[i].t = t;
    out[i].data = t->data ? static_cast<char*>(t->data) + t->byte_offset : nullptr;
    out[i].count = count;
  }
  return 0;
}

bool same_shape(const DLTensor* a, const DLTensor* b) {
  if (a->ndim != b->ndim) return false;
  for (int d = 0; d < a->ndim; ++d)
    if (a->shape[d] != b->shape[d]) return false;
  return true;
}

// rows = all leading axes, cols = the last one
void rows_cols(const DLTensor* t, int64_t* rows, int64_t* cols) {
  *cols = t->shape[t->ndim - 1];
  *rows = 1;
  for (int d = 0; d + 1 < t->ndim; ++d) *rows *= t->shape[d];
}

// host.cc:70-83: the device of the first buffer becomes current (nothing to do for an empty call)
int enter_device(const char* fn, const Arg& first) {
  if (first.count == 0) return 0;
  const hipError_t e = hipSetDevice(first.t->device.device_id);
  if (e != hipSuccess) return bad("%s: hipSetDevice(%d): %s", fn, first.t->device.device_id, hipGetErrorString(e));
  return 0;
}

}  // namespace

extern "C" void dtas_packed_set_stream(void* stream) { t_stream = stream; }
extern "C" const char* dtas_packed_last_error(void) { return t_own_error ? t_error : dtas_last_error(); }

extern "C" int32_t add(void* args, int32_t* codes, int32_t num_args, void*, int32_t*, void*) {
  Arg a[3];
  if (unpack("add", args, codes, num_args, 3, a) != 0) return -1;
  const Kind k = kind_of(a[0].t->dtype);
  if (k == kOther || kind_of(a[1].t->dtype) != k || kind_of(a[2].t->dtype) != k)
    return bad("add: the three buffers must share one of float16, float32, int8 (A is %s)", kind_name(k));
  if (!same_shape(a[0].t, a[1].t) || !same_shape(a[0].t, a[2].t)) return bad("add: the three buffers must have one shape");
  if (a[0].t->ndim < 2) return bad("add: buffers are (1, n, H)");
  if (enter_device("add", a[0]) != 0) return -1;
  // n = shape[1] (host.cc:54-55); H = what follows
  int64_t n = a[0].t->shape[1], H = 1;
  for (int d = 2; d < a[0].t->ndim; ++d) H *= a[0].t->shape[d];
  n *= a[0].t->shape[0];
  auto fn = k == kF16 ? dtas_add_f16 : k == kF32 ? dtas_add_f32 : dtas_add_i8;
  return fn(a[0].data, a[1].data, a[2].data, n, H, nullptr, t_stream);
}

extern "C" int32_t copy(void* args, int32_t* codes, int32_t num_args, void*, int32_t*, void*) {
  Arg a[2];
  if (unpack("copy", args, codes, num_args, 2, a) != 0) return -1;
  const Kind k = kind_of(a[0].t->dtype);
  if (k == kOther || kind_of(a[1].t->dtype) != k) return bad("copy: both buffers must share one of float16, float32, int8 (A is %s)", kind_name(k));
  if (!same_shape(a[0].t, a[1].t)) return bad("copy: both buffers must have one shape");
  if (a[0].t->ndim < 2) return bad("copy: buffers are (1, n, H)");
  if (enter_device("copy", a[0]) != 0) return -1;
  int64_t n = a[0].t->shape[0] * a[0].t->shape[1], H = 1;
  for (int d = 2; d < a[0].t->ndim; ++d) H *= a[0].t->shape[d];
  auto fn = k == kF16 ? dtas_copy_f16 : k == kF32 ? dtas_copy_f32 : dtas_copy_i8;
  return fn(a[0].data, a[1].data, n, H, nullptr, t_stream);
}

extern "C" int32_t cast(void* args, int32_t* codes, int32_t num_args, void*, int32_t*, void*) {
  Arg a[2];
  if (unpack("cast", args, codes, num_args, 2, a) != 0) return -1;
  const Kind from = kind_of(a[0].t->dtype), to = kind_of(a[1].t->dtype);
  if (!((from == kF16 && to == kF32) || (from == kF32 && to == kF16)))
    return bad("cast: float16 -> float32 or float32 -> float16, got %s -> %s", kind_name(from), kind_name(to));
  if (!same_shape(a[0].t, a[1].t)) return bad("cast: both buffers must have one shape");
  if (a[0].t->ndim < 2) return bad("cast: buffers are (1, n, H)");
  if (enter_device("cast", a[0]) != 0) return -1;
  int64_t n = a[0].t->shape[0] * a[0].t->shape[1], H = 1;
  for (int d = 2; d < a[0].t->ndim; ++d) H *= a[0].t->shape[d];
  return (from == kF16 ? dtas_cast_f16_f32 : dtas_cast_f32_f16)(a[0].data, a[1].data, n, H, nullptr, t_stream);
}

extern "C" int32_t fused_layer_norm_cast1(void* args, int32_t* codes, int32_t num_args, void*, int32_t*, void*) {
  Arg a[4];
  if (unpack("fused_layer_norm_cast1", args, codes, num_args, 4, a) != 0) return -1;
  if (kind_of(a[0].t->dtype) != kF32 || kind_of(a[1].t->dtype) != kF32 || kind_of(a[2].t->dtype) != kF32 || kind_of(a[3].t->dtype) != kF16)
    return bad("fused_layer_norm_cast1: (float32 x, float32 gamma, float32 beta) -> float16");
  int64_t n, H;
  rows_cols(a[0].t, &n, &H);
  if (!same_shape(a[0].t, a[3].t) || a[1].count != H || a[2].count != H)
    return bad("fused_layer_norm_cast1: x and the output are (1, n, H), gamma and beta (H)");
  if (enter_device("fused_layer_norm_cast1", a[0]) != 0) return -1;
  return dtas_layer_norm_f32_f16(a[0].data, a[1].data, a[2].data, a[3].data, n, H, 1e-5f, nullptr, t_stream);
}

extern "C" int32_t fused_softmax_cast(void* args, int32_t* codes, int32_t num_args, void*, int32_t*, void*) {
  Arg a[2];
  if (unpack("fused_softmax_cast", args, codes, num_args, 2, a) != 0) return -1;
  const Kind from = kind_of(a[0].t->dtype);
  if ((from != kF32 && from != kF16) || kind_of(a[1].t->dtype) != kF16) return bad("fused_softmax_cast: float32 or float16 -> float16");
  if (!same_shape(a[0].t, a[1].t)) return bad("fused_softmax_cast: both buffers must have one shape");
  int64_t rows, cols;
  rows_cols(a[0].t, &rows, &cols);
  if (enter_device("fused_softmax_cast", a[0]) != 0) return -1;
  return (from == kF32 ? dtas_softmax_f32_f16 : dtas_softmax_f16)(a[0].data, a[1].data, rows, cols, nullptr, t_stream);
}

static int32_t matmul_add(const char* fn, void* args, int32_t* codes, int32_t num_args, bool one_row) {
  Arg a[4];
  if (unpack(fn, args, codes, num_args, 4, a) != 0) return -1;
  for (int i = 0; i < 4; ++i)
    if (kind_of(a[i].t->dtype) != kF16) return bad("%s: every buffer is float16 (argument %d is %s)", fn, i, kind_name(kind_of(a[i].t->dtype)));
  if (a[1].t->ndim != 2) return bad("%s: W is (N, K)", fn);
  const int64_t N = a[1].t->shape[0], K = a[1].t->shape[1];
  int64_t M, k_in, m_out, n_out;
  rows_cols(a[0].t, &M, &k_in);
  rows_cols(a[3].t, &m_out, &n_out);
  if (k_in != K || n_out != N || m_out != M || a[2].count != N)
    return bad("%s: lv is (1, n, K), W (N, K), bias (N), the output (1, n, N)", fn);
  if (one_row && M != 1) return bad("%s: takes one row, got %lld", fn, (long long)M);
  if (enter_device(fn, a[0]) != 0) return -1;
  if (M == 1) return dtas_gemv_f16(a[0].data, a[1].data, a[2].data, a[3].data, N, K, nullptr, t_stream);
  return dtas_gemm_f16(a[0].data, a[1].data, a[2].data, a[3].data, M, N, K, nullptr, t_stream);
}

extern "C" int32_t fused_NT_matmul4_add1(void* args, int32_t* codes, int32_t num_args, void*, int32_t*, void*) {
  return matmul_add("fused_NT_matmul4_add1", args, codes, num_args, false);
}
extern "C" int32_t fused_NT_matmul10_add5(void* args, int32_t* codes, int32_t num_args, void*, int32_t*, void*) {
  return matmul_add("fused_NT_matmul10_add5", args, codes, num_args, true);
}

// ---- the fused-epilogue GEMMs (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:163-318, :408-549): parameter order
// (lv (1, n, K), W (N, K), bias (N), [res1 (1, n, N), res2 (1, n, N),] out (1, n, N)); n is read from the shapes, so
// the prefill form (dynamic n) and the decode form (n = 1) of a name are one function
static int32_t matmul_fused(const char* fn, void* args, int32_t* codes, int32_t num_args, int32_t epilogue) {
  const bool add2 = epilogue == DTAS_EPI_BIAS_ADD2 || epilogue == DTAS_EPI_BIAS_ADD2_CAST_F32;
  const int want = add2 ? 6 : 4, out_i = want - 1;
  Arg a[6];
  if (unpack(fn, args, codes, num_args, want, a) != 0) return -1;
  for (int i = 0; i < out_i; ++i)
    if (kind_of(a[i].t->dtype) != kF16) return bad("%s: every input is float16 (argument %d is %s)", fn, i, kind_name(kind_of(a[i].t->dtype)));
  const Kind out_kind = epilogue == DTAS_EPI_BIAS_ADD2_CAST_F32 ? kF32 : kF16;
  if (kind_of(a[out_i].t->dtype) != out_kind) return bad("%s: the output is %s, got %s", fn, kind_name(out_kind), kind_name(kind_of(a[out_i].t->dtype)));
  if (a[1].t->ndim != 2) return bad("%s: W is (N, K)", fn);
  const int64_t N = a[1].t->shape[0], K = a[1].t->shape[1];
  int64_t M, k_in, m_out, n_out;
  rows_cols(a[0].t, &M, &k_in);
  rows_cols(a[out_i].t, &m_out, &n_out);
  if (k_in != K || n_out != N || m_out != M || a[2].count != N) return bad("%s: lv is (1, n, K), W (N, K), bias (N), the output (1, n, N)", fn);
  if (add2 && (!same_shape(a[3].t, a[4].t) || a[3].count != M * N || a[3].t->shape[a[3].t->ndim - 1] != N))
    return bad("%s: both residuals are (1, n, N)", fn);
  if (enter_device(fn, a[0]) != 0) return -1;
  return dtas_gemm_f16_fused(a[0].data, a[1].data, a[2].data, add2 ? a[3].data : nullptr, add2 ? a[4].data : nullptr, a[out_i].data, M, N, K,
                             epilogue, nullptr, t_stream);
}

// ---- attention scores (before_dl.py:116-160, :363-406): (q (1, H, n, d), k (1, H, m, d), mask (1, 1, n, m), out (1, H, n, m)
// float32); the PrimFunc multiplies by the fp16 constant 1 / sqrt(d) (0.1118 for the model's d = 80)
static int32_t scores(const char* fn, void* args, int32_t* codes, int32_t num_args) {
  Arg a[4];
  if (unpack(fn, args, codes, num_args, 4, a) != 0) return -1;
  for (int i = 0; i < 3; ++i)
    if (kind_of(a[i].t->dtype) != kF16) return bad("%s: q, k and the mask are float16 (argument %d is %s)", fn, i, kind_name(kind_of(a[i].t->dtype)));
  if (kind_of(a[3].t->dtype) != kF32) return bad("%s: the output is float32, got %s", fn, kind_name(kind_of(a[3].t->dtype)));
  for (int i = 0; i < 4; ++i)
    if (a[i].t->ndim != 4 || a[i].t->shape[0] != 1) return bad("%s: every buffer is (1, heads, rows, columns) (argument %d)", fn, i);
  const int64_t H = a[0].t->shape[1], n = a[0].t->shape[2], d = a[0].t->shape[3], m = a[1].t->shape[2];
  const int64_t* ms = a[2].t->shape;
  const int64_t* os = a[3].t->shape;
  if (a[1].t->shape[1] != H || a[1].t->shape[3] != d || ms[1] != 1 || ms[2] != n || ms[3] != m || os[1] != H || os[2] != n || os[3] != m)
    return bad("%s: q is (1, H, n, d), k (1, H, m, d), the mask (1, 1, n, m), the output (1, H, n, m)", fn);
  if (d <= 0) return bad("%s: the head dimension is %lld", fn, (long long)d);
  if (enter_device(fn, a[3]) != 0) return -1;
  return dtas_attn_scores_f16_f32(a[0].data, a[1].data, a[2].data, a[3].data, H, n, m, d, static_cast<float>(1.0 / sqrt(static_cast<double>(d))),
                                  nullptr, t_stream);
}

// ---- P.V (before_dl.py:899-929): (A (1, H, n, m), B (1, H, m, d), out (1, H, n, d)), all float16
static int32_t pv(const char* fn, void* args, int32_t* codes, int32_t num_args) {
  Arg a[3];
  if (unpack(fn, args, codes, num_args, 3, a) != 0) return -1;
  for (int i = 0; i < 3; ++i) {
    if (kind_of(a[i].t->dtype) != kF16) return bad("%s: every buffer is float16 (argument %d is %s)", fn, i, kind_name(kind_of(a[i].t->dtype)));
    if (a[i].t->ndim != 4 || a[i].t->shape[0] != 1) return bad("%s: every buffer is (1, heads, rows, columns) (argument %d)", fn, i);
  }
  const int64_t H = a[0].t->shape[1], n = a[0].t->shape[2], m = a[0].t->shape[3], d = a[1].t->shape[3];
  const int64_t* os = a[2].t->shape;
  if (a[1].t->shape[1] != H || a[1].t->shape[2] != m || os[1] != H || os[2] != n || os[3] != d)
    return bad("%s: A is (1, H, n, m), B (1, H, m, d), the output (1, H, n, d)", fn);
  if (enter_device(fn, a[2]) != 0) return -1;
  return dtas_attn_pv_f16(a[0].data, a[1].data, a[2].data, H, n, m, d, nullptr, t_stream);
}

// ---- GEMMs on 8-bit weights (experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py:371-638): (Wq (N, K/4) uint32, scale
// (N, K/32) float16, lv (1, n, K), bias (N), out (1, n, N)); n from the shapes (one row lands on the dequantising GEMV)
static int32_t matmul_q8(const char* fn, void* args, int32_t* codes, int32_t num_args, int32_t epilogue) {
  Arg a[5];
  if (unpack(fn, args, codes, num_args, 5, a) != 0) return -1;
  if (kind_of(a[0].t->dtype) != kU32) return bad("%s: the packed weights are uint32, got %s", fn, kind_name(kind_of(a[0].t->dtype)));
  for (int i = 1; i < 5; ++i)
    if (kind_of(a[i].t->dtype) != kF16) return bad("%s: scales, lv, bias and the output are float16 (argument %d is %s)", fn, i, kind_name(kind_of(a[i].t->dtype)));
  if (a[0].t->ndim != 2 || a[1].t->ndim != 2) return bad("%s: the packed weights are (N, K/4), the scales (N, K/32)", fn);
  const int64_t N = a[0].t->shape[0], K = a[0].t->shape[1] * 4;
  int64_t M, k_in, m_out, n_out;
  rows_cols(a[2].t, &M, &k_in);
  rows_cols(a[4].t, &m_out, &n_out);
  if (a[1].t->shape[0] != N || a[1].t->shape[1] * 32 != K || k_in != K || a[3].count != N || n_out != N || m_out != M)
    return bad("%s: the packed weights are (N, K/4), the scales (N, K/32), lv (1, n, K), bias (N), the output (1, n, N)", fn);
  if (enter_device(fn, a[2]) != 0) return -1;
  return dtas_gemm_q8_f16_fused(a[2].data, a[0].data, a[1].data, a[3].data, nullptr, nullptr, a[4].data, M, N, K, epilogue, nullptr, t_stream);
}

#define DTAS_PACKED(NAME, CALL) \
  extern "C" int32_t NAME(void* args, int32_t* codes, int32_t num_args, void*, int32_t*, void*) { return CALL; }
// dolly-v2-3b-q0f16/before_dl.py (prefill: dynamic n; decode: n = 1) and the names the 8-bit model gives the same forms
DTAS_PACKED(fused_NT_matmul_add, matmul_add("fused_NT_matmul_add", args, codes, num_args, false))
DTAS_PACKED(fused_NT_matmul6_add4, matmul_add("fused_NT_matmul6_add4", args, codes, num_args, true))
DTAS_PACKED(fused_NT_matmul2_add1_add3_add3, matmul_fused("fused_NT_matmul2_add1_add3_add3", args, codes, num_args, DTAS_EPI_BIAS_ADD2))
DTAS_PACKED(fused_NT_matmul2_add1_add3_add3_cast, matmul_fused("fused_NT_matmul2_add1_add3_add3_cast", args, codes, num_args, DTAS_EPI_BIAS_ADD2_CAST_F32))
DTAS_PACKED(fused_NT_matmul3_add2_gelu, matmul_fused("fused_NT_matmul3_add2_gelu", args, codes, num_args, DTAS_EPI_BIAS_GELU))
DTAS_PACKED(fused_NT_matmul8_add5_add7_add7, matmul_fused("fused_NT_matmul8_add5_add7_add7", args, codes, num_args, DTAS_EPI_BIAS_ADD2))
DTAS_PACKED(fused_NT_matmul8_add5_add7_add7_cast5, matmul_fused("fused_NT_matmul8_add5_add7_add7_cast5", args, codes, num_args, DTAS_EPI_BIAS_ADD2_CAST_F32))
DTAS_PACKED(fused_NT_matmul9_add6_gelu1, matmul_fused("fused_NT_matmul9_add6_gelu1", args, codes, num_args, DTAS_EPI_BIAS_GELU))
DTAS_PACKED(fused_NT_matmul1_divide_maximum_minimum_cast2, scores("fused_NT_matmul1_divide_maximum_minimum_cast2", args, codes, num_args))
DTAS_PACKED(fused_NT_matmul7_divide1_maximum1_minimum1_cast7, scores("fused_NT_matmul7_divide1_maximum1_minimum1_cast7", args, codes, num_args))
DTAS_PACKED(fused_NT_matmul1_divide1_maximum_minimum_cast2, scores("fused_NT_matmul1_divide1_maximum_minimum_cast2", args, codes, num_args))
DTAS_PACKED(fused_NT_matmul7_divide2_maximum1_minimum1_cast7, scores("fused_NT_matmul7_divide2_maximum1_minimum1_cast7", args, codes, num_args))
DTAS_PACKED(matmul8, pv("matmul8", args, codes, num_args))
DTAS_PACKED(matmul10, pv("matmul10", args, codes, num_args))
DTAS_PACKED(matmul9, pv("matmul9", args, codes, num_args))
DTAS_PACKED(matmul1, pv("matmul1", args, codes, num_args))
// dolly-v2-3b-q8f16_1/before_dl.py
DTAS_PACKED(fused_fused_decode2_fused_NT_matmul_add, matmul_q8("fused_fused_decode2_fused_NT_matmul_add", args, codes, num_args, DTAS_EPI_BIAS))
DTAS_PACKED(fused_fused_decode2_fused_NT_matmul6_add4, matmul_q8("fused_fused_decode2_fused_NT_matmul6_add4", args, codes, num_args, DTAS_EPI_BIAS))
DTAS_PACKED(fused_fused_decode4_fused_NT_matmul3_add2_gelu, matmul_q8("fused_fused_decode4_fused_NT_matmul3_add2_gelu", args, codes, num_args, DTAS_EPI_BIAS_GELU))
DTAS_PACKED(fused_fused_decode4_fused_NT_matmul9_add6_gelu1, matmul_q8("fused_fused_decode4_fused_NT_matmul9_add6_gelu1", args, codes, num_args, DTAS_EPI_BIAS_GELU))
DTAS_PACKED(fused_fused_decode5_fused_NT_matmul4_add1, matmul_q8("fused_fused_decode5_fused_NT_matmul4_add1", args, codes, num_args, DTAS_EPI_BIAS))
DTAS_PACKED(fused_fused_decode5_fused_NT_matmul10_add5, matmul_q8("fused_fused_decode5_fused_NT_matmul10_add5", args, codes, num_args, DTAS_EPI_BIAS))
#undef DTAS_PACKED

/* dtas_packed.h -- the reference's own host interface over libdtas_gfx950.so
 *
 * What TVM's runtime binds from a DTAS-built host.so is one function per PrimFunc with the
 * PackedFunc C signature
 *     int32_t <name>(void* args, int32_t* arg_type_ids, int32_t num_args,
 *                    void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle)
 * (experiment/dtas_tuned/elementwise/add/float16/top1_256/host.cc:38-42): `args` is a TVMValue
 * array whose v_handle members point to DLTensors in PrimFunc parameter order, the dynamic extent
 * is read from the first buffer's shape (host.cc:54-55: n = shape[1]), strides are NULL or compact
 * (:64-69), the device comes from the first tensor (:56, :70-83), the result is 0 or -1
 * (:75-83, :133-143).  libdtas_packed.so exports those functions under the PrimFuncs' names; each
 * unpacks its DLTensors, checks them, makes the tensors' device current and calls the dtas_*
 * entry point of include/dtas_abi.h that matches the element types.
 *
 * The structs below are DLPack's and TVM's, field for field (dlpack.h, c_runtime_api.h); a caller
 * that includes TVM's headers first gets theirs instead.
 */
#ifndef DTAS_PACKED_H_
#define DTAS_PACKED_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef DLPACK_DLPACK_H_
typedef struct {
  int32_t device_type; /* 2 = kDLCUDA (what the reference's host code passes), 10 = kDLROCM */
  int32_t device_id;
} DLDevice;
typedef struct {
  uint8_t code; /* 0 = int, 1 = uint, 2 = float */
  uint8_t bits;
  uint16_t lanes;
} DLDataType;
typedef struct {
  void* data;
  DLDevice device;
  int32_t ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides; /* NULL = compact row-major */
  uint64_t byte_offset;
} DLTensor;
#endif

#ifndef TVM_RUNTIME_C_RUNTIME_API_H_
typedef union {
  int64_t v_int64;
  double v_float64;
  void* v_handle;
  const char* v_str;
  DLDataType v_type;
  DLDevice v_device;
} TVMValue;
#endif

/* argument type codes a buffer may arrive with (c_runtime_api.h: TVMArgTypeCode) */
#define DTAS_TCODE_OPAQUE_HANDLE 3
#define DTAS_TCODE_NULLPTR 4
#define DTAS_TCODE_DLTENSOR_HANDLE 7
#define DTAS_TCODE_NDARRAY_HANDLE 13

/* The module context slot TVM's loader fills (host.cc:17); unused here, exported because loaders look it up. */
extern void* __tvm_module_ctx;

/* add / copy / cast (tuning_test/tune_ele_add.py:10-22, tune_ele_copy.py:10-21, tune_cast.py:10-21):
 * buffers (1, n, H); add and copy in float16, float32 or int8, cast float16 -> float32 or float32 -> float16,
 * by the tensors' dtype.  add(A, B, T_add), copy(A, T_copy), cast(A, compute). */
int32_t add(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t copy(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t cast(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
/* fused_layer_norm_cast1(lv6 (1, n, H) float32, gamma (H) float32, beta (H) float32, out (1, n, H) float16)
 * (experiment/dtas_tuned/general_reduction/layernorm/top1_256/host.cc; eps = 1e-5 as in the PrimFunc) */
int32_t fused_layer_norm_cast1(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
/* fused_softmax_cast(A (..., m) float32 or float16, out (..., m) float16): softmax over the last axis, every
 * leading axis a row (the reference's (1, 32, n, m) and (1, 12800, n) forms:
 * experiment/dtas_tuned/general_reduction/softmax/row_12800/top10_256_10_nounroll/host.cc) */
int32_t fused_softmax_cast(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
/* fused_NT_matmul4_add1(lv (1, n, K), W (N, K), bias (N), out (1, n, N)), all float16
 * (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:320-341); fused_NT_matmul10_add5: the same with n = 1 (:96-113) */
int32_t fused_NT_matmul4_add1(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul10_add5(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
/* the same PrimFunc under the names the model graphs use for the 7680 x 2560 projection: dynamic n (:552-572) and n = 1 (:343-360) */
int32_t fused_NT_matmul_add(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul6_add4(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);

/* ---- the fused-epilogue GEMMs of the model graph (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py); every step an fp16
 * tensor, as dtas_gemm_f16_fused spells them.  n is read from the shapes: the prefill form (dynamic n) and the decode form
 * (n = 1; the 8-bit model's graph swaps the two names) of a PrimFunc are one function.
 * fused_NT_matmul2_add1_add3_add3(lv (1, n, K), W (N, K), bias (N), res1 (1, n, N), res2 (1, n, N), out (1, n, N)) (:163-200),
 * .._cast: the same with a float32 output (:202-246); decode names fused_NT_matmul8_add5_add7_add7 (:408-439), .._cast5 (:442-480).
 * fused_NT_matmul3_add2_gelu(lv (1, n, K), W (N, K), bias (N), out (1, n, N)) (:248-318); decode name fused_NT_matmul9_add6_gelu1 (:483-549). */
int32_t fused_NT_matmul2_add1_add3_add3(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul2_add1_add3_add3_cast(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul3_add2_gelu(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul8_add5_add7_add7(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul8_add5_add7_add7_cast5(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul9_add6_gelu1(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);

/* ---- the two batched attention matmuls.
 * fused_NT_matmul1_divide_maximum_minimum_cast2(q (1, H, n, d), k (1, H, m, d), mask (1, 1, n, m), out (1, H, n, m) float32)
 * (:116-160; n and m dynamic; the product is multiplied by the fp16 constant 1 / sqrt(d), 0.1118 for d = 80, clamped at -65504 and
 * cut by the mask); decode name fused_NT_matmul7_divide1_maximum1_minimum1_cast7 (:363-406); in the 8-bit model's file
 * (dolly-v2-3b-q8f16_1/before_dl.py:83-126, :203-248) the same two are fused_NT_matmul1_divide1_maximum_minimum_cast2 and
 * fused_NT_matmul7_divide2_maximum1_minimum1_cast7.
 * matmul8(A (1, H, n, m), B (1, H, m, d), out (1, H, n, d)) (:915-929) and matmul10, its n = 1 form (:899-912); matmul9 / matmul1 in
 * the 8-bit model's file (:1000-1015, :984-998). */
int32_t fused_NT_matmul1_divide_maximum_minimum_cast2(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul7_divide1_maximum1_minimum1_cast7(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul1_divide1_maximum_minimum_cast2(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_NT_matmul7_divide2_maximum1_minimum1_cast7(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t matmul8(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t matmul10(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t matmul9(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t matmul1(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);

/* ---- GEMMs on 8-bit weights (experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py): W = (fp16(byte) - 127) * scale, four bytes to
 * a uint32 word, an fp16 scale per 32 elements of a row; parameter order (Wq (N, K/4) uint32, scale (N, K/32), lv (1, n, K), bias (N),
 * out (1, n, N)).  fused_fused_decode2_fused_NT_matmul_add (:401-426, n = 1) / .._matmul6_add4 (:371-399, dynamic n);
 * fused_fused_decode4_fused_NT_matmul3_add2_gelu (:428-502, n = 1) / .._matmul9_add6_gelu1 (:504-581, dynamic n);
 * fused_fused_decode5_fused_NT_matmul4_add1 (:613-638, n = 1) / .._matmul10_add5 (:583-611, dynamic n). */
int32_t fused_fused_decode2_fused_NT_matmul_add(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_fused_decode2_fused_NT_matmul6_add4(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_fused_decode4_fused_NT_matmul3_add2_gelu(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_fused_decode4_fused_NT_matmul9_add6_gelu1(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_fused_decode5_fused_NT_matmul4_add1(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);
int32_t fused_fused_decode5_fused_NT_matmul10_add5(void* args, int32_t* arg_type_ids, int32_t num_args, void* out_ret_value, int32_t* out_ret_tcode, void* resource_handle);

/* TVM enqueues on the calling thread's current stream; this sets that stream (a hipStream_t, NULL = the default
 * stream) for the calls the calling host thread makes through the functions above. */
void dtas_packed_set_stream(void* stream);
/* Message of the last failed call of this thread (the argument check's, or dtas_last_error()'s). */
const char* dtas_packed_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* DTAS_PACKED_H_ */

// Device-side helpers for gfx950: 128-bit vector types, wave64 DPP reductions,
// workgroup reductions through LDS.  Internal to libdtas_gfx950.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dtas {

typedef _Float16 half_t;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// ---- wave64 cross-lane reduction on the DPP datapath -------------------------------
// quad_perm xor-1, quad_perm xor-2, row_half_mirror, row_mirror leave every lane of a
// 16-lane row holding the row's result; row_bcast:15 / row_bcast:31 fold the four rows
// into lane 63, which v_readlane broadcasts as a scalar.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_mov(float old, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old),
                                                                __builtin_bit_cast(int, v), CTRL,
                                                                ROW_MASK, 0xf, false));
}

__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_mov<0xB1, 0xf>(0.f, v);
  v += dpp_mov<0x4E, 0xf>(0.f, v);
  v += dpp_mov<0x141, 0xf>(0.f, v);
  v += dpp_mov<0x140, 0xf>(0.f, v);
  v += dpp_mov<0x142, 0xa>(0.f, v);
  v += dpp_mov<0x143, 0xc>(0.f, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_mov<0xB1, 0xf>(v, v));
  v = fmaxf(v, dpp_mov<0x4E, 0xf>(v, v));
  v = fmaxf(v, dpp_mov<0x141, 0xf>(v, v));
  v = fmaxf(v, dpp_mov<0x140, 0xf>(v, v));
  v = fmaxf(v, dpp_mov<0x142, 0xa>(v, v));
  v = fmaxf(v, dpp_mov<0x143, 0xc>(v, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// ---- workgroup reduction: DPP inside each wavefront, one LDS slot per wavefront ------
// `slots` needs blockDim.x / 64 floats; every thread of the workgroup must call.
struct SumOp {
  static __device__ __forceinline__ float wave(float v) { return wave_sum(v); }
  static __device__ __forceinline__ float join(float a, float b) { return a + b; }
};
struct MaxOp {
  static __device__ __forceinline__ float wave(float v) { return wave_max(v); }
  static __device__ __forceinline__ float join(float a, float b) { return fmaxf(a, b); }
};

// Workgroup reductions through 2 x 16 LDS slots.  Consecutive reductions alternate between the
// two banks (`phase` counts them), so a bank is rewritten only after a barrier that every reader
// of its previous contents has passed: one barrier per reduction.  The partial results are
// joined in wavefront order by every thread, so all threads hold the same bits.
template <typename Op>
__device__ __forceinline__ float block_reduce(float v, float* slots, int& phase) {
  const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const float w = Op::wave(v);
  if (nwaves == 1) return w;
  float* bank = slots + ((phase++ & 1) << 4);
  if ((threadIdx.x & 63) == 0) bank[wave] = w;
  __syncthreads();
  float r = bank[0];
  for (int i = 1; i < nwaves; ++i) r = Op::join(r, bank[i]);
  return r;
}

// Two sums behind one barrier; `slots` holds 2 x 32 floats.
__device__ __forceinline__ void block_sum2(float& a, float& b, float* slots, int& phase) {
  const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const float wa = SumOp::wave(a), wb = SumOp::wave(b);
  if (nwaves == 1) {
    a = wa;
    b = wb;
    return;
  }
  float* bank = slots + ((phase++ & 1) << 5);
  if ((threadIdx.x & 63) == 0) {
    bank[wave] = wa;
    bank[16 + wave] = wb;
  }
  __syncthreads();
  float ra = bank[0], rb = bank[16];
  for (int i = 1; i < nwaves; ++i) {
    ra += bank[i];
    rb += bank[16 + i];
  }
  a = ra;
  b = rb;
}

// ---- erf-GELU on an fp16 value, every step an fp16 tensor as the fused PrimFuncs spell it
// (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:248-318): t * (0.5 + 0.5 * erf(t * fp16(0.7071...)))
// erf of a value that is an fp16 number, for a result that is rounded to fp16: x * P(x^2) with P a
// degree-10 polynomial fitted for relative error on [0, 2.75], +-1 beyond (erf rounds to 1.0 in fp16 from
// 2.596 on).  Over all 63 488 finite fp16 inputs the rounded result differs from libm's erff rounded in
// 6 (by one fp16 ulp); it costs 15 instructions where erff costs ~35, which the GELU epilogue of a GEMM
// pays per output element.
__device__ __forceinline__ float erf_of_f16(float x) {
  const float t = fmaf(x * x, 0.2644628f, -1.f);
  float p = 3.507727815e-04f;
  p = fmaf(p, t, -1.175096375e-03f);
  p = fmaf(p, t, 2.496362897e-03f);
  p = fmaf(p, t, -6.172187161e-03f);
  p = fmaf(p, t, 1.496723015e-02f);
  p = fmaf(p, t, -3.152125701e-02f);
  p = fmaf(p, t, 5.924283713e-02f);
  p = fmaf(p, t, -1.007829085e-01f);
  p = fmaf(p, t, 1.577374041e-01f);
  p = fmaf(p, t, -2.427380979e-01f);
  p = fmaf(p, t, 5.111947656e-01f);
  return fabsf(x) >= 2.75f ? copysignf(1.f, x) : x * p;
}

// The same for a value that is rounded to fp16 afterwards, without the branch: at the clamped argument 2.75 the
// polynomial gives 0.9999, which is 1.0 in fp16 (checked over every non-NaN fp16 input: the rounded results are the
// same 65 536 values).  A NaN comes back as a finite number; the GELU multiplies it with its NaN argument again.
__device__ __forceinline__ float erf_of_f16_for_f16(float x) {
  const float c = __builtin_amdgcn_fmed3f(x, -2.75f, 2.75f);
  const float t = fmaf(c * c, 0.2644628f, -1.f);
  float p = 3.507727815e-04f;
  p = fmaf(p, t, -1.175096375e-03f);
  p = fmaf(p, t, 2.496362897e-03f);
  p = fmaf(p, t, -6.172187161e-03f);
  p = fmaf(p, t, 1.496723015e-02f);
  p = fmaf(p, t, -3.152125701e-02f);
  p = fmaf(p, t, 5.924283713e-02f);
  p = fmaf(p, t, -1.007829085e-01f);
  p = fmaf(p, t, 1.577374041e-01f);
  p = fmaf(p, t, -2.427380979e-01f);
  p = fmaf(p, t, 5.111947656e-01f);
  return c * p;
}

__device__ __forceinline__ half_t gelu_erf_f16_steps(half_t t) {
  const float x = static_cast<float>(t);
  const half_t m = static_cast<half_t>(x * static_cast<float>(static_cast<half_t>(0.70710678118654757f)));
  const half_t e = static_cast<half_t>(erf_of_f16(static_cast<float>(m)));
  const half_t h = static_cast<half_t>(static_cast<float>(e) * 0.5f);
  const half_t a = static_cast<half_t>(0.5f + static_cast<float>(h));
  return static_cast<half_t>(x * static_cast<float>(a));
}

// The same steps on a vector of N fp16 values (+ a bias first, when given), the fp16 steps as packed fp16 instructions:
// an fp16 product or sum rounded once is what the step computed through fp32 gives (fp32 holds the product of two
// fp16 numbers exactly, and rounding a sum first to 24 and then to 11 bits is rounding it to 11), so the results are
// the same bits; contraction is off because e * 0.5 + 0.5 as one fused operation would round once where the steps
// round twice.  8 instructions per element fewer than the scalar form in the GEMM epilogue, which is bound by them.
template <typename V, int N>
__device__ __forceinline__ V gelu_erf_f16_steps_vec(V t, bool has_bias, V bias) {
#pragma clang fp contract(off)
  if (has_bias) t = t + bias;
  const V m = t * static_cast<half_t>(0.70710678118654757f);
  V e;
#pragma unroll
  for (int i = 0; i < N; ++i) e[i] = static_cast<half_t>(erf_of_f16_for_f16(static_cast<float>(m[i])));
  const V h = e * static_cast<half_t>(0.5f);
  const V a = h + static_cast<half_t>(0.5f);
  return t * a;
}

// ---- four 8-bit weights of a word as two packed fp16 pairs {W[4w], W[4w+1]}, {W[4w+2], W[4w+3]}:
// W = (fp16(byte) - 127) * scale in fp16 arithmetic.  0x6400 | byte is the fp16 number 1024 + byte, so one byte
// permute builds two such halves, a packed subtract of 1151 leaves byte - 127 exactly, the packed multiply rounds
// as an fp16 product does.
__device__ __forceinline__ void dequant_q8_word(unsigned word, f16x2 scale2, f16x2& lo, f16x2& hi) {
  const f16x2 bias2 = {static_cast<half_t>(1151.f), static_cast<half_t>(1151.f)};
  const unsigned plo = __builtin_amdgcn_perm(0x64646464u, word, 0x04010400u);  // bytes: b0, 0x64, b1, 0x64
  const unsigned phi = __builtin_amdgcn_perm(0x64646464u, word, 0x04030402u);  // bytes: b2, 0x64, b3, 0x64
  lo = (__builtin_bit_cast(f16x2, plo) - bias2) * scale2;
  hi = (__builtin_bit_cast(f16x2, phi) - bias2) * scale2;
}

// ---- streaming (touch-once) global accesses ---------------------------------------
template <typename V>
__device__ __forceinline__ V load_stream(const V* p) { return __builtin_nontemporal_load(p); }
template <typename V>
__device__ __forceinline__ void store_stream(V v, V* p) { __builtin_nontemporal_store(v, p); }

}  // namespace dtas

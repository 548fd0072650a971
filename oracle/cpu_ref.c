/*
 * CPU oracle for the DTAS hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C restatement of the loop nests of the TIR PrimFuncs whose scheduled
 * GPU kernels the library replaces.  Only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may load this file's shared object; the
 * product path never calls into it.
 *
 * Every function follows the PrimFunc text it cites (paths are relative to the
 * reference checkout): same accumulation dtype, same operation order inside a
 * row (sequential over the reduction axis, as an unscheduled PrimFunc built
 * for an llvm CPU target executes).  Rows are independent, so the optional
 * OpenMP split over rows (nthreads > 1) does not change any result bit.
 *
 * Parity status: the reference holds no numerical tests or golden vectors, so
 * every function here is pinned by closed forms, library routines (numpy /
 * torch CPU), exhaustive enumeration and invariants in tests/ -- see each
 * function's comment.  rms_norm has no counterpart in the reference at all
 * ("parity unpinned" by the reference; pinned by its closed form only).
 *
 * Build: gcc -O3 -march=x86-64-v3 -fopenmp -shared -fPIC (see oracle/Makefile).
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
/* every function below names its thread-count parameter nthreads */
#define OMP_FOR(nt) _Pragma("omp parallel for schedule(static) num_threads(nthreads)")
#else
#define OMP_FOR(nt) (void)(nt);
#endif

typedef uint16_t f16; /* IEEE binary16 bit pattern */

/* ---- fp16 <-> fp32: hardware F16C (IEEE RNE, subnormals kept) ------------- */
static inline float h2f(f16 h) { return _cvtsh_ss(h); }
static inline f16 f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }

/* ---- fp16 <-> fp32 in integer arithmetic only: pins the F16C path in tests - */
float oracle_soft_h2f(f16 h) {
  uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu, u;
  if (e == 0) {
    if (m == 0) {
      u = s;
    } else { /* subnormal: normalise */
      int sh = 0;
      while (!(m & 0x400u)) { m <<= 1; ++sh; }
      u = s | ((uint32_t)(127 - 15 - sh + 1) << 23) | ((m & 0x3ffu) << 13);
    }
  } else if (e == 31) {
    u = s | 0x7f800000u | (m << 13);
  } else {
    u = s | ((e + 112u) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

f16 oracle_soft_f2h(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t s = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (f16)(s | 0x7e00u | ((a >> 13) & 0x3ffu)); /* NaN, quieted */
  if (a >= 0x477ff000u) return (f16)(s | 0x7c00u); /* |x| >= 65520 -> inf (also inf) */
  if (a < 0x33000001u) return (f16)s;              /* |x| <= 2^-25 -> +-0 (tie to even) */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift = (e < -14) ? (13 + (-14 - e)) : 13; /* bits dropped */
  uint32_t keep = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (keep & 1u))) ++keep;
  if (e < -14) return (f16)(s | keep); /* subnormal (carry into exponent is the right bits) */
  /* keep has the hidden bit at position 10; a rounding carry bumps the exponent */
  return (f16)(s | (((uint32_t)(e + 15) << 10) + (keep - 0x400u)));
}

/* ===========================================================================
 * Elementwise: tuning_test/tune_ele_add.py:10-22 (add), tune_cast.py:10-21
 * (cast fp16->fp32), tune_ele_copy.py:10-21 (copy); fp16/fp32/int8 variants as
 * in experiment/dtas_tuned/elementwise/{add,copy}/{float16,float32,int8}/ .
 * The fused (1, n, H) iteration space is one flat array of count elements.
 * ======================================================================== */

/* T_add = A + B in fp16: one IEEE rounding of the exact sum (the exact sum of
 * two fp16 values fits fp32 exactly or rounds innocuously: 24 >= 2*11+2).
 * Pinned by: numpy.float16 addition over seeded and special-value inputs. */
void oracle_add_f16(const f16* A, const f16* B, f16* out, int64_t count, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t i = 0; i < count; ++i) out[i] = f2h(h2f(A[i]) + h2f(B[i]));
}

void oracle_add_f32(const float* A, const float* B, float* out, int64_t count, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t i = 0; i < count; ++i) out[i] = A[i] + B[i];
}

/* int8 add wraps modulo 256 (two's complement), as the generated kernel's
 * per-byte add does.  Pinned by: exhaustive 256x256 table vs numpy int8. */
void oracle_add_i8(const int8_t* A, const int8_t* B, int8_t* out, int64_t count, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t i = 0; i < count; ++i) out[i] = (int8_t)(uint8_t)((uint8_t)A[i] + (uint8_t)B[i]);
}

/* B = A, bit for bit (NaN payloads included). */
void oracle_copy_bytes(const void* A, void* B, int64_t nbytes, int nthreads) {
  const int64_t chunk = 1 << 20;
  const int64_t nchunks = (nbytes + chunk - 1) / chunk;
  OMP_FOR(nthreads)
  for (int64_t c = 0; c < nchunks; ++c) {
    int64_t lo = c * chunk, len = nbytes - lo < chunk ? nbytes - lo : chunk;
    memcpy((char*)B + lo, (const char*)A + lo, (size_t)len);
  }
}

/* compute = Cast(float32, A): exact widening.  Pinned by: all 65536 patterns
 * against numpy and against oracle_soft_h2f. */
void oracle_cast_f16_f32(const f16* A, float* out, int64_t count, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t i = 0; i < count; ++i) out[i] = h2f(A[i]);
}

/* Narrowing cast: round to nearest even, overflow to +-inf, subnormals kept,
 * NaN stays NaN.  Pinned by: boundary table + 2^24 random patterns vs numpy
 * and vs oracle_soft_f2h. */
void oracle_cast_f32_f16(const float* A, f16* out, int64_t count, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t i = 0; i < count; ++i) out[i] = f2h(A[i]);
}

/* ===========================================================================
 * Row reductions.
 * ======================================================================== */

/* fused_layer_norm_cast1: experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:607-
 * 636 and experiment/dtas_tuned/general_reduction/layernorm/profile_dlight.py:
 * 7-40.  s0 = sum x, s1 = sum x*x (fp32, sequential); the PrimFunc multiplies
 * by the fp32 literal 1/H (0.000390625 for H = 2560), it does not divide;
 * out = f16((x - s0*inv)*rsqrt(s1*inv - (s0*inv)*(s0*inv) + eps)*gamma + beta).
 * Pinned by: fp64 numpy layer norm (atol 1e-2), torch.layer_norm on CPU,
 * affine invariance, gamma=1/beta=0 => row mean 0 / variance 1. */
void oracle_layer_norm_f32_f16(const float* x, const float* gamma, const float* beta, f16* out,
                               int64_t n, int64_t H, float eps, int nthreads) {
  const float inv = (float)(1.0 / (double)H);
  OMP_FOR(nthreads)
  for (int64_t r = 0; r < n; ++r) {
    const float* xr = x + r * H;
    float s0 = 0.f, s1 = 0.f;
    for (int64_t k = 0; k < H; ++k) {
      s0 = s0 + xr[k];
      s1 = s1 + xr[k] * xr[k];
    }
    const float mean = s0 * inv;
    const float rstd = 1.0f / sqrtf(s1 * inv - mean * mean + eps);
    for (int64_t k = 0; k < H; ++k) out[r * H + k] = f2h((xr[k] - mean) * rstd * gamma[k] + beta[k]);
  }
}

/* layer_norm / layer_norm1: experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:846-896, the same arithmetic
 * with the result left in fp32.
 * Pinned by: rounds to the fused function's fp16 result bit for bit; fp64 closed form (1e-4); torch.layer_norm. */
void oracle_layer_norm_f32(const float* x, const float* gamma, const float* beta, float* out, int64_t n, int64_t H,
                           float eps, int nthreads) {
  const float inv = (float)(1.0 / (double)H);
  OMP_FOR(nthreads)
  for (int64_t r = 0; r < n; ++r) {
    const float* xr = x + r * H;
    float s0 = 0.f, s1 = 0.f;
    for (int64_t k = 0; k < H; ++k) {
      s0 = s0 + xr[k];
      s1 = s1 + xr[k] * xr[k];
    }
    const float mean = s0 * inv;
    const float rstd = 1.0f / sqrtf(s1 * inv - mean * mean + eps);
    for (int64_t k = 0; k < H; ++k) out[r * H + k] = (xr[k] - mean) * rstd * gamma[k] + beta[k];
  }
}

/* rms_norm: no counterpart in the reference (PARITY UNPINNED by the
 * reference).  Closed form: ss = sum f32(x)^2 in fp32;
 * out = f16(f32(x) * rsqrt(ss/H + eps) * f32(w)), one final rounding.
 * Pinned by: fp64 numpy closed form (atol 1e-2), torch.nn.functional.rms_norm
 * on CPU, scale invariance, w = 1 => row rms 1. */
void oracle_rms_norm_f16(const f16* x, const f16* w, f16* out, int64_t n, int64_t H, float eps,
                         int nthreads) {
  const float inv = (float)(1.0 / (double)H);
  OMP_FOR(nthreads)
  for (int64_t r = 0; r < n; ++r) {
    const f16* xr = x + r * H;
    float ss = 0.f;
    for (int64_t k = 0; k < H; ++k) {
      float v = h2f(xr[k]);
      ss = ss + v * v;
    }
    const float rs = 1.0f / sqrtf(ss * inv + eps);
    for (int64_t k = 0; k < H; ++k) out[r * H + k] = f2h(h2f(xr[k]) * rs * h2f(w[k]));
  }
}

/* fused_softmax_cast: experiment/dtas_tuned/general_reduction/softmax/
 * profile_dlight.py:8-52 (3-D form) and experiment/ModelIR/dolly-v2-3b-q0f16/
 * before_dl.py:756-800 (fused_softmax_cast3, 4-D (1,32,n,m) form): per row
 * mx = max(-FLT_MAX, x...) (the init is -3.4028234663852886e+38, not -inf),
 * e = exp(x - mx) in fp32, s = sum e (sequential), out = f16(e / s).
 * Pinned by: fp64 numpy / scipy.special.softmax (atol 1e-2), rows sum to 1,
 * shift invariance, a single column gives exactly 1.0, a constant row 1/cols. */
void oracle_softmax_f32_f16(const float* x, f16* out, int64_t rows, int64_t cols, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float mx = -3.4028234663852886e+38f;
    for (int64_t k = 0; k < cols; ++k) mx = xr[k] > mx ? xr[k] : mx;
    float s = 0.f;
    for (int64_t k = 0; k < cols; ++k) s = s + expf(xr[k] - mx);
    for (int64_t k = 0; k < cols; ++k) out[r * cols + k] = f2h(expf(xr[k] - mx) / s);
  }
}

/* divide2: experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:57-65, T_divide[k] = A[k] / B[()] in fp32.
 * Pinned by: numpy float32 division (bit-exact), the float64 quotient rounded once, B = 1 is the identity. */
void oracle_divide_f32(const float* a, const float* b, float* out, int64_t count) {
  for (int64_t k = 0; k < count; ++k) out[k] = a[k] / *b;
}

/* softmax_with_temperature: experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:4154-4161 = divide2 (:57-65,
 * A / B[()] in fp32) then softmax2 (:1062-1096: max from -FLT_MAX, exp(x - max), sequential sum, exp / sum;
 * fp32 throughout).
 * Pinned by: fp64 numpy softmax(x / t), rows sum to 1, temperature 1 equals the plain softmax of the row,
 * a single column gives exactly 1.0. */
void oracle_softmax_temperature_f32(const float* x, const float* temperature, float* out, int64_t rows, int64_t cols,
                                    int nthreads) {
  const float t = *temperature;
  OMP_FOR(nthreads)
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float* o = out + r * cols;
    float mx = -3.4028234663852886e+38f;
    for (int64_t k = 0; k < cols; ++k) {
      o[k] = xr[k] / t;
      mx = o[k] > mx ? o[k] : mx;
    }
    float s = 0.f;
    for (int64_t k = 0; k < cols; ++k) {
      o[k] = expf(o[k] - mx);
      s = s + o[k];
    }
    for (int64_t k = 0; k < cols; ++k) o[k] = o[k] / s;
  }
}

/* Same PrimFunc with an fp16 input buffer (the [32n, n] attention-score form):
 * the values are widened to fp32 first, then the identical fp32 pipeline. */
void oracle_softmax_f16_f16(const f16* x, f16* out, int64_t rows, int64_t cols, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t r = 0; r < rows; ++r) {
    const f16* xr = x + r * cols;
    float mx = -3.4028234663852886e+38f;
    for (int64_t k = 0; k < cols; ++k) {
      float v = h2f(xr[k]);
      mx = v > mx ? v : mx;
    }
    float s = 0.f;
    for (int64_t k = 0; k < cols; ++k) s = s + expf(h2f(xr[k]) - mx);
    for (int64_t k = 0; k < cols; ++k) out[r * cols + k] = f2h(expf(h2f(xr[k]) - mx) / s);
  }
}

/* ===========================================================================
 * GEMV / GEMM: C[i, j] = sum_k A[i, k] * W[j, k] (+ bias[j]).
 * GEMV is fused_NT_matmul10_add5 (before_dl.py:96-113), GEMM is
 * fused_NT_matmul4_add1 (before_dl.py:320-341); GEMV is the M = 1 case.
 * acc_f16 = 0: products and the running sum in fp32, one rounding to fp16 at
 *              the end (then "+ bias" in fp16 if bias is given) -- the
 *              fp32-accumulate contract of the benchmark configs.
 * acc_f16 = 1: the PrimFunc text literally: the running sum is an fp16 buffer,
 *              acc = f16(acc + f16(a*w)) for k ascending.
 * acc_f16 = 2: the reference's scheduled GEMM: an fp16 accumulator fragment updated once per k step of 16 by
 *              one tensor-core instruction (wmma 16x16x16 with "wmma.accumulator" in float16,
 *              experiment/testIR/GEMM/m_n2560_k10240/wmma/16x16x16/i2j4_x7y2_in8.py:19,37): the 16 exact products
 *              of a step are added to the accumulator at fp32 precision (k ascending here; the order inside
 *              the instruction is not part of any interface) and the result is rounded to fp16 once per step.
 * Pinned by: fp64 numpy A @ W.T (rtol 1e-2), exact cases (K = 1, identity /
 * permutation W, one-hot rows), brute force on tiny ragged shapes,
 * torch.matmul on CPU.
 * ======================================================================== */
/* One element's product with an fp16 accumulator rounded once per k step of 16 (acc_f16 = 2). */
static f16 dot_f16_k16(const f16* a, const f16* w, int64_t K) {
  f16 acc = 0;
  for (int64_t k0 = 0; k0 < K; k0 += 16) {
    float s = h2f(acc);
    const int64_t k1 = k0 + 16 < K ? k0 + 16 : K;
    for (int64_t k = k0; k < k1; ++k) s = s + h2f(a[k]) * h2f(w[k]);
    acc = f2h(s);
  }
  return acc;
}

void oracle_gemm_f16(const f16* A, const f16* W, const f16* bias, f16* C, int64_t M, int64_t N,
                     int64_t K, int acc_f16, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t ij = 0; ij < M * N; ++ij) {
    const int64_t i = ij / N, j = ij % N;
    const f16* a = A + i * K;
    const f16* w = W + j * K;
    f16 r;
    if (acc_f16 == 2) {
      r = dot_f16_k16(a, w, K);
    } else if (acc_f16) {
      f16 acc = 0;
      for (int64_t k = 0; k < K; ++k) acc = f2h(h2f(acc) + h2f(f2h(h2f(a[k]) * h2f(w[k]))));
      r = acc;
    } else {
      float acc = 0.f;
      for (int64_t k = 0; k < K; ++k) acc = acc + h2f(a[k]) * h2f(w[k]);
      r = f2h(acc);
    }
    if (bias) r = f2h(h2f(r) + h2f(bias[j]));
    C[ij] = r;
  }
}

/* GEMV in the order of the reference's own scheduled kernel
 * (experiment/testIR/GEMV/m1n2560k10240/IR/5wt.py:11-92: the GEMV rule's two-level rfactor, every buffer fp16):
 *   rf[j], j < 256 (:12, :35-56): for o ascending, rf[j] = f16(rf[j] + f16(x[256 o + j] * W[row][256 o + j]))
 *   rf1[t], t < 32 (:13, :57-73): from 0, + rf[8 t], + rf[8 t + 1], ..., + rf[8 t + 7], each step rounded
 *   the 32 rf1 over threadIdx.x (:74-84): a cross-thread reduction, which TVM lowers to the shuffle tree that
 *     the reference's committed kernels show (experiment/dtas_tuned/general_reduction/layernorm/top1_256/
 *     tvm_device_kernels.cu:184-203): v[t] = f16(v[t] + v[t + d]) for d = 16, 8, 4, 2, 1; lane 0 holds the sum
 *   y = f16(sum + bias[row]) (:85-91)
 * The schedule is written for K = 10240; k past K contributes nothing here (the rule predicates it).
 * Pinned by: hand-built inputs whose result depends on each of the three stages' order (tests/
 * test_oracle_matmul.py), exactness on small integers, and agreement with the fp64 product within fp16 error. */
void oracle_gemv_f16_rf(const f16* x, const f16* W, const f16* bias, f16* y, int64_t N, int64_t K, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t row = 0; row < N; ++row) {
    const f16* w = W + row * K;
    f16 rf[256];
    for (int j = 0; j < 256; ++j) rf[j] = 0;
    for (int64_t o = 0; o * 256 < K; ++o)
      for (int j = 0; j < 256; ++j) {
        const int64_t k = o * 256 + j;
        if (k < K) rf[j] = f2h(h2f(rf[j]) + h2f(f2h(h2f(x[k]) * h2f(w[k]))));
      }
    f16 v[32];
    for (int t = 0; t < 32; ++t) {
      f16 acc = 0;
      for (int i = 0; i < 8; ++i) acc = f2h(h2f(acc) + h2f(rf[8 * t + i]));
      v[t] = acc;
    }
    for (int d = 16; d >= 1; d >>= 1)
      for (int t = 0; t < d; ++t) v[t] = f2h(h2f(v[t]) + h2f(v[t + d]));
    f16 r = v[0];
    if (bias) r = f2h(h2f(r) + h2f(bias[row]));
    y[row] = r;
  }
}

/* The same sum with the fp32 accumulator returned unrounded; the parity tests
 * use it to bound the GPU's fp32 partial-sum reordering separately from the
 * final fp16 rounding. */
void oracle_gemm_f16_f32out(const f16* A, const f16* W, float* C, int64_t M, int64_t N, int64_t K,
                            int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t ij = 0; ij < M * N; ++ij) {
    const int64_t i = ij / N, j = ij % N;
    const f16* a = A + i * K;
    const f16* w = W + j * K;
    float acc = 0.f;
    for (int64_t k = 0; k < K; ++k) acc = acc + h2f(a[k]) * h2f(w[k]);
    C[ij] = acc;
  }
}

/* ==========================================================================
 * GEMM with the model's fused epilogues: fused_NT_matmul2_add1_add3_add3
 * (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:163-200), ..._add3_cast (:202-246) and
 * fused_NT_matmul3_add2_gelu (:248-318).  Every intermediate of those PrimFuncs is an fp16
 * buffer, so every line below rounds to fp16, in the PrimFunc's operand order.
 *   kind 0: C = mm (+ bias)                              (same as oracle_gemm_f16)
 *   kind 1: C = (res1 + (mm + bias)) + res2              fp16 out
 *   kind 2: the same, T.Cast("float32")                  fp32 out
 *   kind 3: t = mm + bias; C = t * (0.5 + f16(f16(erf(f32(f16(t * f16(0.70710678...))))) * 0.5))
 * mm is the fp32-accumulated product rounded once (acc_f16 = 1: the literal fp16 running sum; 2: an fp16
 * accumulator rounded once per k step of 16, see oracle_gemm_f16).
 * erf is libm's erff; the device uses its own erff, both well inside the fp16 rounding that
 * follows except at rounding boundaries, which the parity tests allow for (1 fp16 ulp).
 * Pinned by: numpy float16 arithmetic step by step, scipy.special.erf in float64 (tolerance),
 * kind 1 with zero residuals == kind 0, gelu(0) = 0, gelu(x) -> x / 0 for large |x|, kind 2 ==
 * widened kind 1.
 * ======================================================================== */
void oracle_gemm_f16_fused(const f16* A, const f16* W, const f16* bias, const f16* res1, const f16* res2,
                           void* C, int64_t M, int64_t N, int64_t K, int kind, int acc_f16, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t ij = 0; ij < M * N; ++ij) {
    const int64_t i = ij / N, j = ij % N;
    const f16* a = A + i * K;
    const f16* w = W + j * K;
    f16 t;
    if (acc_f16 == 2) {
      t = dot_f16_k16(a, w, K);
    } else if (acc_f16) {
      f16 acc = 0;
      for (int64_t k = 0; k < K; ++k) acc = f2h(h2f(acc) + h2f(f2h(h2f(a[k]) * h2f(w[k]))));
      t = acc;
    } else {
      float acc = 0.f;
      for (int64_t k = 0; k < K; ++k) acc = acc + h2f(a[k]) * h2f(w[k]);
      t = f2h(acc);
    }
    if (bias) t = f2h(h2f(t) + h2f(bias[j]));                    /* T_add */
    if (kind == 1 || kind == 2) {
      t = f2h(h2f(res1[ij]) + h2f(t));                           /* T_add_1 = lv58 + T_add */
      t = f2h(h2f(t) + h2f(res2[ij]));                           /* T_add_2 = T_add_1 + lv2 */
    } else if (kind == 3) {
      const f16 m = f2h(h2f(t) * h2f(f2h(0.70710678118654757f))); /* T_multiply */
      const f16 e = f2h(erff(h2f(m)));                            /* compute .. compute_2 */
      const f16 h = f2h(h2f(e) * 0.5f);                           /* T_multiply_1 */
      const f16 g = f2h(0.5f + h2f(h));                           /* T_add_1 */
      t = f2h(h2f(t) * h2f(g));                                   /* T_multiply_2 */
    }
    if (kind == 2) ((float*)C)[ij] = h2f(t);
    else ((f16*)C)[ij] = t;
  }
}

/* ==========================================================================
 * Attention scores: fused_NT_matmul1_divide_maximum_minimum_cast2
 * (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:116-160).
 *   NT_matmul[h,i,j] = sum_k Q[h,i,k] * K[h,j,k]            (fp16 buffer)
 *   T_divide  = NT_matmul * T.float16(0.11179...)            (a multiply by the fp16 constant)
 *   T_maximum = max(T_divide, T.float16(-65504))
 *   T_minimum = min(T_maximum, mask[0,0,i,j])
 *   compute   = T.Cast("float32", T_minimum)
 * The product is accumulated in fp32 and rounded once (acc_f16 = 1: the literal fp16 running sum).
 * Pinned by: numpy float16 arithmetic step by step (bit-exact), the float64 closed form, a mask of
 * +65504 (no effect) / -65504 (everything masked) / a causal triangle, heads independent, -inf
 * products clamped to -65504.
 * ======================================================================== */
void oracle_attn_scores_f16_f32(const f16* Q, const f16* Kmat, const f16* mask, float* out, int64_t heads, int64_t n,
                                int64_t m, int64_t d, float scale, int acc_f16, int nthreads) {
  const f16 scale_h = f2h(scale);
  OMP_FOR(nthreads)
  for (int64_t idx = 0; idx < heads * n * m; ++idx) {
    const int64_t h = idx / (n * m), i = (idx / m) % n, j = idx % m;
    const f16* q = Q + (h * n + i) * d;
    const f16* k = Kmat + (h * m + j) * d;
    f16 t;
    if (acc_f16) {
      f16 acc = 0;
      for (int64_t e = 0; e < d; ++e) acc = f2h(h2f(acc) + h2f(f2h(h2f(q[e]) * h2f(k[e]))));
      t = acc;
    } else {
      float acc = 0.f;
      for (int64_t e = 0; e < d; ++e) acc = acc + h2f(q[e]) * h2f(k[e]);
      t = f2h(acc);
    }
    t = f2h(h2f(t) * h2f(scale_h));
    t = f2h(fmaxf(h2f(t), -65504.f));
    t = f2h(fminf(h2f(t), h2f(mask[i * m + j])));
    out[idx] = h2f(t);
  }
}

/* ========================================================================
 * attention output: matmul8 (before_dl.py:915-929) and, with n = 1, matmul10 (:899-912)
 *   matmul[0, h, i, e] = sum_k A[0, h, i, k] * B[0, h, k, e]        (an fp16 buffer)
 * P[heads, n, m], V[heads, m, d] (k-major: V's rows run along d), out[heads, n, d].  The product is
 * accumulated in fp32 and rounded once (acc_f16 = 1: the literal fp16 running sum, k ascending).
 * Pinned by: numpy's float64 matmul, P = identity / a one-hot row selector (out = rows of V, bit
 * exact), a constant row 1/m of P (column means of V), linearity in P for exactly representable
 * data, heads independent, m = 0 (zeros), n = 1 equal to a row of the n > 1 case.
 * ======================================================================== */
void oracle_attn_pv_f16(const f16* P, const f16* V, f16* out, int64_t heads, int64_t n, int64_t m, int64_t d,
                        int acc_f16, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t idx = 0; idx < heads * n * d; ++idx) {
    const int64_t h = idx / (n * d), i = (idx / d) % n, e = idx % d;
    const f16* p = P + (h * n + i) * m;
    const f16* v = V + h * m * d + e;
    if (acc_f16) {
      f16 acc = 0;
      for (int64_t k = 0; k < m; ++k) acc = f2h(h2f(acc) + h2f(f2h(h2f(p[k]) * h2f(v[k * d]))));
      out[idx] = acc;
    } else {
      float acc = 0.f;
      for (int64_t k = 0; k < m; ++k) acc = acc + h2f(p[k]) * h2f(v[k * d]);
      out[idx] = f2h(acc);
    }
  }
}

/* ========================================================================
 * 8-bit weights with fp16 group scales (experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py)
 *   decode[i, j] = (Cast("float16", (Wq[i, j/4] >> (8 * (j % 4))) & 255) - float16(127)) * S[i, j/32]
 * fused_decode3 (:335-343) stores it; fused_fused_decode2_fused_NT_matmul_add (:401-426) and
 * fused_fused_decode4_fused_NT_matmul3_add2_gelu (:428-502) multiply x by it (fp32 accumulation here,
 * acc_f16 = 1 the literal fp16 running sum), then + bias (and GELU) in fp16 steps as in
 * oracle_gemm_f16_fused.
 * Pinned by: numpy float16 arithmetic on the bytes of the little-endian words (bit-exact), bytes
 * 127 / 0 / 255 (0, -127 s, 128 s), the byte order inside a word, the scale group boundary at 32,
 * float64 closed form; the GEMV equals the pinned GEMM oracle on the decoded matrix bit for bit.
 * ======================================================================== */
static f16 decode_q8(const uint32_t* Wq, const f16* S, int64_t K, int64_t i, int64_t j) {
  const uint32_t byte = (Wq[i * (K / 4) + j / 4] >> (8 * (j % 4))) & 255u;
  const f16 q = f2h(h2f(f2h((float)byte)) - 127.f);
  return f2h(h2f(q) * h2f(S[i * (K / 32) + j / 32]));
}

void oracle_decode_q8_f16(const uint32_t* Wq, const f16* S, f16* W, int64_t N, int64_t K, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t ij = 0; ij < N * K; ++ij) W[ij] = decode_q8(Wq, S, K, ij / K, ij % K);
}

void oracle_gemv_q8_f16(const f16* x, const uint32_t* Wq, const f16* S, const f16* bias, f16* y, int64_t N, int64_t K,
                        int kind, int acc_f16, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t i = 0; i < N; ++i) {
    f16 t;
    if (acc_f16) {
      f16 acc = 0;
      for (int64_t k = 0; k < K; ++k) acc = f2h(h2f(acc) + h2f(f2h(h2f(x[k]) * h2f(decode_q8(Wq, S, K, i, k)))));
      t = acc;
    } else {
      float acc = 0.f;
      for (int64_t k = 0; k < K; ++k) acc = acc + h2f(x[k]) * h2f(decode_q8(Wq, S, K, i, k));
      t = f2h(acc);
    }
    if (bias) t = f2h(h2f(t) + h2f(bias[i]));
    if (kind == 3) {
      const f16 m = f2h(h2f(t) * h2f(f2h(0.70710678118654757f)));
      const f16 e = f2h(erff(h2f(m)));
      const f16 h = f2h(h2f(e) * 0.5f);
      const f16 g = f2h(0.5f + h2f(h));
      t = f2h(h2f(t) * h2f(g));
    }
    y[i] = t;
  }
}

/* ========================================================================
 * fp32 GEMV: NT_matmul5 (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:8-19)
 *   NT_matmul[0,0,i] = sum_k A[0,0,k] * B[i,k]     fp32 throughout, k ascending, no contraction
 * Pinned by: float64 closed form (error bound from sum |x||w|), numpy's float32 dot on short rows,
 * one-hot x (a column of W, exact), K = 1 (one rounded product), exactly representable integers.
 * ======================================================================== */
void oracle_gemv_f32(const float* x, const float* W, float* y, int64_t N, int64_t K, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t i = 0; i < N; ++i) {
    float acc = 0.f;
    for (int64_t k = 0; k < K; ++k) acc = acc + x[k] * W[i * K + k];
    y[i] = acc;
  }
}

/* ========================================================================
 * The other q8 forms of the same model file (experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py):
 *  fused_fused_decode1_take1 (:357-369; the one-row form fused_fused_decode1_take :346-355):
 *      out[i, j] = decode(Wq, S)[ids[i], j]                      -- the embedding rows, dequantised
 *  fused_fused_decode6_NT_matmul5 (:640-657): fp32 scales, fp32 x and y
 *      W[i, j] = float32(fp16(byte) - fp16(127)) * S32[i, j/32]   -- one fp32 rounding (the product)
 *      y[i]    = sum_k x[k] * W[i, k]                             -- fp32, k ascending, no contraction
 * Pinned by: rows of the pinned dequantiser picked with numpy indexing (bit-exact); numpy float32 arithmetic on the
 * bytes (bit-exact W), the pinned fp32 GEMV on that W (bit-exact y), float64 closed form, one-hot x.
 * ======================================================================== */
/* rotary_embedding (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:1023-1035), every step an fp16 tensor op:
 *   rotary[s,h,j] = j < rot ? B[pos,j] * A[s,h,j] + C[pos,j] * (j < rot/2 ? A[s,h,j+rot/2] * -1 : A[s,h,j-rot/2]) : A[s,h,j]
 * with pos = m + s - n.  Pinned by: numpy float16 arithmetic step by step (bit-exact), cos = 1 / sin = 0 (identity),
 * the float64 rotation (tolerance), preserved pair norms for cos^2 + sin^2 = 1. */
void oracle_rotary_f16(const f16* A, const f16* B, const f16* C, f16* out, int64_t n, int64_t m, int64_t heads, int64_t d,
                       int64_t rot, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t sh = 0; sh < n * heads; ++sh) {
    const int64_t pos = m + sh / heads - n;
    const f16* a = A + sh * d;
    for (int64_t j = 0; j < d; ++j) {
      if (j >= rot) { out[sh * d + j] = a[j]; continue; }
      const f16 partner = j < rot / 2 ? f2h(h2f(a[j + rot / 2]) * -1.f) : a[j - rot / 2];
      const f16 t1 = f2h(h2f(B[pos * rot + j]) * h2f(a[j]));
      const f16 t2 = f2h(h2f(C[pos * rot + j]) * h2f(partner));
      out[sh * d + j] = f2h(h2f(t1) + h2f(t2));
    }
  }
}

/* take (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:1151-1163): T_take[i, j] = A[B[i], j].
 * Pinned by: numpy indexing (bit-exact). */
void oracle_take_f16(const f16* A, const int32_t* ids, f16* out, int64_t n, int64_t H, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t ij = 0; ij < n * H; ++ij) out[ij] = A[(int64_t)ids[ij / H] * H + ij % H];
}

void oracle_take_q8_f16(const uint32_t* Wq, const f16* S, const int32_t* ids, f16* out, int64_t n, int64_t K, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t ij = 0; ij < n * K; ++ij) out[ij] = decode_q8(Wq, S, K, ids[ij / K], ij % K);
}

void oracle_gemv_q8_f32(const float* x, const uint32_t* Wq, const float* S, float* y, int64_t N, int64_t K, int nthreads) {
  OMP_FOR(nthreads)
  for (int64_t i = 0; i < N; ++i) {
    float acc = 0.f;
    for (int64_t k = 0; k < K; ++k) {
      const uint32_t byte = (Wq[i * (K / 4) + k / 4] >> (8 * (k % 4))) & 255u;
      const float q = h2f(f2h(h2f(f2h((float)byte)) - 127.f));
      const float w = q * S[i * (K / 32) + k / 32];
      acc = acc + x[k] * w;
    }
    y[i] = acc;
  }
}

int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

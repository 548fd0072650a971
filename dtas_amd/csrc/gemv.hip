// Decode GEMV for gfx950: y[N] = epilogue(W[N,K] . x[K]), fp16 in/out, fp32 accumulate; the epilogues are
// those of the fused decode PrimFuncs (+ bias; + bias + two residuals, optionally widened; + bias, GELU).
//
// Replaces the kernel DTAS's GEMV rule generates (python/dtas/schedule/tir_gemv.py:33-249:
// two-level rfactor split-K over TR lanes x VEC_C elements, weight to registers with vector
// loads, x staged in shared memory; example output
// experiment/testIR/GEMV/m1n2560k10240/IR/5wt.py:8-92, block 32x16, grid N/16).
//
// MI355X shape: a workgroup owns `rows` consecutive rows of W and splits K over all of its
// lanes and wavefronts: lane t takes the 128-bit chunks t, t+block, ... of every row, so each
// wavefront access is one contiguous 1 KiB span of a W row and W is streamed from HBM exactly
// once, non-temporal.  The matching x chunk is loaded once per step and reused for all `rows`
// rows (x is a few KiB and stays in L2/L1).  fp32 partial sums are folded with DPP inside a
// wavefront and through one LDS slot per wavefront across them.
#include "dtas_device.h"
#include "dtas_host.h"

namespace dtas {
namespace {

__device__ __forceinline__ float dot8(u32x4 a, u32x4 b, float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // copy the lanes out first: a bit_cast applied directly to a vector element reads element 0
    const unsigned ai = a[i], bi = b[i];
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, ai), __builtin_bit_cast(f16x2, bi), acc, false);
  }
  return acc;
}

// What follows the dot product in the fused decode PrimFuncs (one fp16 tensor per step, each step
// rounded): + bias; then either nothing, or res1 + t, then + res2 (optionally widened to an fp32 y), or
// the erf-GELU.  `kind` is a DTAS_EPI_* value.
struct GemvEpilogue {
  const half_t* bias;  // [N] or nullptr
  const half_t* res1;  // [N]: the ADD2 kinds
  const half_t* res2;  // [N]: the ADD2 kinds
  int kind;
};

__device__ __forceinline__ void finish(float acc, const GemvEpilogue& ep, void* y, int64_t j) {
  // round the fp32 sum to fp16 first, then "+ bias" as the PrimFunc's separate fp16 T_add block
  half_t t = static_cast<half_t>(acc);
  if (ep.bias) t = static_cast<half_t>(static_cast<float>(t) + static_cast<float>(ep.bias[j]));
  if (ep.kind == DTAS_EPI_BIAS_ADD2 || ep.kind == DTAS_EPI_BIAS_ADD2_CAST_F32) {
    t = static_cast<half_t>(static_cast<float>(ep.res1[j]) + static_cast<float>(t));
    t = static_cast<half_t>(static_cast<float>(t) + static_cast<float>(ep.res2[j]));
  } else if (ep.kind == DTAS_EPI_BIAS_GELU) {
    t = gelu_erf_f16_steps(t);
  }
  if (ep.kind == DTAS_EPI_BIAS_ADD2_CAST_F32) static_cast<float*>(y)[j] = static_cast<float>(t);
  else static_cast<half_t*>(y)[j] = t;
}

// The same with the operands already in registers (the split-K kernel requests them before it streams W: read at the
// end, each would cost the launch a round trip to memory of its own).
__device__ __forceinline__ void finish_with(float acc, int kind, bool has_bias, half_t bias, half_t r1, half_t r2, void* y, int64_t j) {
  half_t t = static_cast<half_t>(acc);
  if (has_bias) t = static_cast<half_t>(static_cast<float>(t) + static_cast<float>(bias));
  if (kind == DTAS_EPI_BIAS_ADD2 || kind == DTAS_EPI_BIAS_ADD2_CAST_F32) {
    t = static_cast<half_t>(static_cast<float>(r1) + static_cast<float>(t));
    t = static_cast<half_t>(static_cast<float>(t) + static_cast<float>(r2));
  } else if (kind == DTAS_EPI_BIAS_GELU) {
    t = gelu_erf_f16_steps(t);
  }
  if (kind == DTAS_EPI_BIAS_ADD2_CAST_F32) static_cast<float*>(y)[j] = static_cast<float>(t);
  else static_cast<half_t*>(y)[j] = t;
}

template <int R>
__global__ void __launch_bounds__(512) gemv_splitk_kernel(const half_t* __restrict__ x, const half_t* __restrict__ W,
                                                          GemvEpilogue ep, void* __restrict__ y, int64_t N, int64_t K) {
  __shared__ float part[8][R];
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
  const int64_t nvec = K >> 3;
  const u32x4* xv = reinterpret_cast<const u32x4*>(x);
  const u32x4* wv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    // rows past N re-read the last row; their sums are never stored
    const int64_t row = row0 + r < N ? row0 + r : N - 1;
    wv[r] = reinterpret_cast<const u32x4*>(W + row * K);
  }
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  // thread r < R stores row row0 + r: its bias and residual elements, requested now and kept as loaded
  const bool stores = threadIdx.x < R && row0 + threadIdx.x < N;
  const bool add2 = ep.kind == DTAS_EPI_BIAS_ADD2 || ep.kind == DTAS_EPI_BIAS_ADD2_CAST_F32;
  const half_t zero = static_cast<half_t>(0.f);
  const half_t e_bias = stores && ep.bias ? ep.bias[row0 + threadIdx.x] : zero;
  const half_t e_r1 = stores && add2 ? ep.res1[row0 + threadIdx.x] : zero;
  const half_t e_r2 = stores && add2 ? ep.res2[row0 + threadIdx.x] : zero;

#pragma unroll 2
  for (int64_t i = threadIdx.x; i < nvec; i += blockDim.x) {
    const u32x4 xr = xv[i];
    u32x4 wr[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wr[r] = load_stream(wv[r] + i);
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = dot8(xr, wr[r], acc[r]);
  }
  asm volatile("" ::"v"(e_bias), "v"(e_r1), "v"(e_r2));  // (they exist by now: their loads stay where they were written)

  const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float s = wave_sum(acc[r]);
    if ((threadIdx.x & 63) == 0) part[wave][r] = s;
  }
  __syncthreads();
  if (threadIdx.x < R && row0 + threadIdx.x < N) {
    float s = 0.f;
    for (int w = 0; w < nwaves; ++w) s += part[w][threadIdx.x];
    finish_with(s, ep.kind, ep.bias != nullptr, e_bias, e_r1, e_r2, y, row0 + threadIdx.x);
  }
}

// The same product with every sum in fp16, in the order of the reference's own scheduled kernel
// (experiment/testIR/GEMV/m1n2560k10240/IR/5wt.py:11-92: rfactor over 256 strided chains per row, held 8 per
// thread by 32 threads; the 8 folded in order; the 32 threads joined by the shuffle tree TVM lowers a
// cross-thread reduction to, strides 16, 8, 4, 2, 1 as in .../layernorm/top1_256/tvm_device_kernels.cu:184-203).
// Half a wavefront plays the 32 threads of a row: lane t owns chains j = 8t .. 8t+7, i.e. the 16-byte chunk t of
// every 256-element step, so a step is 512 contiguous bytes of the row.  Products are rounded to fp16 before they
// are added (no fused multiply-add: the PrimFunc has two fp16 operations).  Bit-identical to the CPU restatement.
template <bool VEC>
__global__ void __launch_bounds__(256) gemv_rf16_kernel(const half_t* __restrict__ x, const half_t* __restrict__ W,
                                                        GemvEpilogue ep, void* __restrict__ y, int64_t N, int64_t K) {
#pragma clang fp contract(off)
  const int t = threadIdx.x & 31;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 8 + (threadIdx.x >> 5);
  const half_t* w = W + (row < N ? row : N - 1) * K;  // rows past N re-read the last row; never stored
  half_t rf[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) rf[i] = static_cast<half_t>(0.f);
  for (int64_t k0 = 8 * t; k0 < K; k0 += 256) {
    if (VEC) {  // K % 8 == 0: a chunk is all inside the row
      const f16x8 xv = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(x + k0));
      const f16x8 wv = __builtin_bit_cast(f16x8, load_stream(reinterpret_cast<const u32x4*>(w + k0)));
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const half_t p = xv[i] * wv[i];
        rf[i] = rf[i] + p;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (k0 + i < K) {
          const half_t p = x[k0 + i] * w[k0 + i];
          rf[i] = rf[i] + p;
        }
    }
  }
  half_t acc = static_cast<half_t>(0.f);
#pragma unroll
  for (int i = 0; i < 8; ++i) acc = acc + rf[i];
#pragma unroll
  for (int d = 16; d >= 1; d >>= 1) {
    // lane t adds lane t + d of its group of 32 (past the group: its own value, which lane 0's chain never reads)
    const half_t other = __builtin_bit_cast(half_t, static_cast<unsigned short>(__shfl_down(static_cast<int>(__builtin_bit_cast(unsigned short, acc)), d, 32)));
    acc = acc + other;
  }
  if (t == 0 && row < N) finish(static_cast<float>(acc), ep, y, row);
}

// fp32 operands and result (NT_matmul5, experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:8-19: the
// 50280 x 2560 vocabulary projection of the decode graph): the same workgroup shape, 4 elements per
// 128-bit access, fused multiply-adds in fp32.
template <int R>
__global__ void __launch_bounds__(512) gemv_f32_kernel(const float* __restrict__ x, const float* __restrict__ W,
                                                       float* __restrict__ y, int64_t N, int64_t K) {
  __shared__ float part[8][R];
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
  const int64_t nvec = K >> 2;
  const f32x4* xv = reinterpret_cast<const f32x4*>(x);
  const f32x4* wv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + r < N ? row0 + r : N - 1;  // rows past N re-read the last row; never stored
    wv[r] = reinterpret_cast<const f32x4*>(W + row * K);
  }
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
#pragma unroll 2
  for (int64_t i = threadIdx.x; i < nvec; i += blockDim.x) {
    const f32x4 xr = xv[i];
    f32x4 wr[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wr[r] = load_stream(wv[r] + i);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[r] = fmaf(xr[e], wr[r][e], acc[r]);
  }
  const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float s = wave_sum(acc[r]);
    if ((threadIdx.x & 63) == 0) part[wave][r] = s;
  }
  __syncthreads();
  if (threadIdx.x < R && row0 + threadIdx.x < N) {
    float s = 0.f;
    for (int w = 0; w < nwaves; ++w) s += part[w][threadIdx.x];
    y[row0 + threadIdx.x] = s;
  }
}

__global__ void __launch_bounds__(256) gemv_f32_scalar_kernel(const float* __restrict__ x, const float* __restrict__ W,
                                                              float* __restrict__ y, int64_t N, int64_t K) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= N) return;  // whole wavefronts leave together; no workgroup barrier below
  const float* w = W + row * K;
  float acc = 0.f;
  for (int64_t k = threadIdx.x & 63; k < K; k += 64) acc = fmaf(x[k], w[k], acc);
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) y[row] = acc;
}

// Any K and any alignment: one wavefront per row, element accesses.
__global__ void __launch_bounds__(256) gemv_scalar_kernel(const half_t* __restrict__ x, const half_t* __restrict__ W,
                                                          GemvEpilogue ep, void* __restrict__ y, int64_t N, int64_t K) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= N) return;  // whole wavefronts leave together; no workgroup barrier below
  const half_t* w = W + row * K;
  float acc = 0.f;
  for (int64_t k = threadIdx.x & 63; k < K; k += 64) acc += static_cast<float>(x[k]) * static_cast<float>(w[k]);
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) finish(acc, ep, y, row);
}

}  // namespace

// launch_args: {grid, 1, 1, block, static LDS bytes, rows per workgroup, 0}
int describe_gemv(int64_t N, int64_t K, const dtas_config& cfg, int64_t la[7]) {
  (void)K;
  for (int i = 0; i < 7; ++i) la[i] = 0;
  la[1] = la[2] = 1;
  if (cfg.variant == DTAS_GEMV_RF16) {  // half a wavefront per row, 8 rows per workgroup
    if (cfg.block != 256) return fail("gemv: the fp16-accumulate kernel uses 256 threads, got %d", cfg.block);
    if (cfg.vec != 8 && cfg.vec != 1) return fail("gemv: vector width must be 8 (128 bit) or 1, got %d", cfg.vec);
    la[0] = ceil_div(N, 8);
    la[3] = 256;
    la[5] = 8;
    if (la[0] > 0x7fffffff) return fail("gemv: N=%lld needs too many workgroups", (long long)N);
    return 0;
  }
  if (cfg.variant != DTAS_GEMV_SPLITK) return fail("gemv: unknown variant %d", cfg.variant);
  if (cfg.block < 64 || cfg.block > 512 || cfg.block % 64 != 0)
    return fail("gemv: block must be a multiple of 64 in [64, 512], got %d", cfg.block);
  const int rows = cfg.tile[0];
  if (cfg.vec == 1) {  // element-access fallback: one wavefront per row
    la[0] = ceil_div(N, 4);
    la[3] = 256;
    la[5] = 4;
    return 0;
  }
  if (cfg.vec != 8) return fail("gemv: vector width must be 8 (128 bit) or 1, got %d", cfg.vec);
  if (rows != 1 && rows != 2 && rows != 4 && rows != 8) return fail("gemv: rows per workgroup %d not in {1, 2, 4, 8}", rows);
  la[0] = ceil_div(N, rows);
  la[3] = cfg.block;
  la[4] = 8 * rows * 4;
  la[5] = rows;
  if (la[0] > 0x7fffffff) return fail("gemv: N=%lld needs too many workgroups", (long long)N);
  return 0;
}

}  // namespace dtas

extern "C" int dtas_gemv_f16_fused(const void* x, const void* W, const void* bias, const void* res1, const void* res2,
                                   void* y, int64_t N, int64_t K, int32_t epilogue, const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (epilogue < DTAS_EPI_BIAS || epilogue > DTAS_EPI_BIAS_GELU) return fail("gemv: unknown epilogue %d", epilogue);
  const bool add2 = epilogue == DTAS_EPI_BIAS_ADD2 || epilogue == DTAS_EPI_BIAS_ADD2_CAST_F32;
  const int out_bytes = epilogue == DTAS_EPI_BIAS_ADD2_CAST_F32 ? 4 : 2;
  if (N < 0 || K < 0) return fail("gemv: negative extent N=%lld K=%lld", (long long)N, (long long)K);
  if (N == 0) return 0;
  if (K != 0 && N > INT64_MAX / 4 / K) return fail("gemv: N*K overflows");
  if (!y || (K > 0 && (!x || !W))) return fail("gemv: NULL buffer");
  if (add2 && (!res1 || !res2)) return fail("gemv: the add-add epilogue needs both residual buffers");
  if (!add2 && (res1 || res2)) return fail("gemv: residual buffers given for an epilogue that takes none");
  if (overlaps(y, N * out_bytes, W, N * K * 2) || overlaps(y, N * out_bytes, x, K * 2) ||
      (add2 && (overlaps(y, N * out_bytes, res1, N * 2) || overlaps(y, N * out_bytes, res2, N * 2))))
    return fail("gemv: output overlaps an input");
  dtas_config cfg = user ? *user : builtin_config(DTAS_OP_GEMV_F16, 1, N, K).cfg;
  const bool vec_ok = K % 8 == 0 && aligned(x, 16) && aligned(W, 16);
  if (cfg.vec == 8 && !vec_ok) cfg.vec = 1;  // K % 8 != 0 or odd pointers: element accesses
  int64_t la[7];
  if (describe_gemv(N, K, cfg, la) != 0) return -1;
  const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* xp = static_cast<const half_t*>(x);
  const half_t* wp = static_cast<const half_t*>(W);
  const GemvEpilogue ep = {static_cast<const half_t*>(bias), static_cast<const half_t*>(res1),
                           static_cast<const half_t*>(res2), epilogue};
  if (cfg.variant == DTAS_GEMV_RF16) {
    if (cfg.vec == 8) hipLaunchKernelGGL(gemv_rf16_kernel<true>, grid, block, 0, s, xp, wp, ep, y, N, K);
    else hipLaunchKernelGGL(gemv_rf16_kernel<false>, grid, block, 0, s, xp, wp, ep, y, N, K);
    return check_launch("gemv");
  }
  if (cfg.vec == 1) {
    hipLaunchKernelGGL(gemv_scalar_kernel, grid, block, 0, s, xp, wp, ep, y, N, K);
    return check_launch("gemv");
  }
  switch (cfg.tile[0]) {
    case 1: hipLaunchKernelGGL(gemv_splitk_kernel<1>, grid, block, 0, s, xp, wp, ep, y, N, K); break;
    case 2: hipLaunchKernelGGL(gemv_splitk_kernel<2>, grid, block, 0, s, xp, wp, ep, y, N, K); break;
    case 4: hipLaunchKernelGGL(gemv_splitk_kernel<4>, grid, block, 0, s, xp, wp, ep, y, N, K); break;
    case 8: hipLaunchKernelGGL(gemv_splitk_kernel<8>, grid, block, 0, s, xp, wp, ep, y, N, K); break;
  }
  return check_launch("gemv");
}

extern "C" int dtas_gemv_f16(const void* x, const void* W, const void* bias, void* y, int64_t N, int64_t K,
                             const dtas_config* user, void* stream) {
  return dtas_gemv_f16_fused(x, W, bias, nullptr, nullptr, y, N, K, DTAS_EPI_BIAS, user, stream);
}

extern "C" int dtas_gemv_f32(const void* x, const void* W, void* y, int64_t N, int64_t K, const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (N < 0 || K < 0) return fail("gemv_f32: negative extent N=%lld K=%lld", (long long)N, (long long)K);
  if (N == 0) return 0;
  if (K != 0 && N > INT64_MAX / 8 / K) return fail("gemv_f32: N*K overflows");
  if (!y || (K > 0 && (!x || !W))) return fail("gemv_f32: NULL buffer");
  if (overlaps(y, N * 4, W, N * K * 4) || overlaps(y, N * 4, x, K * 4)) return fail("gemv_f32: output overlaps an input");
  // the fp16 table, read for a weight matrix of the same bytes (2K fp16 columns)
  dtas_config cfg = user ? *user : builtin_config(DTAS_OP_GEMV_F16, 1, N, 2 * K).cfg;
  if (cfg.vec == 8) cfg.vec = 4;  // (a row of the fp16 table says 8 elements per access: 128 bits are 4 floats)
  const bool vec_ok = K % 4 == 0 && aligned(x, 16) && aligned(W, 16);
  if (cfg.vec == 4 && !vec_ok) cfg.vec = 1;
  if (cfg.vec != 4 && cfg.vec != 1) return fail("gemv_f32: vector width must be 4 (128 bit) or 1, got %d", cfg.vec);
  dtas_config shape = cfg;
  shape.vec = cfg.vec == 4 ? 8 : 1;  // describe_gemv speaks of 128-bit accesses as vec 8
  int64_t la[7];
  if (describe_gemv(N, K, shape, la) != 0) return -1;
  const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float* xp = static_cast<const float*>(x);
  const float* wp = static_cast<const float*>(W);
  float* yp = static_cast<float*>(y);
  if (cfg.vec == 1) {
    hipLaunchKernelGGL(gemv_f32_scalar_kernel, grid, block, 0, s, xp, wp, yp, N, K);
    return check_launch("gemv_f32");
  }
  switch (cfg.tile[0]) {
    case 1: hipLaunchKernelGGL(gemv_f32_kernel<1>, grid, block, 0, s, xp, wp, yp, N, K); break;
    case 2: hipLaunchKernelGGL(gemv_f32_kernel<2>, grid, block, 0, s, xp, wp, yp, N, K); break;
    case 4: hipLaunchKernelGGL(gemv_f32_kernel<4>, grid, block, 0, s, xp, wp, yp, N, K); break;
    case 8: hipLaunchKernelGGL(gemv_f32_kernel<8>, grid, block, 0, s, xp, wp, yp, N, K); break;
  }
  return check_launch("gemv_f32");
}

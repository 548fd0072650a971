// 8-bit weights with group scales (the q8f16_1 layout) for gfx950: the standalone dequantiser, the
// dequantising row gather of the embedding, and the decode GEMVs that dequantise in registers (fp16 with
// fp16 scales; fp32 with fp32 scales for the vocabulary projection).
//
// Layout and arithmetic, as the PrimFuncs spell them
// (experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py:335-343 fused_decode3, :401-426
// fused_fused_decode2_fused_NT_matmul_add, :428-502 fused_fused_decode4_fused_NT_matmul3_add2_gelu):
//   Wq[N, K/4] uint32: element j of a row is byte j % 4 of word j / 4;  S[N, K/32] fp16: one scale per 32
//   W[i, j] = (fp16(byte) - fp16(127)) * S[i, j / 32]           -- fp16 arithmetic, one rounding (the product)
//   y[i]    = sum_k x[k] * W[i, k]  (+ bias[i], then GELU)      -- fp32 accumulation here, fp16 after
//
// byte -> fp16 without a conversion: 0x6400 is 1024.0 and fp16 counts in ones from 1024 to 2047, so
// 0x6400 | byte is 1024 + byte exactly; one byte permute builds two such halves from a weight word,
// one packed subtract of 1151 leaves byte - 127 (exact), one packed multiply by the scale rounds as
// the PrimFunc's fp16 product does, one dot2 accumulates against x in fp32: 4 VALU instructions per
// two weights, so the kernel stays bound by the weight stream (one byte per weight).
#include "dtas_device.h"
#include "dtas_host.h"

namespace dtas {
namespace {

// One item = 8 weights: 8 bytes in, 16 bytes out, so that a wavefront's loads and stores are each one
// contiguous span (512 bytes in, 1 KiB out).  A thread requests four items, a grid stride apart, before
// it uses the first.  K % 32 == 0, so an item's weights share a scale and the flat scale index is (8 i) / 32.
// STREAM: non-temporal stores (the output is larger than the Infinity Cache); otherwise plain stores, so that
// the GEMM that reads the matrix next finds it in the cache.
template <bool STREAM>
__global__ void __launch_bounds__(256) decode_q8_kernel(const u32x2* __restrict__ Wq, const half_t* __restrict__ S,
                                                        u32x4* __restrict__ W, int64_t items) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i0 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i0 < items; i0 += 4 * stride) {
    u32x2 q[4];
    half_t s[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = i0 + u * stride;
      if (i < items) {
        q[u] = load_stream(Wq + i);
        s[u] = S[i >> 2];
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = i0 + u * stride;
      if (i >= items) break;
      const f16x2 s2 = {s[u], s[u]};
      f16x2 a, b, c, d;
      const unsigned w0 = q[u][0], w1 = q[u][1];
      dequant_q8_word(w0, s2, a, b);
      dequant_q8_word(w1, s2, c, d);
      const u32x4 out = {__builtin_bit_cast(unsigned, a), __builtin_bit_cast(unsigned, b), __builtin_bit_cast(unsigned, c),
                         __builtin_bit_cast(unsigned, d)};
      if (STREAM) store_stream(out, W + i);
      else W[i] = out;
    }
  }
}

// any alignment: one thread per weight
__global__ void __launch_bounds__(256) decode_q8_scalar_kernel(const unsigned char* __restrict__ Wq,
                                                               const half_t* __restrict__ S, half_t* __restrict__ W,
                                                               int64_t total) {
  for (int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; j < total;
       j += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const half_t q = static_cast<half_t>(static_cast<float>(Wq[j])) - static_cast<half_t>(127.f);  // little endian: byte j
    W[j] = q * S[j >> 5];
  }
}

// The embedding rows, dequantised: out[i, :] = decode(Wq, S)[ids[i], :].  Items of 8 weights as above; item t of
// the output is item ids[t / per_row] * per_row + t % per_row of the table.  Ids outside [0, V) are clipped
// to the nearest row (the PrimFunc reads whatever address they make).
__global__ void __launch_bounds__(256) take_q8_kernel(const u32x2* __restrict__ Wq, const half_t* __restrict__ S,
                                                      const int* __restrict__ ids, u32x4* __restrict__ out, int64_t items,
                                                      int64_t per_row, int64_t V) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < items; t += stride) {
    int64_t row = ids[t / per_row];
    row = row < 0 ? 0 : row >= V ? V - 1 : row;
    const int64_t src = row * per_row + t % per_row;
    const u32x2 q = Wq[src];
    const half_t s = S[src >> 2];
    const f16x2 s2 = {s, s};
    f16x2 a, b, c, d;
    const unsigned w0 = q[0], w1 = q[1];
    dequant_q8_word(w0, s2, a, b);
    dequant_q8_word(w1, s2, c, d);
    const u32x4 v = {__builtin_bit_cast(unsigned, a), __builtin_bit_cast(unsigned, b), __builtin_bit_cast(unsigned, c),
                     __builtin_bit_cast(unsigned, d)};
    out[t] = v;
  }
}

// any alignment: one thread per weight
__global__ void __launch_bounds__(256) take_q8_scalar_kernel(const unsigned char* __restrict__ Wq, const half_t* __restrict__ S,
                                                             const int* __restrict__ ids, half_t* __restrict__ out,
                                                             int64_t total, int64_t K, int64_t V) {
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < total;
       t += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    int64_t row = ids[t / K];
    row = row < 0 ? 0 : row >= V ? V - 1 : row;
    const int64_t j = row * K + t % K;
    const half_t q = static_cast<half_t>(static_cast<float>(Wq[j])) - static_cast<half_t>(127.f);
    out[t] = q * S[j >> 5];
  }
}

// fp32 scales, fp32 x and y (fused_fused_decode6_NT_matmul5, before_dl.py:640-657: the vocabulary projection
// of the 8-bit model): W = float(byte - 127) * S32, one fp32 rounding, then fp32 multiply-adds against x.
// Workgroup shape and weight stream as gemv_q8_kernel; a 16-byte chunk of weights meets 64 bytes of x.  The weights
// of a chunk share a scale, so a chunk's sum of x * (byte - 127) -- exact factors -- is formed first and scaled once:
// three VALU instructions per weight instead of four, in a kernel that has as many VALU cycles as memory cycles
// (50280 x 2560: 28.7 -> 26.1 us).  Holding x in registers, a wavefront per set of rows, is no faster than 8 rows per
// workgroup here (24.4 us either way).
template <int R>
__global__ void __launch_bounds__(512) gemv_q8_f32_kernel(const float* __restrict__ x, const unsigned* __restrict__ Wq,
                                                          const float* __restrict__ S, float* __restrict__ y, int64_t N,
                                                          int64_t K) {
  __shared__ float part[8][R];
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
  const int64_t nchunk = K >> 4, ngroup = K >> 5;
  const f32x4* xv = reinterpret_cast<const f32x4*>(x);
  const u32x4* wv[R];
  const float* sv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + r < N ? row0 + r : N - 1;  // rows past N re-read the last row; never stored
    wv[r] = reinterpret_cast<const u32x4*>(Wq + row * (K >> 2));
    sv[r] = S + row * ngroup;
  }
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;

#pragma unroll 2
  for (int64_t i = threadIdx.x; i < nchunk; i += blockDim.x) {
    f32x4 xr[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) xr[w] = xv[4 * i + w];
    u32x4 q[R];
    float s[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      q[r] = load_stream(wv[r] + i);
      s[r] = sv[r][i >> 1];
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float p = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const unsigned word = q[r][w];
#pragma unroll
        for (int e = 0; e < 4; ++e) p = fmaf(xr[w][e], static_cast<float>((word >> (8 * e)) & 255u) - 127.f, p);
      }
      acc[r] = fmaf(p, s[r], acc[r]);
    }
  }

  const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float sum = wave_sum(acc[r]);
    if ((threadIdx.x & 63) == 0) part[wave][r] = sum;
  }
  __syncthreads();
  if (threadIdx.x < R && row0 + threadIdx.x < N) {
    float sum = 0.f;
    for (int w = 0; w < nwaves; ++w) sum += part[w][threadIdx.x];
    y[row0 + threadIdx.x] = sum;
  }
}

// any alignment: one wavefront per row, byte accesses
__global__ void __launch_bounds__(256) gemv_q8_f32_scalar_kernel(const float* __restrict__ x, const unsigned char* __restrict__ Wq,
                                                                 const float* __restrict__ S, float* __restrict__ y, int64_t N,
                                                                 int64_t K) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= N) return;  // whole wavefronts leave together; no workgroup barrier below
  float acc = 0.f;
  for (int64_t k = threadIdx.x & 63; k < K; k += 64) {
    const float wt = (static_cast<float>(Wq[row * K + k]) - 127.f) * S[row * (K >> 5) + (k >> 5)];
    acc = fmaf(x[k], wt, acc);
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) y[row] = acc;
}

__device__ __forceinline__ half_t finish_q8(float acc, const half_t* bias, int64_t j, int kind) {
  half_t t = static_cast<half_t>(acc);
  if (bias) t = static_cast<half_t>(static_cast<float>(t) + static_cast<float>(bias[j]));
  if (kind == DTAS_EPI_BIAS_GELU) t = gelu_erf_f16_steps(t);
  return t;
}
// the same with the bias element already in a register (requested before W is streamed: read at the end it costs the
// launch a round trip to memory of its own)
__device__ __forceinline__ half_t finish_q8_with(float acc, bool has_bias, half_t bias_j, int kind) {
  half_t t = static_cast<half_t>(acc);
  if (has_bias) t = static_cast<half_t>(static_cast<float>(t) + static_cast<float>(bias_j));
  if (kind == DTAS_EPI_BIAS_GELU) t = gelu_erf_f16_steps(t);
  return t;
}

// Workgroup = R rows of Wq; lane t takes the 16-byte chunks t, t + block, ... (16 weights, 32 bytes
// of x) of every row, so a wavefront reads 1 KiB of a row at a time, non-temporal.
template <int R>
__global__ void __launch_bounds__(512) gemv_q8_kernel(const half_t* __restrict__ x, const unsigned* __restrict__ Wq,
                                                      const half_t* __restrict__ S, const half_t* __restrict__ bias,
                                                      half_t* __restrict__ y, int64_t N, int64_t K, int kind) {
  __shared__ float part[8][R];
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
  const int64_t nchunk = K >> 4, ngroup = K >> 5;
  const u32x4* xv = reinterpret_cast<const u32x4*>(x);
  const u32x4* wv[R];
  const half_t* sv[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + r < N ? row0 + r : N - 1;  // rows past N re-read the last row; never stored
    wv[r] = reinterpret_cast<const u32x4*>(Wq + row * (K >> 2));
    sv[r] = S + row * ngroup;
  }
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  // thread r < R stores row row0 + r: its bias element, requested now and kept as loaded
  const half_t e_bias = bias && threadIdx.x < R && row0 + threadIdx.x < N ? bias[row0 + threadIdx.x] : static_cast<half_t>(0.f);

#pragma unroll 2
  for (int64_t i = threadIdx.x; i < nchunk; i += blockDim.x) {
    const u32x4 x0 = xv[2 * i], x1 = xv[2 * i + 1];
    u32x4 q[R];
    half_t s[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      q[r] = load_stream(wv[r] + i);
      s[r] = sv[r][i >> 1];
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const f16x2 s2 = {s[r], s[r]};
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        f16x2 lo, hi;
        const unsigned word = q[r][w];
        dequant_q8_word(word, s2, lo, hi);
        const unsigned xa = w < 2 ? x0[2 * w] : x1[2 * w - 4], xb = w < 2 ? x0[2 * w + 1] : x1[2 * w - 3];
        acc[r] = __builtin_amdgcn_fdot2(lo, __builtin_bit_cast(f16x2, xa), acc[r], false);
        acc[r] = __builtin_amdgcn_fdot2(hi, __builtin_bit_cast(f16x2, xb), acc[r], false);
      }
    }
  }

  asm volatile("" ::"v"(e_bias));  // (it exists by now: its load stays where it was written)
  const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float sum = wave_sum(acc[r]);
    if ((threadIdx.x & 63) == 0) part[wave][r] = sum;
  }
  __syncthreads();
  if (threadIdx.x < R && row0 + threadIdx.x < N) {
    float sum = 0.f;
    for (int w = 0; w < nwaves; ++w) sum += part[w][threadIdx.x];
    y[row0 + threadIdx.x] = finish_q8_with(sum, bias != nullptr, e_bias, kind);
  }
}

// any alignment: one wavefront per row, byte accesses
__global__ void __launch_bounds__(256) gemv_q8_scalar_kernel(const half_t* __restrict__ x, const unsigned char* __restrict__ Wq,
                                                             const half_t* __restrict__ S, const half_t* __restrict__ bias,
                                                             half_t* __restrict__ y, int64_t N, int64_t K, int kind) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= N) return;  // whole wavefronts leave together; no workgroup barrier below
  float acc = 0.f;
  for (int64_t k = threadIdx.x & 63; k < K; k += 64) {
    const half_t q = static_cast<half_t>(static_cast<float>(Wq[row * K + k])) - static_cast<half_t>(127.f);
    const half_t w = q * S[row * (K >> 5) + (k >> 5)];
    acc += static_cast<float>(x[k]) * static_cast<float>(w);
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) y[row] = finish_q8(acc, bias, row, kind);
}

int check_q8_shape(const char* what, int64_t N, int64_t K) {
  if (N < 0 || K < 0) return fail("%s: negative extent N=%lld K=%lld", what, (long long)N, (long long)K);
  if (K % 32 != 0) return fail("%s: K must be a multiple of the scale group, 32 (K=%lld)", what, (long long)K);
  if (K != 0 && N > INT64_MAX / 4 / K) return fail("%s: N*K overflows", what);
  return 0;
}

}  // namespace
}  // namespace dtas

extern "C" int dtas_decode_q8_f16(const void* Wq, const void* scale, void* W, int64_t N, int64_t K, const dtas_config* user,
                                  void* stream) {
  using namespace dtas;
  clear_error();
  if (check_q8_shape("decode_q8", N, K) != 0) return -1;
  if (N == 0 || K == 0) return 0;
  if (!Wq || !scale || !W) return fail("decode_q8: NULL buffer");
  if (overlaps(W, N * K * 2, Wq, N * K) || overlaps(W, N * K * 2, scale, N * (K / 32) * 2))
    return fail("decode_q8: output overlaps an input");
  dtas_config cfg = user ? *user : dtas_config{DTAS_ELT_VECTOR, 256, 8, 1, {0, 0, 0}, 1, 0};
  if (cfg.block != 256) return fail("decode_q8: the kernels use 256 threads, got %d", cfg.block);
  if (cfg.vec != 8 && cfg.vec != 1) return fail("decode_q8: vector width must be 8 (128-bit stores) or 1, got %d", cfg.vec);
  if (cfg.vec == 8 && !(aligned(Wq, 8) && aligned(W, 16))) cfg.vec = 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t items = cfg.vec == 8 ? N * K / 8 : N * K;
  int64_t grid = ceil_div(items, cfg.vec == 8 ? 4 * 256 : 256);
  const int64_t cap = cfg.grid_cap > 0 ? cfg.grid_cap : int64_t{kNumCU} * 64;
  grid = grid > cap ? cap : grid;
  const bool stream_out = N * K * 2 > (int64_t{128} << 20);  // half of the 256 MiB Infinity Cache
  if (cfg.vec == 8 && stream_out)
    hipLaunchKernelGGL(decode_q8_kernel<true>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, s, static_cast<const u32x2*>(Wq),
                       static_cast<const half_t*>(scale), static_cast<u32x4*>(W), items);
  else if (cfg.vec == 8)
    hipLaunchKernelGGL(decode_q8_kernel<false>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, s, static_cast<const u32x2*>(Wq),
                       static_cast<const half_t*>(scale), static_cast<u32x4*>(W), items);
  else
    hipLaunchKernelGGL(decode_q8_scalar_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, s,
                       static_cast<const unsigned char*>(Wq), static_cast<const half_t*>(scale), static_cast<half_t*>(W), items);
  return check_launch("decode_q8");
}

extern "C" int dtas_gemv_q8_f16(const void* x, const void* Wq, const void* scale, const void* bias, void* y, int64_t N,
                                int64_t K, int32_t epilogue, const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (check_q8_shape("gemv_q8", N, K) != 0) return -1;
  if (epilogue != DTAS_EPI_BIAS && epilogue != DTAS_EPI_BIAS_GELU)
    return fail("gemv_q8: epilogue must be DTAS_EPI_BIAS or DTAS_EPI_BIAS_GELU, got %d", epilogue);
  if (N == 0) return 0;
  if (!y || (K > 0 && (!x || !Wq || !scale))) return fail("gemv_q8: NULL buffer");
  if (overlaps(y, N * 2, Wq, N * K) || overlaps(y, N * 2, x, K * 2) || overlaps(y, N * 2, scale, N * (K / 32) * 2))
    return fail("gemv_q8: output overlaps an input");
  // measured over N = 2560 .. 50280 against K = 2560 .. 11008 (12 launch shapes each): 4 rows per workgroup from 4096 rows
  // on, 2 below; 8 wavefronts for K >= 8192 with those 4 rows, 4 wavefronts otherwise (7680 x 10240: 15.4 us against 17.7 for 2 rows on 4 wavefronts,
  // 11008 x 5120: 11.8 / 13.9, 4096 x 5120: 6.4 / 7.4; level at K = 4096)
  // short rows (K <= 2048) from 12288 rows on: 2 wavefronts, and 8 rows per workgroup when K <= 1024 and N >= 16384 (28672 x 1024:
  // 8.1 us against 10.0; 13824 x 1024: 5.4 / 6.3 with 4 rows; 28672 x 2048: 11.8 / 13.0)
  // (one wavefront on 4 rows up to K = 1024: 50280 x 768 11.0 -> 9.3 us, x 512 10.2 -> 8.8)
  const int q8_block = K >= 8192 && N >= 4096 ? 512 : K <= 1024 && N >= 12288 ? 64 : K <= 2048 && N >= 12288 ? 128 : 256;
  const int q8_rows = N >= 4096 ? 4 : 2;
  dtas_config cfg = user ? *user : dtas_config{DTAS_GEMV_SPLITK, q8_block, 8, 2, {q8_rows, 0, 0}, 1, 0};
  if (cfg.vec == 8 && !(aligned(x, 16) && aligned(Wq, 16))) cfg.vec = 1;
  int64_t la[7];
  if (describe_gemv(N, K, cfg, la) != 0) return -1;
  const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* xp = static_cast<const half_t*>(x);
  const half_t* sp = static_cast<const half_t*>(scale);
  const half_t* bp = static_cast<const half_t*>(bias);
  half_t* yp = static_cast<half_t*>(y);
  if (cfg.vec == 1) {
    hipLaunchKernelGGL(gemv_q8_scalar_kernel, grid, block, 0, s, xp, static_cast<const unsigned char*>(Wq), sp, bp, yp, N, K, epilogue);
    return check_launch("gemv_q8");
  }
  const unsigned* wp = static_cast<const unsigned*>(Wq);
  switch (cfg.tile[0]) {
    case 1: hipLaunchKernelGGL(gemv_q8_kernel<1>, grid, block, 0, s, xp, wp, sp, bp, yp, N, K, epilogue); break;
    case 2: hipLaunchKernelGGL(gemv_q8_kernel<2>, grid, block, 0, s, xp, wp, sp, bp, yp, N, K, epilogue); break;
    case 4: hipLaunchKernelGGL(gemv_q8_kernel<4>, grid, block, 0, s, xp, wp, sp, bp, yp, N, K, epilogue); break;
    case 8: hipLaunchKernelGGL(gemv_q8_kernel<8>, grid, block, 0, s, xp, wp, sp, bp, yp, N, K, epilogue); break;
  }
  return check_launch("gemv_q8");
}

extern "C" int dtas_take_q8_f16(const void* Wq, const void* scale, const void* ids, void* out, int64_t n, int64_t V, int64_t K,
                                const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (check_q8_shape("take_q8", V, K) != 0) return -1;
  if (n < 0) return fail("take_q8: negative extent n=%lld", (long long)n);
  if (K != 0 && n > INT64_MAX / 4 / K) return fail("take_q8: n*K overflows");
  if (n == 0 || K == 0) return 0;
  if (V == 0) return fail("take_q8: an empty table has no row to take");
  if (!Wq || !scale || !ids || !out) return fail("take_q8: NULL buffer");
  if (overlaps(out, n * K * 2, Wq, V * K) || overlaps(out, n * K * 2, scale, V * (K / 32) * 2) || overlaps(out, n * K * 2, ids, n * 4))
    return fail("take_q8: output overlaps an input");
  dtas_config cfg = user ? *user : dtas_config{DTAS_ELT_VECTOR, 256, 8, 1, {0, 0, 0}, 1, 0};
  if (cfg.block != 256) return fail("take_q8: the kernels use 256 threads, got %d", cfg.block);
  if (cfg.vec != 8 && cfg.vec != 1) return fail("take_q8: vector width must be 8 (128-bit stores) or 1, got %d", cfg.vec);
  if (cfg.vec == 8 && !(aligned(Wq, 8) && aligned(out, 16))) cfg.vec = 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t items = cfg.vec == 8 ? n * K / 8 : n * K;
  int64_t grid = ceil_div(items, 256);
  const int64_t cap = cfg.grid_cap > 0 ? cfg.grid_cap : int64_t{1} << 23;   // (a thread per item while a launch may hold them: a capped grid that loops is slower)
  grid = grid > cap ? cap : grid;
  if (cfg.vec == 8)
    hipLaunchKernelGGL(take_q8_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, s, static_cast<const u32x2*>(Wq),
                       static_cast<const half_t*>(scale), static_cast<const int*>(ids), static_cast<u32x4*>(out), items, K / 8, V);
  else
    hipLaunchKernelGGL(take_q8_scalar_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, s,
                       static_cast<const unsigned char*>(Wq), static_cast<const half_t*>(scale), static_cast<const int*>(ids),
                       static_cast<half_t*>(out), items, K, V);
  return check_launch("take_q8");
}

extern "C" int dtas_gemv_q8_f32(const void* x, const void* Wq, const void* scale, void* y, int64_t N, int64_t K,
                                const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (check_q8_shape("gemv_q8_f32", N, K) != 0) return -1;
  if (N == 0) return 0;
  if (!y || (K > 0 && (!x || !Wq || !scale))) return fail("gemv_q8_f32: NULL buffer");
  if (overlaps(y, N * 4, Wq, N * K) || overlaps(y, N * 4, x, K * 4) || overlaps(y, N * 4, scale, N * (K / 32) * 4))
    return fail("gemv_q8_f32: output overlaps an input");
  // (50280 x 2560: 45 / 30 / 25 / 24 us with 1 / 2 / 4 / 8 rows per workgroup; short rows leave most of 4 wavefronts idle:
  // one wavefront on 4 rows up to K = 1024 -- 50257 x 768 16.0 -> 9.7 us, 128256 x 1024 35.3 -> 23.6 -- two up to 2048)
  dtas_config cfg = user ? *user
                    : K <= 1024 ? dtas_config{DTAS_GEMV_SPLITK, 64, 8, 2, {4, 0, 0}, 1, 0}
                    : K <= 2048 ? dtas_config{DTAS_GEMV_SPLITK, 128, 8, 2, {4, 0, 0}, 1, 0}
                                : dtas_config{DTAS_GEMV_SPLITK, 256, 8, 2, {N >= 16384 ? 8 : 2, 0, 0}, 1, 0};
  if (cfg.vec == 8 && !(aligned(x, 16) && aligned(Wq, 16))) cfg.vec = 1;
  int64_t la[7];
  if (describe_gemv(N, K, cfg, la) != 0) return -1;
  const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float* xp = static_cast<const float*>(x);
  const float* sp = static_cast<const float*>(scale);
  float* yp = static_cast<float*>(y);
  if (cfg.vec == 1) {
    hipLaunchKernelGGL(gemv_q8_f32_scalar_kernel, grid, block, 0, s, xp, static_cast<const unsigned char*>(Wq), sp, yp, N, K);
    return check_launch("gemv_q8_f32");
  }
  const unsigned* wp = static_cast<const unsigned*>(Wq);
  switch (cfg.tile[0]) {
    case 1: hipLaunchKernelGGL(gemv_q8_f32_kernel<1>, grid, block, 0, s, xp, wp, sp, yp, N, K); break;
    case 2: hipLaunchKernelGGL(gemv_q8_f32_kernel<2>, grid, block, 0, s, xp, wp, sp, yp, N, K); break;
    case 4: hipLaunchKernelGGL(gemv_q8_f32_kernel<4>, grid, block, 0, s, xp, wp, sp, yp, N, K); break;
    case 8: hipLaunchKernelGGL(gemv_q8_f32_kernel<8>, grid, block, 0, s, xp, wp, sp, yp, N, K); break;
  }
  return check_launch("gemv_q8_f32");
}

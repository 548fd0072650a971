// Row reductions for gfx950: RMSNorm, LayerNorm(+cast), softmax(+cast).
//
// Replaces the kernels DTAS's general-reduction rule generates
// (python/dtas/schedule/tir_reduction.py:36-105: one block per row, len_tx threads stride the
// row, partial results staged in shared memory; generated form
// experiment/dtas_tuned/general_reduction/layernorm/top1_256/tvm_device_kernels.cu:75-253 and
// .../softmax/row_12800/top10_256_10_nounroll/tvm_device_kernels.cu, which re-reads each row
// three times).
//
// MI355X shape: a row is read from HBM exactly once, as 128-bit accesses, and stays in
// registers for the statistics and the output pass.
//   WAVE_ROW  : one wavefront per row (block/64 rows per workgroup); 64 lanes x ITERS
//               vectors cover the row; reduction entirely on the DPP datapath.
//   BLOCK_ROW : one workgroup per row for few, long rows; DPP inside each wavefront,
//               one LDS slot per wavefront across them.
//   STREAM_ROW: any row length and alignment; element accesses, the row is re-read per
//               pass (from L2), statistics as in BLOCK_ROW.
#include "dtas_device.h"
#include "dtas_host.h"

namespace dtas {
namespace {

enum { kRms = 0, kLayerNorm = 1, kSoftmaxF32 = 2, kSoftmaxF16 = 3 };

constexpr float kNegMax = -3.4028234663852886e+38f;  // the PrimFunc's max init, not -inf
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }

template <int OP>
struct RowTraits;
template <>
struct RowTraits<kRms> {
  typedef half_t In;
  static constexpr int kVec = 8;
};
template <>
struct RowTraits<kLayerNorm> {
  typedef float In;
  static constexpr int kVec = 4;
};
template <>
struct RowTraits<kSoftmaxF32> {
  typedef float In;
  static constexpr int kVec = 4;
};
template <>
struct RowTraits<kSoftmaxF16> {
  typedef half_t In;
  static constexpr int kVec = 8;
};

// 16 bytes of a row, viewed as kVec floats
template <typename In, int VEC>
struct RowVec {
  u32x4 raw;
  __device__ __forceinline__ float get(int e) const {
    if (sizeof(In) == 2) {
      f16x8 h = __builtin_bit_cast(f16x8, raw);
      return static_cast<float>(h[e]);
    } else {
      f32x4 f = __builtin_bit_cast(f32x4, raw);
      return f[e];
    }
  }
};

// kVec fp16 results: 16 bytes for kVec = 8, 8 bytes for kVec = 4
template <int VEC>
__device__ __forceinline__ void store_half_vec(half_t* dst, const float (&v)[VEC]) {
  if (VEC == 8) {
    f16x8 h;
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = static_cast<half_t>(v[e]);
    store_stream(__builtin_bit_cast(u32x4, h), reinterpret_cast<u32x4*>(dst));
  } else {
    f16x4 h;
#pragma unroll
    for (int e = 0; e < 4; ++e) h[e] = static_cast<half_t>(v[e]);
    store_stream(__builtin_bit_cast(u32x2, h), reinterpret_cast<u32x2*>(dst));
  }
}

template <bool BLOCK, typename Op>
__device__ __forceinline__ float group_reduce(float v, float* slots) {
  return BLOCK ? block_reduce<Op>(v, slots) : Op::wave(v);
}

// ---- row held in registers ----------------------------------------------------------
// rows: number of rows; cols: row length, a multiple of kVec, every row 16-byte aligned.
template <int OP, int ITERS, bool BLOCK>
__global__ void __launch_bounds__(1024) row_reg_kernel(const void* __restrict__ xin, const void* __restrict__ p1,
                                                       const void* __restrict__ p2, void* __restrict__ outp,
                                                       int64_t rows, int64_t cols, float eps) {
  typedef typename RowTraits<OP>::In In;
  constexpr int VEC = RowTraits<OP>::kVec;
  typedef RowVec<In, VEC> V;
  __shared__ float slots[16];

  const int lane = BLOCK ? threadIdx.x : (threadIdx.x & 63);
  const int width = BLOCK ? blockDim.x : 64;
  const int64_t rows_per_wg = BLOCK ? 1 : (blockDim.x >> 6);
  const int64_t nvec = cols / VEC;
  const float inv_cols = 1.0f / static_cast<float>(cols);
  half_t* out = static_cast<half_t*>(outp);

  // every thread of a workgroup runs the same number of trips (BLOCK: same row;
  // WAVE: rows differ per wavefront but no workgroup barrier is used)
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * rows_per_wg + (BLOCK ? 0 : (threadIdx.x >> 6)); row < rows;
       row += static_cast<int64_t>(gridDim.x) * rows_per_wg) {
    const u32x4* src = reinterpret_cast<const u32x4*>(static_cast<const In*>(xin) + row * cols);
    V v[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int64_t i = lane + static_cast<int64_t>(it) * width;
      if (i < nvec) v[it].raw = load_stream(src + i);
    }

    if (OP == kRms) {
      float ss = 0.f;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (lane + static_cast<int64_t>(it) * width < nvec) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const float f = v[it].get(e);
            ss += f * f;
          }
        }
      }
      ss = group_reduce<BLOCK, SumOp>(ss, slots);
      const float rs = __builtin_amdgcn_rsqf(ss * inv_cols + eps);
      const u32x4* wv = static_cast<const u32x4*>(p1);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int64_t i = lane + static_cast<int64_t>(it) * width;
        if (i < nvec) {
          V w;
          w.raw = wv[i];
          float r[VEC];
#pragma unroll
          for (int e = 0; e < VEC; ++e) r[e] = v[it].get(e) * rs * w.get(e);
          store_half_vec<VEC>(out + row * cols + i * VEC, r);
        }
      }
    } else if (OP == kLayerNorm) {
      float s0 = 0.f, s1 = 0.f;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (lane + static_cast<int64_t>(it) * width < nvec) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const float f = v[it].get(e);
            s0 += f;
            s1 += f * f;
          }
        }
      }
      s0 = group_reduce<BLOCK, SumOp>(s0, slots);
      s1 = group_reduce<BLOCK, SumOp>(s1, slots);
      const float mean = s0 * inv_cols;
      const float rstd = __builtin_amdgcn_rsqf(s1 * inv_cols - mean * mean + eps);
      const u32x4* gv = static_cast<const u32x4*>(p1);
      const u32x4* bv = static_cast<const u32x4*>(p2);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int64_t i = lane + static_cast<int64_t>(it) * width;
        if (i < nvec) {
          V g, b;
          g.raw = gv[i];
          b.raw = bv[i];
          float r[VEC];
#pragma unroll
          for (int e = 0; e < VEC; ++e) r[e] = (v[it].get(e) - mean) * rstd * g.get(e) + b.get(e);
          store_half_vec<VEC>(out + row * cols + i * VEC, r);
        }
      }
    } else {  // softmax
      float mx = kNegMax;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (lane + static_cast<int64_t>(it) * width < nvec) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) mx = fmaxf(mx, v[it].get(e));
        }
      }
      mx = group_reduce<BLOCK, MaxOp>(mx, slots);
      float s = 0.f;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (lane + static_cast<int64_t>(it) * width < nvec) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) s += fast_exp(v[it].get(e) - mx);
        }
      }
      s = group_reduce<BLOCK, SumOp>(s, slots);
      const float inv = 1.0f / s;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int64_t i = lane + static_cast<int64_t>(it) * width;
        if (i < nvec) {
          float r[VEC];
#pragma unroll
          for (int e = 0; e < VEC; ++e) r[e] = fast_exp(v[it].get(e) - mx) * inv;
          store_half_vec<VEC>(out + row * cols + i * VEC, r);
        }
      }
    }
  }
}

// ---- any length, any alignment: element accesses, one workgroup per row ---------------
template <int OP>
__global__ void __launch_bounds__(1024) row_stream_kernel(const void* __restrict__ xin, const void* __restrict__ p1,
                                                          const void* __restrict__ p2, void* __restrict__ outp,
                                                          int64_t rows, int64_t cols, float eps) {
  typedef typename RowTraits<OP>::In In;
  __shared__ float slots[16];
  const float inv_cols = 1.0f / static_cast<float>(cols);
  half_t* out = static_cast<half_t*>(outp);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const In* x = static_cast<const In*>(xin) + row * cols;
    half_t* o = out + row * cols;
    if (OP == kRms) {
      float ss = 0.f;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) {
        const float f = static_cast<float>(x[k]);
        ss += f * f;
      }
      ss = block_reduce<SumOp>(ss, slots);
      const float rs = __builtin_amdgcn_rsqf(ss * inv_cols + eps);
      const half_t* w = static_cast<const half_t*>(p1);
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x)
        o[k] = static_cast<half_t>(static_cast<float>(x[k]) * rs * static_cast<float>(w[k]));
    } else if (OP == kLayerNorm) {
      float s0 = 0.f, s1 = 0.f;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) {
        const float f = static_cast<float>(x[k]);
        s0 += f;
        s1 += f * f;
      }
      s0 = block_reduce<SumOp>(s0, slots);
      s1 = block_reduce<SumOp>(s1, slots);
      const float mean = s0 * inv_cols;
      const float rstd = __builtin_amdgcn_rsqf(s1 * inv_cols - mean * mean + eps);
      const float* g = static_cast<const float*>(p1);
      const float* b = static_cast<const float*>(p2);
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x)
        o[k] = static_cast<half_t>((static_cast<float>(x[k]) - mean) * rstd * g[k] + b[k]);
    } else {
      float mx = kNegMax;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) mx = fmaxf(mx, static_cast<float>(x[k]));
      mx = block_reduce<MaxOp>(mx, slots);
      float s = 0.f;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) s += fast_exp(static_cast<float>(x[k]) - mx);
      s = block_reduce<SumOp>(s, slots);
      const float inv = 1.0f / s;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x)
        o[k] = static_cast<half_t>(fast_exp(static_cast<float>(x[k]) - mx) * inv);
    }
  }
}

template <int OP, bool BLOCK>
int launch_reg(int iters, dim3 grid, dim3 block, hipStream_t s, const void* x, const void* p1, const void* p2, void* out,
               int64_t rows, int64_t cols, float eps) {
#define DTAS_ROW_CASE(I)                                                                                         \
  case I:                                                                                                        \
    hipLaunchKernelGGL((row_reg_kernel<OP, I, BLOCK>), grid, block, 0, s, x, p1, p2, out, rows, cols, eps);      \
    break;
  switch (iters) {
    DTAS_ROW_CASE(1)
    DTAS_ROW_CASE(2)
    DTAS_ROW_CASE(4)
    DTAS_ROW_CASE(8)
    DTAS_ROW_CASE(16)
    default:
      return fail("reduction: %d vectors per lane is not one of 1, 2, 4, 8, 16", iters);
  }
#undef DTAS_ROW_CASE
  return check_launch("reduction");
}

struct RedInfo {
  int kind, in_bytes, vec;
  const char* name;
};

bool red_info(int op, RedInfo* r) {
  switch (op) {
    case DTAS_OP_RMS_NORM_F16: *r = {kRms, 2, 8, "rms_norm"}; return true;
    case DTAS_OP_LAYER_NORM_F32_F16: *r = {kLayerNorm, 4, 4, "fused_layer_norm_cast1"}; return true;
    case DTAS_OP_SOFTMAX_F32_F16: *r = {kSoftmaxF32, 4, 4, "fused_softmax_cast"}; return true;
    case DTAS_OP_SOFTMAX_F16: *r = {kSoftmaxF16, 2, 8, "fused_softmax_cast"}; return true;
  }
  return false;
}

int pow2_at_least(int64_t v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

template <int OP>
int launch_rows(const dtas_config& cfg, const int64_t la[7], hipStream_t s, const void* x, const void* p1,
                const void* p2, void* out, int64_t rows, int64_t cols, float eps) {
  const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
  if (cfg.variant == DTAS_RED_STREAM_ROW) {
    hipLaunchKernelGGL((row_stream_kernel<OP>), grid, block, 0, s, x, p1, p2, out, rows, cols, eps);
    return check_launch("reduction");
  }
  const int iters = static_cast<int>(la[5]);
  if (cfg.variant == DTAS_RED_WAVE_ROW) return launch_reg<OP, false>(iters, grid, block, s, x, p1, p2, out, rows, cols, eps);
  return launch_reg<OP, true>(iters, grid, block, s, x, p1, p2, out, rows, cols, eps);
}

int run_reduction(int op, const void* x, const void* p1, const void* p2, void* out, int64_t rows, int64_t cols,
                  float eps, const dtas_config* user, void* stream) {
  clear_error();
  RedInfo r;
  if (!red_info(op, &r)) return fail("reduction: unknown op %d", op);
  if (rows < 0 || cols < 0) return fail("%s: negative extent rows=%lld cols=%lld", r.name, (long long)rows, (long long)cols);
  if (rows == 0 || cols == 0) return 0;
  if (cols > INT64_MAX / 8 / rows) return fail("%s: rows*cols overflows", r.name);
  const bool needs_p1 = r.kind == kRms || r.kind == kLayerNorm, needs_p2 = r.kind == kLayerNorm;
  if (!x || !out || (needs_p1 && !p1) || (needs_p2 && !p2)) return fail("%s: NULL buffer", r.name);
  if (overlaps(x, rows * cols * r.in_bytes, out, rows * cols * 2))
    return fail("%s: output overlaps the input (PrimFunc is tir.noalias)", r.name);

  const bool vec_ok = cols % r.vec == 0 && aligned(x, 16) && aligned(out, r.vec * 2) &&
                      (!needs_p1 || aligned(p1, 16)) && (!needs_p2 || aligned(p2, 16));
  // dynamic extent: the row count for the norms, the row length for softmax
  const bool softmax = r.kind == kSoftmaxF32 || r.kind == kSoftmaxF16;
  dtas_config cfg = user ? *user : builtin_config(op, softmax ? cols : rows, softmax ? rows : cols, softmax ? cols : 0).cfg;
  // 128-bit row accesses need cols % vec == 0 and 16-byte aligned buffers; other rows take the
  // element-access kernel (a bucket's config must serve every n in the bucket)
  if (cfg.variant != DTAS_RED_STREAM_ROW && !vec_ok) {
    cfg.variant = DTAS_RED_STREAM_ROW;
    if (!user) cfg.block = cols >= 4096 ? 1024 : cols >= 1024 ? 512 : 256;
    cfg.vec = 1;
  }
  int64_t la[7];
  if (describe_reduction(op, rows, cols, cfg, la) != 0) return -1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (r.kind) {
    case kRms: return launch_rows<kRms>(cfg, la, s, x, p1, p2, out, rows, cols, eps);
    case kLayerNorm: return launch_rows<kLayerNorm>(cfg, la, s, x, p1, p2, out, rows, cols, eps);
    case kSoftmaxF32: return launch_rows<kSoftmaxF32>(cfg, la, s, x, p1, p2, out, rows, cols, eps);
    case kSoftmaxF16: return launch_rows<kSoftmaxF16>(cfg, la, s, x, p1, p2, out, rows, cols, eps);
  }
  return fail("reduction: unknown op %d", op);
}

}  // namespace

// launch_args: {grid, 1, 1, block, 0, vectors per lane (register variants), rows per workgroup}
int describe_reduction(int op, int64_t rows, int64_t cols, const dtas_config& cfg, int64_t la[7]) {
  RedInfo r;
  if (!red_info(op, &r)) return fail("reduction: unknown op %d", op);
  if (cfg.block < 64 || cfg.block > 1024 || cfg.block % 64 != 0)
    return fail("%s: block must be a multiple of 64 in [64, 1024], got %d", r.name, cfg.block);
  for (int i = 0; i < 7; ++i) la[i] = 0;
  la[1] = la[2] = 1;
  la[3] = cfg.block;
  int64_t grid;
  if (cfg.variant == DTAS_RED_WAVE_ROW) {
    const int64_t nvec = ceil_div(cols, r.vec);
    const int iters = pow2_at_least(ceil_div(nvec, 64));
    if (iters > 16) return fail("%s: a row of %lld elements does not fit one wavefront's registers", r.name, (long long)cols);
    la[5] = iters;
    la[6] = cfg.block / 64;
    grid = ceil_div(rows, cfg.block / 64);
  } else if (cfg.variant == DTAS_RED_BLOCK_ROW) {
    const int64_t nvec = ceil_div(cols, r.vec);
    const int iters = pow2_at_least(ceil_div(nvec, cfg.block));
    if (iters > 16) return fail("%s: a row of %lld elements does not fit %d threads' registers", r.name, (long long)cols, cfg.block);
    la[5] = iters;
    la[6] = 1;
    grid = rows;
  } else if (cfg.variant == DTAS_RED_STREAM_ROW) {
    la[6] = 1;
    grid = rows;
  } else {
    return fail("%s: unknown variant %d", r.name, cfg.variant);
  }
  if (cfg.grid_cap > 0 && grid > cfg.grid_cap) grid = cfg.grid_cap;
  if (grid > 0x7fffffff) grid = 0x7fffffff;
  la[0] = grid < 1 ? 1 : grid;
  return 0;
}

}  // namespace dtas

extern "C" {
int dtas_layer_norm_f32_f16(const void* x, const void* gamma, const void* beta, void* out, int64_t n, int64_t H,
                            float eps, const dtas_config* cfg, void* stream) {
  return dtas::run_reduction(DTAS_OP_LAYER_NORM_F32_F16, x, gamma, beta, out, n, H, eps, cfg, stream);
}
int dtas_rms_norm_f16(const void* x, const void* w, void* out, int64_t n, int64_t H, float eps, const dtas_config* cfg,
                      void* stream) {
  return dtas::run_reduction(DTAS_OP_RMS_NORM_F16, x, w, nullptr, out, n, H, eps, cfg, stream);
}
int dtas_softmax_f32_f16(const void* A, void* out, int64_t rows, int64_t cols, const dtas_config* cfg, void* stream) {
  return dtas::run_reduction(DTAS_OP_SOFTMAX_F32_F16, A, nullptr, nullptr, out, rows, cols, 0.f, cfg, stream);
}
int dtas_softmax_f16(const void* A, void* out, int64_t rows, int64_t cols, const dtas_config* cfg, void* stream) {
  return dtas::run_reduction(DTAS_OP_SOFTMAX_F16, A, nullptr, nullptr, out, rows, cols, 0.f, cfg, stream);
}
}

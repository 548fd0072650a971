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

// ---- rows whose length is not a multiple of the vector width, or whose buffers are only element-aligned
// (softmax over a dynamic row length: (1,32,n,m) with any m).  Vector slots that lie wholly inside a row are
// moved with the same 16-byte accesses at the row's own alignment (2 or 4 bytes: the hardware runs in its
// unaligned access mode, and the compiler emits one dwordx4 for these under-aligned types); the one slot that
// straddles the end of a row is moved element by element, its missing elements set to -inf, which max and
// exp-sum ignore.
typedef u32x4 __attribute__((aligned(2))) u32x4_a2;
typedef u32x4 __attribute__((aligned(4))) u32x4_a4;
typedef u32x2 __attribute__((aligned(2))) u32x2_a2;

template <typename In, int VEC>
__device__ __forceinline__ u32x4 load_ragged(const In* p, int64_t left) {  // left = elements of the row from p on
  if (left >= VEC) {
    if (sizeof(In) == 2) return __builtin_nontemporal_load(reinterpret_cast<const u32x4_a2*>(p));
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4_a4*>(p));
  }
  if (sizeof(In) == 2) {
    unsigned short h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = e < left ? reinterpret_cast<const unsigned short*>(p)[e] : 0xFC00u;  // -inf
    return u32x4{h[0] | (static_cast<unsigned>(h[1]) << 16), h[2] | (static_cast<unsigned>(h[3]) << 16),
                 h[4] | (static_cast<unsigned>(h[5]) << 16), h[6] | (static_cast<unsigned>(h[7]) << 16)};
  }
  u32x4 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = e < left ? reinterpret_cast<const unsigned*>(p)[e] : 0xFF800000u;  // -inf
  return r;
}

template <int VEC>
__device__ __forceinline__ void store_half_ragged(half_t* dst, const float (&v)[VEC], int64_t left) {
  if (left >= VEC) {
    if (VEC == 8) {
      f16x8 h;
#pragma unroll
      for (int e = 0; e < 8; ++e) h[e] = static_cast<half_t>(v[e]);
      __builtin_nontemporal_store(__builtin_bit_cast(u32x4, h), reinterpret_cast<u32x4_a2*>(dst));
    } else {
      f16x4 h;
#pragma unroll
      for (int e = 0; e < 4; ++e) h[e] = static_cast<half_t>(v[e]);
      __builtin_nontemporal_store(__builtin_bit_cast(u32x2, h), reinterpret_cast<u32x2_a2*>(dst));
    }
    return;
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e)
    if (e < left) dst[e] = static_cast<half_t>(v[e]);
}

// N independent reductions at once: DPP inside each wavefront, then (BLOCK) one LDS slot per
// wavefront and value, joined in wavefront order by every thread.  Consecutive calls alternate
// between two banks of N x 16 slots (`phase` counts them), so a bank is rewritten only after a
// barrier that every reader of its previous contents has passed: one barrier per call.
template <bool BLOCK, typename Op, int N>
__device__ __forceinline__ void group_reduce(float (&a)[N], float* slots, int& phase) {
#pragma unroll
  for (int k = 0; k < N; ++k) a[k] = Op::wave(a[k]);
  if (!BLOCK) return;
  const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  if (nwaves == 1) return;
  float* bank = slots + (phase++ & 1) * (N * 16);
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int k = 0; k < N; ++k) bank[k * 16 + wave] = a[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < N; ++k) {
    float r = bank[k * 16];
    for (int i = 1; i < nwaves; ++i) r = Op::join(r, bank[k * 16 + i]);
    a[k] = r;
  }
}

// ---- rows held in registers ---------------------------------------------------------
// rows: number of rows; cols: row length, a multiple of kVec, every row 16-byte aligned.
// A lane group (wavefront or workgroup) takes R consecutive rows per trip: all R x ITERS loads
// are in flight together, the R rows share each barrier, and the per-column parameters
// (w, or gamma and beta) are fetched once for the R rows.
// More than 8 vectors per lane need more registers than a 1024-thread workgroup leaves each lane.
// RAGGED (softmax): cols is any length and the buffers are element-aligned (see load_ragged).
template <int OP, int ITERS, bool BLOCK, int R, bool RAGGED = false>
__global__ void __launch_bounds__(ITERS * R > 8 ? 512 : 1024) row_reg_kernel(
    const void* __restrict__ xin, const void* __restrict__ p1, const void* __restrict__ p2, void* __restrict__ outp,
    int64_t rows, int64_t cols, float eps) {
  typedef typename RowTraits<OP>::In In;
  constexpr int VEC = RowTraits<OP>::kVec;
  typedef RowVec<In, VEC> V;
  __shared__ float slots[BLOCK ? 2 * 2 * R * 16 : 1];
  int phase = 0;

  const int lane = BLOCK ? threadIdx.x : (threadIdx.x & 63);
  const int width = BLOCK ? blockDim.x : 64;
  const int64_t trip_rows = static_cast<int64_t>(R) * (BLOCK ? 1 : (blockDim.x >> 6));
  static_assert(!RAGGED || OP == kSoftmaxF32 || OP == kSoftmaxF16, "ragged rows: softmax only");
  const int64_t nvec = RAGGED ? (cols + VEC - 1) / VEC : cols / VEC;
  const float inv_cols = 1.0f / static_cast<float>(cols);
  half_t* out = static_cast<half_t*>(outp);
  bool has[ITERS];  // which of this lane's vector slots lie inside the row
#pragma unroll
  for (int it = 0; it < ITERS; ++it) has[it] = lane + static_cast<int64_t>(it) * width < nvec;

  // A lane covers the same columns of every row, so its slices of the parameters are loaded
  // once per kernel; very long rows re-read them from the cache per trip
  // instead and keep the registers for the rows.
  constexpr bool HOIST = (OP == kRms || OP == kLayerNorm) && ITERS * (R + (OP == kLayerNorm ? 2 : 1)) <= 16;
  V pw[HOIST ? ITERS : 1], pb[HOIST ? ITERS : 1];
  if (HOIST) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      if (has[it]) {
        pw[it].raw = static_cast<const u32x4*>(p1)[lane + it * width];
        if (OP == kLayerNorm) pb[it].raw = static_cast<const u32x4*>(p2)[lane + it * width];
      }
    }
  }
  auto param = [&](const void* p, const V* held, int it) -> V {
    if (HOIST) return held[it];
    V r;
    r.raw = static_cast<const u32x4*>(p)[lane + it * width];
    return r;
  };

  // every thread of a workgroup runs the same number of trips (BLOCK: same rows;
  // WAVE: rows differ per wavefront but no workgroup barrier is used)
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * trip_rows + (BLOCK ? 0 : (threadIdx.x >> 6) * R); base < rows;
       base += static_cast<int64_t>(gridDim.x) * trip_rows) {
    V v[R][ITERS];
    bool live[R];  // rows past the end take part in the barriers only
#pragma unroll
    for (int r = 0; r < R; ++r) {
      live[r] = base + r < rows;
      const In* row_in = static_cast<const In*>(xin) + (base + r) * cols;
      const u32x4* src = reinterpret_cast<const u32x4*>(row_in);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        v[r][it].raw = u32x4{0u, 0u, 0u, 0u};
        if (live[r] && has[it]) {
          const int64_t at = (lane + static_cast<int64_t>(it) * width) * VEC;
          if (RAGGED) v[r][it].raw = load_ragged<In, VEC>(row_in + at, cols - at);
          else v[r][it].raw = load_stream(src + lane + it * width);
        }
      }
    }
    auto store_row = [&](int r, int it, const float (&res)[VEC]) {
      const int64_t at = (lane + static_cast<int64_t>(it) * width) * VEC;
      if (RAGGED) store_half_ragged<VEC>(out + (base + r) * cols + at, res, cols - at);
      else store_half_vec<VEC>(out + (base + r) * cols + at, res);
    };

    if (OP == kRms) {
      float ss[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        ss[r] = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          if (has[it]) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
              const float f = v[r][it].get(e);
              ss[r] += f * f;
            }
          }
        }
      }
      group_reduce<BLOCK, SumOp>(ss, slots, phase);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (has[it]) {
          const V w = param(p1, pw, it);
#pragma unroll
          for (int r = 0; r < R; ++r) {
            if (live[r]) {
              const float rs = __builtin_amdgcn_rsqf(ss[r] * inv_cols + eps);
              float res[VEC];
#pragma unroll
              for (int e = 0; e < VEC; ++e) res[e] = v[r][it].get(e) * rs * w.get(e);
              store_row(r, it, res);
            }
          }
        }
      }
    } else if (OP == kLayerNorm) {
      float st[2 * R];  // sum and sum of squares per row
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          if (has[it]) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
              const float f = v[r][it].get(e);
              s0 += f;
              s1 += f * f;
            }
          }
        }
        st[2 * r] = s0;
        st[2 * r + 1] = s1;
      }
      group_reduce<BLOCK, SumOp>(st, slots, phase);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (has[it]) {
          const V g = param(p1, pw, it), b = param(p2, pb, it);
#pragma unroll
          for (int r = 0; r < R; ++r) {
            if (live[r]) {
              const float mean = st[2 * r] * inv_cols;
              const float rstd = __builtin_amdgcn_rsqf(st[2 * r + 1] * inv_cols - mean * mean + eps);
              float res[VEC];
#pragma unroll
              for (int e = 0; e < VEC; ++e) res[e] = (v[r][it].get(e) - mean) * rstd * g.get(e) + b.get(e);
              store_row(r, it, res);
            }
          }
        }
      }
    } else {  // softmax
      float mx[R], sm[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        mx[r] = kNegMax;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          if (has[it]) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) mx[r] = fmaxf(mx[r], v[r][it].get(e));
          }
        }
      }
      group_reduce<BLOCK, MaxOp>(mx, slots, phase);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        sm[r] = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          if (has[it]) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) sm[r] += fast_exp(v[r][it].get(e) - mx[r]);
          }
        }
      }
      group_reduce<BLOCK, SumOp>(sm, slots, phase);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (!live[r]) continue;
        const float inv = 1.0f / sm[r];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          if (has[it]) {
            float res[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) res[e] = fast_exp(v[r][it].get(e) - mx[r]) * inv;
            store_row(r, it, res);
          }
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
  __shared__ float slots[64];
  int phase = 0;
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
      ss = block_reduce<SumOp>(ss, slots, phase);
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
      block_sum2(s0, s1, slots, phase);
      const float mean = s0 * inv_cols;
      const float rstd = __builtin_amdgcn_rsqf(s1 * inv_cols - mean * mean + eps);
      const float* g = static_cast<const float*>(p1);
      const float* b = static_cast<const float*>(p2);
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x)
        o[k] = static_cast<half_t>((static_cast<float>(x[k]) - mean) * rstd * g[k] + b[k]);
    } else {
      float mx = kNegMax;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) mx = fmaxf(mx, static_cast<float>(x[k]));
      mx = block_reduce<MaxOp>(mx, slots, phase);
      float s = 0.f;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) s += fast_exp(static_cast<float>(x[k]) - mx);
      s = block_reduce<SumOp>(s, slots, phase);
      const float inv = 1.0f / s;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x)
        o[k] = static_cast<half_t>(fast_exp(static_cast<float>(x[k]) - mx) * inv);
    }
  }
}

// instantiated (vectors per lane, rows per trip) pairs: ITERS * R <= 16
template <int OP, bool BLOCK, bool RAGGED = false>
int launch_reg(int iters, int rpt, dim3 grid, dim3 block, hipStream_t s, const void* x, const void* p1,
               const void* p2, void* out, int64_t rows, int64_t cols, float eps) {
#define DTAS_ROW_CASE(I, R)                                                                                              \
  case I * 8 + R:                                                                                                        \
    hipLaunchKernelGGL((row_reg_kernel<OP, I, BLOCK, R, RAGGED>), grid, block, 0, s, x, p1, p2, out, rows, cols, eps);   \
    break;
  switch (iters * 8 + rpt) {
    DTAS_ROW_CASE(1, 1) DTAS_ROW_CASE(1, 2) DTAS_ROW_CASE(1, 4)
    DTAS_ROW_CASE(2, 1) DTAS_ROW_CASE(2, 2) DTAS_ROW_CASE(2, 4)
    DTAS_ROW_CASE(3, 1) DTAS_ROW_CASE(3, 2) DTAS_ROW_CASE(3, 4)
    DTAS_ROW_CASE(4, 1) DTAS_ROW_CASE(4, 2) DTAS_ROW_CASE(4, 4)
    DTAS_ROW_CASE(5, 1) DTAS_ROW_CASE(5, 2)
    DTAS_ROW_CASE(6, 1) DTAS_ROW_CASE(6, 2)
    DTAS_ROW_CASE(8, 1) DTAS_ROW_CASE(8, 2)
    DTAS_ROW_CASE(10, 1)
    DTAS_ROW_CASE(12, 1)
    DTAS_ROW_CASE(16, 1)
    default:
      return fail("reduction: %d vectors per lane x %d rows per trip is not instantiated", iters, rpt);
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

// the instantiated vectors-per-lane counts; 17 = too long
int iters_at_least(int64_t v) {
  static const int kIters[] = {1, 2, 3, 4, 5, 6, 8, 10, 12, 16};
  for (int i : kIters)
    if (i >= v) return i;
  return 17;
}

// cfg.unroll of a register variant: rows a lane group takes per trip (0 and 1 both mean one)
int rows_per_trip(const dtas_config& cfg) { return cfg.unroll <= 1 ? 1 : cfg.unroll; }

template <int OP>
int launch_rows(const dtas_config& cfg, const int64_t la[7], hipStream_t s, const void* x, const void* p1,
                const void* p2, void* out, int64_t rows, int64_t cols, float eps, bool ragged) {
  const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
  if (cfg.variant == DTAS_RED_STREAM_ROW) {
    hipLaunchKernelGGL((row_stream_kernel<OP>), grid, block, 0, s, x, p1, p2, out, rows, cols, eps);
    return check_launch("reduction");
  }
  const int iters = static_cast<int>(la[5]), rpt = rows_per_trip(cfg);
  if constexpr (OP == kSoftmaxF32 || OP == kSoftmaxF16) {
    if (ragged) {
      if (cfg.variant == DTAS_RED_WAVE_ROW) return launch_reg<OP, false, true>(iters, rpt, grid, block, s, x, p1, p2, out, rows, cols, eps);
      return launch_reg<OP, true, true>(iters, rpt, grid, block, s, x, p1, p2, out, rows, cols, eps);
    }
  }
  if (cfg.variant == DTAS_RED_WAVE_ROW) return launch_reg<OP, false>(iters, rpt, grid, block, s, x, p1, p2, out, rows, cols, eps);
  return launch_reg<OP, true>(iters, rpt, grid, block, s, x, p1, p2, out, rows, cols, eps);
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
  // 128-bit row accesses at 16-byte alignment need cols % vec == 0 and aligned buffers.  Softmax rows of any
  // other length (the row length is its dynamic extent) keep the register kernels, with accesses at the rows'
  // own alignment; the norms take the element-access kernel (a bucket's config must serve every n in the bucket)
  const bool ragged = softmax && !vec_ok && aligned(x, r.in_bytes) && aligned(out, 2);
  if (cfg.variant != DTAS_RED_STREAM_ROW && !vec_ok && !ragged) {
    cfg.variant = DTAS_RED_STREAM_ROW;
    if (!user) cfg.block = cols >= 4096 ? 1024 : cols >= 1024 ? 512 : 256;
    cfg.vec = 1;
  }
  int64_t la[7];
  if (describe_reduction(op, rows, cols, cfg, la) != 0) return -1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (r.kind) {
    case kRms: return launch_rows<kRms>(cfg, la, s, x, p1, p2, out, rows, cols, eps, false);
    case kLayerNorm: return launch_rows<kLayerNorm>(cfg, la, s, x, p1, p2, out, rows, cols, eps, false);
    case kSoftmaxF32: return launch_rows<kSoftmaxF32>(cfg, la, s, x, p1, p2, out, rows, cols, eps, ragged);
    case kSoftmaxF16: return launch_rows<kSoftmaxF16>(cfg, la, s, x, p1, p2, out, rows, cols, eps, ragged);
  }
  return fail("reduction: unknown op %d", op);
}

}  // namespace

namespace {
bool rows_per_trip_ok(const char* name, int iters, int rpt, int block) {
  if (iters * rpt > 8 && block > 512) {
    fail("%s: %d vectors per lane x %d rows per trip need a block of at most 512 threads, got %d", name, iters, rpt, block);
    return false;
  }
  if (rpt == 1 || (rpt == 2 && iters <= 8) || (rpt == 4 && iters <= 4)) return true;
  fail("%s: unroll (rows per trip) %d is not available with %d vectors per lane (1, 2 or 4; 2 up to 8 vectors, 4 up to 4)",
       name, rpt, iters);
  return false;
}
}  // namespace

// launch_args: {grid, 1, 1, block, 0, vectors per lane (register variants), rows per workgroup and trip}
int describe_reduction(int op, int64_t rows, int64_t cols, const dtas_config& cfg, int64_t la[7]) {
  RedInfo r;
  if (!red_info(op, &r)) return fail("reduction: unknown op %d", op);
  if (cfg.block < 64 || cfg.block > 1024 || cfg.block % 64 != 0)
    return fail("%s: block must be a multiple of 64 in [64, 1024], got %d", r.name, cfg.block);
  for (int i = 0; i < 7; ++i) la[i] = 0;
  la[1] = la[2] = 1;
  la[3] = cfg.block;
  int64_t grid;
  const int rpt = rows_per_trip(cfg);
  if (cfg.variant == DTAS_RED_WAVE_ROW) {
    const int64_t nvec = ceil_div(cols, r.vec);
    const int iters = iters_at_least(ceil_div(nvec, 64));
    if (iters > 16) return fail("%s: a row of %lld elements does not fit one wavefront's registers", r.name, (long long)cols);
    if (!rows_per_trip_ok(r.name, iters, rpt, cfg.block)) return -1;
    la[5] = iters;
    la[6] = cfg.block / 64 * rpt;
    grid = ceil_div(rows, la[6]);
  } else if (cfg.variant == DTAS_RED_BLOCK_ROW) {
    const int64_t nvec = ceil_div(cols, r.vec);
    const int iters = iters_at_least(ceil_div(nvec, cfg.block));
    if (iters > 16) return fail("%s: a row of %lld elements does not fit %d threads' registers", r.name, (long long)cols, cfg.block);
    if (!rows_per_trip_ok(r.name, iters, rpt, cfg.block)) return -1;
    la[5] = iters;
    la[6] = rpt;
    grid = ceil_div(rows, rpt);
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

// layer_norm / layer_norm1 (before_dl.py:846-896): the final layer norm, fp32 in and fp32 out (the fused forms
// above round to fp16).  One workgroup of 256 per row; ITERS > 0 holds the row in registers (H % 4 == 0,
// H <= 1024 ITERS, 16-byte aligned rows), ITERS == 0 walks it twice with element accesses.
template <int ITERS>
__global__ void __launch_bounds__(256) layer_norm_f32_kernel(const float* __restrict__ x, const float* __restrict__ g,
                                                             const float* __restrict__ b, float* __restrict__ out,
                                                             int64_t rows, int64_t H, float eps) {
  __shared__ float slots[64];
  int phase = 0;
  const float inv = 1.0f / static_cast<float>(H);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const float* xr = x + row * H;
    float* o = out + row * H;
    float s0 = 0.f, s1 = 0.f;
    if constexpr (ITERS > 0) {
      f32x4 v[ITERS];
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int64_t k = (static_cast<int64_t>(it) * 256 + threadIdx.x) * 4;   // every load issued before the first use
        v[it] = *reinterpret_cast<const f32x4*>(xr + (k < H ? k : 0));
      }
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int64_t k = (static_cast<int64_t>(it) * 256 + threadIdx.x) * 4;
        if (k < H) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            s0 += v[it][e];
            s1 += v[it][e] * v[it][e];
          }
        }
      }
      block_sum2(s0, s1, slots, phase);
      const float mean = s0 * inv;
      const float rstd = 1.0f / sqrtf(s1 * inv - mean * mean + eps);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int64_t k = (static_cast<int64_t>(it) * 256 + threadIdx.x) * 4;
        if (k < H) {
          const f32x4 gv = *reinterpret_cast<const f32x4*>(g + k), bv = *reinterpret_cast<const f32x4*>(b + k);
          f32x4 r;
#pragma unroll
          for (int e = 0; e < 4; ++e) r[e] = (v[it][e] - mean) * rstd * gv[e] + bv[e];
          *reinterpret_cast<f32x4*>(o + k) = r;
        }
      }
    } else {
      for (int64_t k = threadIdx.x; k < H; k += blockDim.x) {
        s0 += xr[k];
        s1 += xr[k] * xr[k];
      }
      block_sum2(s0, s1, slots, phase);
      const float mean = s0 * inv;
      const float rstd = 1.0f / sqrtf(s1 * inv - mean * mean + eps);
      for (int64_t k = threadIdx.x; k < H; k += blockDim.x) o[k] = (xr[k] - mean) * rstd * g[k] + b[k];
    }
  }
}

// The same with a wavefront per row (four rows per workgroup, no barrier): for many rows.  H % 4 == 0,
// H <= 256 ITERS, 16-byte aligned rows.
template <int ITERS>
__global__ void __launch_bounds__(256) layer_norm_f32_wave_kernel(const float* __restrict__ x, const float* __restrict__ g,
                                                                  const float* __restrict__ b, float* __restrict__ out,
                                                                  int64_t rows, int64_t H, float eps) {
  const float inv = 1.0f / static_cast<float>(H);
  const int lane = threadIdx.x & 63;
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6); row < rows; row += static_cast<int64_t>(gridDim.x) * 4) {
    const float* xr = x + row * H;
    float* o = out + row * H;
    f32x4 v[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {   // every load issued before the first use
      const int64_t k = (it * 64 + lane) * 4;
      v[it] = *reinterpret_cast<const f32x4*>(xr + (k < H ? k : 0));
    }
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int64_t k = (it * 64 + lane) * 4;
      if (k < H) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s0 += v[it][e];
          s1 += v[it][e] * v[it][e];
        }
      }
    }
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    const float mean = s0 * inv;
    const float rstd = 1.0f / sqrtf(s1 * inv - mean * mean + eps);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int64_t k = (it * 64 + lane) * 4;
      if (k < H) {
        const f32x4 gv = *reinterpret_cast<const f32x4*>(g + k), bv = *reinterpret_cast<const f32x4*>(b + k);
        f32x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = (v[it][e] - mean) * rstd * gv[e] + bv[e];
        __builtin_nontemporal_store(r, reinterpret_cast<f32x4*>(o + k));
      }
    }
  }
}

// softmax_with_temperature (before_dl.py:4154-4161): divide2 (:57-65, logits / temperature, the temperature a
// device scalar) then softmax2 (:1062-1096), fp32 in and out, over the vocabulary.  One workgroup of 1024 per
// row; ITERS > 0 keeps the divided row in registers (cols <= 4096 ITERS, cols % 4 == 0, 16-byte aligned rows),
// ITERS == 0 walks the row three times with element accesses.  exp is the library's (the result stays fp32).
template <int ITERS>
__global__ void __launch_bounds__(1024) softmax_temp_kernel(const float* __restrict__ A, const float* __restrict__ temp,
                                                            float* __restrict__ out, int64_t rows, int64_t cols) {
  __shared__ float slots[64];
  int phase = 0;
  const float t = temp ? *temp : 1.f;   // no temperature: softmax2 alone (x / 1 is x)
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const float* x = A + row * cols;
    float* o = out + row * cols;
    if constexpr (ITERS > 0) {
      f32x4 v[ITERS];
      float mx = kNegMax;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {   // every load issued before the first use (slots past the row reread its start)
        const int64_t k = (static_cast<int64_t>(it) * 1024 + threadIdx.x) * 4;
        v[it] = *reinterpret_cast<const f32x4*>(x + (k < cols ? k : 0));
      }
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int64_t k = (static_cast<int64_t>(it) * 1024 + threadIdx.x) * 4;
        if (k < cols) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[it][e] = v[it][e] / t;
            mx = fmaxf(mx, v[it][e]);
          }
        } else {
          v[it] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        }
      }
      mx = block_reduce<MaxOp>(mx, slots, phase);
      float s = 0.f;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[it][e] = expf(v[it][e] - mx);
          s += v[it][e];
        }
      }
      s = block_reduce<SumOp>(s, slots, phase);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int64_t k = (static_cast<int64_t>(it) * 1024 + threadIdx.x) * 4;
        if (k < cols) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[it][e] = v[it][e] / s;
          *reinterpret_cast<f32x4*>(o + k) = v[it];
        }
      }
    } else {
      float mx = kNegMax;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) mx = fmaxf(mx, x[k] / t);
      mx = block_reduce<MaxOp>(mx, slots, phase);
      float s = 0.f;
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) s += expf(x[k] / t - mx);
      s = block_reduce<SumOp>(s, slots, phase);
      for (int64_t k = threadIdx.x; k < cols; k += blockDim.x) o[k] = expf(x[k] / t - mx) / s;
    }
  }
}

// The same result for a few long rows (the model has one row of 50280): a single workgroup spends its time on
// the two divisions and the exp of every element, so a row is shared by `parts` workgroups of 4096 elements.
// Every workgroup needs the row's maximum and sum; rather than exchange them it derives them again from the
// whole row with cheap arithmetic -- max_k(x_k / t) = (max_k x_k) / t for t > 0 ((min_k x_k) / t for t < 0:
// a correctly rounded division is monotone), and the sum of exp((x_k - x_max) / t) through the hardware's
// reciprocal and exp2 -- and pays the exact division and the library's exp only on its own 4096 elements.
// No scratch memory, one launch, the same bits on every run.  cols % 4 == 0, cols <= 4096 ITERS, 16-byte rows.
template <int ITERS>
__global__ void __launch_bounds__(1024) softmax_temp_split_kernel(const float* __restrict__ A, const float* __restrict__ temp,
                                                                  float* __restrict__ out, int64_t cols, int parts) {
  __shared__ float slots[64];
  int phase = 0;
  const float t = temp ? *temp : 1.f;   // no temperature: softmax2 alone (x / 1 is x)
  const int64_t row = blockIdx.x / parts;
  const int part = blockIdx.x % parts;
  const float* x = A + row * cols;
  f32x4 v[ITERS];
  float hi = kNegMax;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {   // every load issued before the first use (slots past the row reread its start)
    const int64_t k = (static_cast<int64_t>(it) * 1024 + threadIdx.x) * 4;
    v[it] = *reinterpret_cast<const f32x4*>(x + (k < cols ? k : 0));
  }
  const float sign = t < 0.f ? -1.f : 1.f;   // the extreme that the division turns into the maximum: max x for t > 0, min x for t < 0
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int64_t k = (static_cast<int64_t>(it) * 1024 + threadIdx.x) * 4;
    if (k < cols) {
#pragma unroll
      for (int e = 0; e < 4; ++e) hi = fmaxf(hi, sign * v[it][e]);
    }
  }
  const float xm = sign * block_reduce<MaxOp>(hi, slots, phase);
  const float mx = fmaxf(kNegMax, xm / t);
  const float rt = kLog2e * __builtin_amdgcn_rcpf(t);
  float s = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int64_t k = (static_cast<int64_t>(it) * 1024 + threadIdx.x) * 4;
    if (k < cols) {
#pragma unroll
      for (int e = 0; e < 4; ++e) s += __builtin_amdgcn_exp2f((v[it][e] - xm) * rt);
    }
  }
  s = block_reduce<SumOp>(s, slots, phase);
  const int64_t k = (static_cast<int64_t>(part) * 1024 + threadIdx.x) * 4;
  if (k < cols) {
    f32x4 w = *reinterpret_cast<const f32x4*>(x + k);
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = expf(w[e] / t - mx) / s;
    *reinterpret_cast<f32x4*>(out + row * cols + k) = w;
  }
}

// The same for rows of more than 65536 elements (vocabularies of 128256 or 151936): the row does not fit the registers
// of one workgroup, so the two passes over the whole row read it from the cache again, four vectors in flight per
// thread; a thread adds up the same elements in the same order as above.
__global__ void __launch_bounds__(1024) softmax_temp_split_loop_kernel(const float* __restrict__ A, const float* __restrict__ temp,
                                                                       float* __restrict__ out, int64_t cols, int parts) {
  __shared__ float slots[64];
  int phase = 0;
  const float t = temp ? *temp : 1.f;
  const int64_t row = blockIdx.x / parts;
  const int part = blockIdx.x % parts;
  const float* x = A + row * cols;
  const float sign = t < 0.f ? -1.f : 1.f;
  float hi = kNegMax;
  for (int64_t k0 = static_cast<int64_t>(threadIdx.x) * 4; k0 < cols; k0 += 4 * 4096) {
    f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t k = k0 + u * 4096;
      v[u] = *reinterpret_cast<const f32x4*>(x + (k < cols ? k : 0));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (k0 + u * 4096 < cols) {
#pragma unroll
        for (int e = 0; e < 4; ++e) hi = fmaxf(hi, sign * v[u][e]);
      }
  }
  const float xm = sign * block_reduce<MaxOp>(hi, slots, phase);
  const float mx = fmaxf(kNegMax, xm / t);
  const float rt = kLog2e * __builtin_amdgcn_rcpf(t);
  float s = 0.f;
  for (int64_t k0 = static_cast<int64_t>(threadIdx.x) * 4; k0 < cols; k0 += 4 * 4096) {
    f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t k = k0 + u * 4096;
      v[u] = *reinterpret_cast<const f32x4*>(x + (k < cols ? k : 0));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (k0 + u * 4096 < cols) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s += __builtin_amdgcn_exp2f((v[u][e] - xm) * rt);
      }
  }
  s = block_reduce<SumOp>(s, slots, phase);
  const int64_t k = (static_cast<int64_t>(part) * 1024 + threadIdx.x) * 4;
  if (k < cols) {
    f32x4 w = *reinterpret_cast<const f32x4*>(x + k);
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = expf(w[e] / t - mx) / s;
    *reinterpret_cast<f32x4*>(out + row * cols + k) = w;
  }
}

}  // namespace dtas

extern "C" {
int dtas_layer_norm_f32(const void* x, const void* gamma, const void* beta, void* out, int64_t n, int64_t H, float eps,
                        void* stream) {
  using namespace dtas;
  clear_error();
  if (n < 0 || H < 0) return fail("layer_norm_f32: negative extent n=%lld H=%lld", (long long)n, (long long)H);
  if (n == 0 || H == 0) return 0;
  if (n > INT64_MAX / 8 / H) return fail("layer_norm_f32: n*H overflows");
  if (!x || !gamma || !beta || !out) return fail("layer_norm_f32: NULL buffer");
  if (!aligned(x, 4) || !aligned(gamma, 4) || !aligned(beta, 4) || !aligned(out, 4)) return fail("layer_norm_f32: buffers must be 4-byte aligned");
  if (overlaps(out, n * H * 4, x, n * H * 4) || overlaps(out, n * H * 4, gamma, H * 4) || overlaps(out, n * H * 4, beta, H * 4))
    return fail("layer_norm_f32: output overlaps an input");
  const bool vec = H % 4 == 0 && H <= 8192 && aligned(x, 16) && aligned(out, 16) && aligned(gamma, 16) && aligned(beta, 16);
  const unsigned grid = static_cast<unsigned>(n > int64_t{kNumCU} * 32 ? int64_t{kNumCU} * 32 : n);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float* xp = static_cast<const float*>(x);
  const float* gp = static_cast<const float*>(gamma);
  const float* bp = static_cast<const float*>(beta);
  float* op = static_cast<float*>(out);
  if (vec && H <= 4096 && n >= 2 * kNumCU) {   // many rows: a wavefront each
    const unsigned wgrid = static_cast<unsigned>(ceil_div(n, 4) > int64_t{kNumCU} * 32 ? int64_t{kNumCU} * 32 : ceil_div(n, 4));
    if (H <= 1024) hipLaunchKernelGGL(layer_norm_f32_wave_kernel<4>, dim3(wgrid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
    else if (H <= 2560) hipLaunchKernelGGL(layer_norm_f32_wave_kernel<10>, dim3(wgrid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
    else hipLaunchKernelGGL(layer_norm_f32_wave_kernel<16>, dim3(wgrid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
    return check_launch("layer_norm_f32");
  }
  if (vec && H <= 1024) hipLaunchKernelGGL(layer_norm_f32_kernel<1>, dim3(grid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
  else if (vec && H <= 2048) hipLaunchKernelGGL(layer_norm_f32_kernel<2>, dim3(grid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
  else if (vec && H <= 3072) hipLaunchKernelGGL(layer_norm_f32_kernel<3>, dim3(grid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
  else if (vec && H <= 4096) hipLaunchKernelGGL(layer_norm_f32_kernel<4>, dim3(grid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
  // (rows of up to 8192: in registers as well -- [4096, 8192] took 83 us with two passes of element accesses)
  else if (vec && H <= 6144) hipLaunchKernelGGL(layer_norm_f32_kernel<6>, dim3(grid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
  else if (vec) hipLaunchKernelGGL(layer_norm_f32_kernel<8>, dim3(grid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
  else hipLaunchKernelGGL(layer_norm_f32_kernel<0>, dim3(grid), dim3(256), 0, st, xp, gp, bp, op, n, H, eps);
  return check_launch("layer_norm_f32");
}
static int run_softmax_f32(const char* what, const void* logits, const void* temperature, bool with_temperature, void* out,
                           int64_t rows, int64_t cols, void* stream) {
  using namespace dtas;
  clear_error();
  if (rows < 0 || cols < 0) return fail("%s: negative extent rows=%lld cols=%lld", what, (long long)rows, (long long)cols);
  if (rows == 0 || cols == 0) return 0;
  if (rows > INT64_MAX / 8 / cols) return fail("%s: rows*cols overflows", what);
  if (!logits || (with_temperature && !temperature) || !out) return fail("%s: NULL buffer", what);
  if (!aligned(logits, 4) || (with_temperature && !aligned(temperature, 4)) || !aligned(out, 4)) return fail("%s: buffers must be 4-byte aligned", what);
  if (overlaps(out, rows * cols * 4, logits, rows * cols * 4)) return fail("%s: output overlaps the input", what);
  const bool vec_any = cols % 4 == 0 && aligned(logits, 16) && aligned(out, 16);
  const bool vec = vec_any && cols <= 4096 * 16;
  const unsigned grid = static_cast<unsigned>(rows > int64_t{kNumCU} * 8 ? int64_t{kNumCU} * 8 : rows);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float* x = static_cast<const float*>(logits);
  const float* t = static_cast<const float*>(temperature);
  float* o = static_cast<float*>(out);
  const int64_t parts = ceil_div(cols, 4096);
  if (vec_any && parts > 1 && rows * parts <= 2 * kNumCU) {
    const unsigned wgs = static_cast<unsigned>(rows * parts);
    if (parts <= 4)
      hipLaunchKernelGGL(softmax_temp_split_kernel<4>, dim3(wgs), dim3(1024), 0, st, x, t, o, cols, static_cast<int>(parts));
    else if (parts <= 16)
      hipLaunchKernelGGL(softmax_temp_split_kernel<16>, dim3(wgs), dim3(1024), 0, st, x, t, o, cols, static_cast<int>(parts));
    else   // (a row of 128256: 86 us with one workgroup walking it element by element)
      hipLaunchKernelGGL(softmax_temp_split_loop_kernel, dim3(wgs), dim3(1024), 0, st, x, t, o, cols, static_cast<int>(parts));
  } else if (vec && cols <= 4096)
    hipLaunchKernelGGL(softmax_temp_kernel<1>, dim3(grid), dim3(1024), 0, st, x, t, o, rows, cols);
  else if (vec && cols <= 4096 * 4)
    hipLaunchKernelGGL(softmax_temp_kernel<4>, dim3(grid), dim3(1024), 0, st, x, t, o, rows, cols);
  else if (vec)
    hipLaunchKernelGGL(softmax_temp_kernel<16>, dim3(grid), dim3(1024), 0, st, x, t, o, rows, cols);
  else
    hipLaunchKernelGGL(softmax_temp_kernel<0>, dim3(grid), dim3(1024), 0, st, x, t, o, rows, cols);
  return check_launch(what);
}
int dtas_softmax_temperature_f32(const void* logits, const void* temperature, void* out, int64_t rows, int64_t cols,
                                 void* stream) {
  return run_softmax_f32("softmax_temperature", logits, temperature, true, out, rows, cols, stream);
}
int dtas_softmax_f32(const void* A, void* out, int64_t rows, int64_t cols, void* stream) {
  return run_softmax_f32("softmax_f32", A, nullptr, false, out, rows, cols, stream);
}
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

// Shared by the GEMM-family sources (gemm_tiles.hip, gemm_stream.hip, attention.hip, gemm_q8.hip, workspace.hip):
// the epilogue descriptor, the LDS layout of operand tiles, the epilogue arithmetic of the fused PrimFuncs, and the
// host-side interfaces between those files.  Internal to libdtas_gfx950.so.
#pragma once
#include "dtas_device.h"
#include "dtas_host.h"

#include <mutex>
#include <type_traits>

namespace dtas {

// What follows the product, as the fused PrimFuncs spell it: every intermediate is an fp16 tensor,
// so every step below rounds to fp16 (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:163-200
// fused_NT_matmul2_add1_add3_add3, :202-246 ..._cast, :248-318 fused_NT_matmul3_add2_gelu).
struct GemmEpilogue {
  const half_t* bias;  // [N] or NULL
  const half_t* res1;  // [M, N]: ADD2 kinds
  const half_t* res2;  // [M, N]: ADD2 kinds
  int kind;            // enum dtas_epilogue, or kEpiScores
  int out_f32;         // the output buffer holds fp32 (ADD2_CAST_F32, scores)
  float scale;         // scores: the fp16 constant the product is multiplied by
  // batched launches: element strides between consecutive problems, and how many there are (the MFMA
  // launcher fills `batches`; the element-access kernel takes the problem from blockIdx.y)
  int64_t stride_a, stride_w, stride_c, stride_res;
  unsigned batches;
  unsigned tiles_pinned;  // batched launches: an XCD keeps its tiles and walks the problems (see the kernel)
  const half_t* wscale;   // 8-bit W: the fp16 scales [N][K/32]
  int64_t lda;            // k-major W only (P.V): row stride of A in elements when its rows are padded; 0 = K
  unsigned tiles_unsplit; // one problem only: tiles [0, tiles_unsplit) are computed whole, only the rest is split over nsplit workgroups
  unsigned k_tail;        // k-major W only (P.V): A's rows and W hold k_tail (< 8) more k than K, which the MFMA loop leaves out and
                          // the epilogue adds (A's rows are then fetched at whatever alignment lda gives them)
  unsigned k_stagger;     // k-major W only (P.V): workgroup i starts at its k tile i mod (its k tiles) and wraps around
};

// Attention scores, fused_NT_matmul1_divide_maximum_minimum_cast2 (before_dl.py:116-160):
// fp32(min(max(fp16(mm * fp16(scale)), -65504), mask)), mask = res1 shared by all heads.
constexpr int kEpiScores = 100;

// ---- workspace.hip: library-owned scratch memory (split-K partial tiles and arrival counters, the rewritten operand)
extern std::recursive_mutex g_ws_mutex;
// Partial tiles and arrival counters of a launch that splits K over `nsplit` workgroups per tile: the static scratch
// if the calling thread is inside dtas_gemm_f16_static, else the stream's workspace, whose lock `lock` then holds
// (the caller keeps it until its kernel is enqueued).
int split_scratch(hipStream_t s, size_t bytes, size_t split_tiles, int nsplit, float** partials, unsigned** arrivals,
                  std::unique_lock<std::recursive_mutex>* lock);
// The stream's buffer for a rewritten operand (g_ws_mutex held by the caller until the launches that use it are enqueued).
int operand_workspace(hipStream_t stream, size_t bytes, void** out);
// Where a launch that splits K keeps its partial tiles when the caller must not allocate: set (per host thread) by
// dtas_gemm_f16_static around its call into the common code, read by split_scratch.
struct FixedScratch {
  float* partials;
  size_t partial_bytes;
  unsigned* arrivals;
  size_t tiles;
};
extern thread_local const FixedScratch* t_fixed_scratch;

// ---- gemm_tiles.hip: the MFMA tile kernels on a row-major fp16 W (every epilogue kind, batched launches)
int launch_tile_f16(const dtas_config& cfg, hipStream_t s, const half_t* A, const half_t* W, const GemmEpilogue& ep, void* C,
                    int64_t M, int64_t N, int64_t K, int batch);

// ---- gemm_stream.hip: the kernels that stream W once (SKINNY, STREAM and its looping form, ROWS) and the
// element-access kernel; `la` = launch_args of describe_gemm for the same cfg
int launch_gemm_rows(const dtas_config& cfg, const int64_t la[7], hipStream_t s, const half_t* A, const half_t* W,
                     const GemmEpilogue& ep, void* C, int64_t M, int64_t N, int64_t K);
int launch_gemm_skinny(const dtas_config& cfg, const int64_t la[7], hipStream_t s, const half_t* A, const half_t* W,
                       const GemmEpilogue& ep, void* C, int64_t M, int64_t N, int64_t K);
// fp16 W: every instantiated STREAM tile, the looping form included (tile[2] == 256)
int launch_gemm_stream(const dtas_config& cfg, hipStream_t s, const half_t* A, const half_t* W, const GemmEpilogue& ep, void* C,
                       int64_t M, int64_t N, int64_t K);
// 8-bit W (bytes [N][K], scales in ep.wscale): rows of A in {16, 32, 64}, K slices of 512 or 1024 (16 rows only)
int launch_gemm_stream_q8(int rows_a, int k_slice, hipStream_t s, const half_t* A, const half_t* Wq, const GemmEpilogue& ep, void* C,
                          int64_t M, int64_t N, int64_t K);
// DTAS_GEMM_MFMA_ACC16: the accumulator rounded to fp16 after every k step of 16 (cfg.vec 8: 16-byte operand loads, else elements)
int launch_gemm_acc16(const dtas_config& cfg, hipStream_t s, const half_t* A, const half_t* W, const GemmEpilogue& ep, void* C,
                      int64_t M, int64_t N, int64_t K);
// one thread per element of C: any K and alignment; grid.y = batch; w_kmajor: W is [K][N]; ep.wscale set: 8-bit W
int launch_gemm_scalar(const char* what, unsigned grid_x, unsigned batch, hipStream_t s, const half_t* A, const half_t* W,
                       const GemmEpilogue& ep, void* C, int64_t M, int64_t N, int64_t K, bool w_kmajor);

// the looping form of the W-streaming kernel (tile[2] == 256): rows of A x columns, and the stages it runs with
inline int stream_loop_stages(int bm, int bn) {
  if (bm == 16 && bn == 64) return 4;  // 160 KiB: one workgroup per CU
  if (bm == 16 && bn == 16) return 4;  // 64 KiB: two one-wavefront workgroups per CU
  return 0;
}
// the instantiated W-streaming shapes: rows of A x columns x K slice
inline bool stream_shape_ok(int bm, int bn, int bk) {
  if ((bm != 16 && bm != 32 && bm != 64) || (bn != 64 && bn != 128) || (bk != 512 && bk != 1024)) return false;
  return (bm + bn) * bk * 2 <= kLdsBytes;
}

namespace {

typedef float f32x4v __attribute__((ext_vector_type(4)));
// The same vectors at the alignment of their elements: rows of a dynamic length start anywhere (the scores'
// m, the residuals' N), the hardware runs in its unaligned access mode and the compiler emits one access for
// these types as it does for the aligned ones.
typedef f32x4v __attribute__((aligned(4))) f32x4v_a4;
typedef f16x4 __attribute__((aligned(2))) f16x4_a2;
typedef float f32x2v __attribute__((ext_vector_type(2)));

constexpr int kBK = 64;             // k extent of a tile: 128 bytes of fp16
constexpr int kRowBytes = kBK * 2;  // one tile row in LDS
constexpr unsigned kOob = 0x80000000u;

// Byte offset, inside an operand tile in LDS, of 16-byte chunk c (0..7) of tile row r.
// Rows are stored in pairs of 256 bytes = 16 slots.  The chunk index is xor-ed with r & 7 and
// the half of the pair with bit 3 of r, so that (a) the 8 chunks of one row, (b) one chunk of 8
// consecutive rows and (c) one chunk of 16 consecutive rows each fall into distinct 16-byte
// bank groups, whether the LDS serves 8 or 16 lanes of a 128-bit access per pass.
__host__ __device__ __forceinline__ constexpr unsigned lds_chunk_offset(unsigned r, unsigned c) {
  return (r >> 1) * 256u + ((((r ^ (r >> 3)) & 1u) << 3) | (c ^ (r & 7u))) * 16u;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

__device__ __forceinline__ half_t round_h(float v) { return static_cast<half_t>(v); }

// mm: the product already rounded to fp16.  Returns the fp16 result (the cast kinds widen it).
// KIND is a compile-time constant where the caller has dispatched on it (the tile epilogue: one
// specialised store loop per kind keeps erf and the residual handling out of the plain path).
template <int KIND>
__device__ __forceinline__ half_t epilogue_value_k(half_t mm, bool has_bias, float scale, float bias_j, float r1, float r2) {
  half_t t = mm;
  if (has_bias) t = round_h(static_cast<float>(t) + bias_j);
  if (KIND == DTAS_EPI_BIAS_ADD2 || KIND == DTAS_EPI_BIAS_ADD2_CAST_F32) {
    t = round_h(r1 + static_cast<float>(t));   // T_add_1 = lv58 + T_add
    t = round_h(static_cast<float>(t) + r2);   // T_add_2 = T_add_1 + lv2
  } else if (KIND == kEpiScores) {
    t = round_h(static_cast<float>(t) * scale);                          // T_divide (a multiply by fp16(1/sqrt(d)))
    t = round_h(fmaxf(static_cast<float>(t), -65504.f));                 // T_maximum
    t = round_h(fminf(static_cast<float>(t), r1));                       // T_minimum with the mask
  } else if (KIND == DTAS_EPI_BIAS_GELU) {
    t = gelu_erf_f16_steps(t);
  }
  return t;
}

// The scores' three steps on four values as packed fp16 instructions: fp32 holds the product of two fp16 numbers exactly,
// so the fp16 product rounded once is what the step computed through fp32 gives, and maximum and minimum are exact (the
// same NaN rule as fmaxf / fminf: the other operand) -- the same bits for a quarter of the instructions, in an epilogue
// that is bound by them (a 128x64 tile is 32 scores per lane).
__device__ __forceinline__ f16x4 scores_steps_vec(f16x4 mm, float scale, f16x4 mask) {
#pragma clang fp contract(off)
  const half_t sc = static_cast<half_t>(scale), low = static_cast<half_t>(-65504.f);
  const f16x4 s4 = {sc, sc, sc, sc}, low4 = {low, low, low, low};
  f16x4 t = mm * s4;                      // T_divide (a multiply by fp16(1/sqrt(d)))
  t = __builtin_elementwise_max(t, low4);  // T_maximum
  t = __builtin_elementwise_min(t, mask);  // T_minimum with the mask
  return t;
}

// "+ bias" and the two residual additions on a vector of fp16 values, each step one packed fp16 addition: T_add = mm +
// bias, T_add_1 = res1 + T_add, T_add_2 = T_add_1 + res2 (before_dl.py:163-206), every one rounded to fp16.
template <typename V, bool ADD2>
__device__ __forceinline__ V add_steps_vec(V t, bool has_bias, V bias, V r1, V r2) {
#pragma clang fp contract(off)
  if (has_bias) t = t + bias;
  if (ADD2) {
    t = r1 + t;
    t = t + r2;
  }
  return t;
}

__device__ __forceinline__ half_t epilogue_value(half_t mm, const GemmEpilogue& ep, float bias_j, float r1, float r2) {
  const bool hb = ep.bias != nullptr;
  switch (ep.kind) {
    case DTAS_EPI_BIAS_ADD2:
    case DTAS_EPI_BIAS_ADD2_CAST_F32: return epilogue_value_k<DTAS_EPI_BIAS_ADD2>(mm, hb, ep.scale, bias_j, r1, r2);
    case DTAS_EPI_BIAS_GELU: return epilogue_value_k<DTAS_EPI_BIAS_GELU>(mm, hb, ep.scale, bias_j, r1, r2);
    case kEpiScores: return epilogue_value_k<kEpiScores>(mm, hb, ep.scale, bias_j, r1, r2);
    default: return epilogue_value_k<DTAS_EPI_BIAS>(mm, hb, ep.scale, bias_j, r1, r2);
  }
}

// one element, any alignment (skinny and element-access kernels)
__device__ __forceinline__ void finish(float acc, const GemmEpilogue& ep, void* C, int64_t row, int64_t col, int64_t N) {
  const bool add2 = ep.kind == DTAS_EPI_BIAS_ADD2 || ep.kind == DTAS_EPI_BIAS_ADD2_CAST_F32;
  const half_t r = epilogue_value(round_h(acc), ep, ep.bias ? static_cast<float>(ep.bias[col]) : 0.f,
                                  add2 || ep.kind == kEpiScores ? static_cast<float>(ep.res1[row * N + col]) : 0.f,
                                  add2 ? static_cast<float>(ep.res2[row * N + col]) : 0.f);
  if (ep.out_f32) static_cast<float*>(C)[row * N + col] = static_cast<float>(r);
  else static_cast<half_t*>(C)[row * N + col] = r;
}

// The 4 * MT sums a lane of the W-streaming kernels holds for column `col` (register v of block i: row i * 16 + 4 * g + v).
// Bias and residuals are few and scattered (2 bytes per lane and row) and come from memory nobody has touched: they are
// requested when the kernel starts, ahead of the operands, and wait in registers, instead of costing a round trip of
// their own after the last MFMA (and one per row, behind the store before it, if they were read element by element).
template <int MT>
struct ColumnOperands {
  half_t bias, r1[MT][4], r2[MT][4];  // as loaded: widening them here would make the wavefront wait for each load where it is issued
};
template <int MT>
__device__ __forceinline__ void load_column_operands(ColumnOperands<MT>& o, const GemmEpilogue& ep, unsigned g, int64_t col, int64_t M,
                                                     int64_t N) {
  const bool add2 = ep.kind == DTAS_EPI_BIAS_ADD2 || ep.kind == DTAS_EPI_BIAS_ADD2_CAST_F32;
  const bool use_r1 = add2 || ep.kind == kEpiScores;
  const half_t zero = static_cast<half_t>(0.f);
  o.bias = ep.bias && col < N ? ep.bias[col] : zero;
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int64_t row = i * 16 + 4 * g + v;
      const bool in = row < M && col < N;
      o.r1[i][v] = use_r1 && in ? ep.res1[row * N + col] : zero;
      o.r2[i][v] = add2 && in ? ep.res2[row * N + col] : zero;
    }
}
// Called where the operands are known to have arrived (behind a wait for younger loads): the values must exist here,
// so the compiler cannot move their loads down to their only use, behind the main loop and the hand-over.
template <int MT>
__device__ __forceinline__ void pin_column_operands(const ColumnOperands<MT>& o) {
  asm volatile("" ::"v"(o.bias));
#pragma unroll
  for (int i = 0; i < MT; ++i)
    asm volatile("" ::"v"(o.r1[i][0]), "v"(o.r1[i][1]), "v"(o.r1[i][2]), "v"(o.r1[i][3]), "v"(o.r2[i][0]), "v"(o.r2[i][1]), "v"(o.r2[i][2]),
                 "v"(o.r2[i][3]));
}
template <int MT>
__device__ __forceinline__ void finish_column(const f32x4v (&acc)[MT], const ColumnOperands<MT>& o, const GemmEpilogue& ep, void* C,
                                              unsigned g, int64_t col, int64_t M, int64_t N) {
  if (col >= N) return;
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int64_t row = i * 16 + 4 * g + v;
      if (row >= M) continue;
      const half_t r = epilogue_value(round_h(acc[i][v]), ep, static_cast<float>(o.bias), static_cast<float>(o.r1[i][v]),
                                      static_cast<float>(o.r2[i][v]));
      if (ep.out_f32) static_cast<float*>(C)[row * N + col] = static_cast<float>(r);
      else static_cast<half_t*>(C)[row * N + col] = r;
    }
}

// Position of workgroup `wg` in a tile order in which each XCD gets a contiguous span:
// the hardware deals consecutive workgroup ids round-robin over the 8 XCDs.
__device__ __forceinline__ unsigned xcd_contiguous_id(unsigned wg, unsigned total) {
  const unsigned xcd = wg % kNumXCD, local = wg / kNumXCD;
  const unsigned base = total / kNumXCD, rem = total % kNumXCD;
  return xcd * base + (xcd < rem ? xcd : rem) + local;
}

#define DTAS_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// s_waitcnt lgkmcnt(0) vmcnt(v): v is a field of the instruction (bits [3:0] and [15:14])
constexpr int waitcnt_imm(int v) { return 0x0070 | (v & 15) | ((v >> 4) << 14); }

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Waits until at most min(n, MAX) whole tiles' loads (KL per lane each) are outstanding (n <= 0: none).  The
// wait count is an immediate, hence the chain of comparisons.
template <int KL, int MAX>
__device__ __forceinline__ void wait_whole_tiles(int n) {
  if constexpr (MAX <= 0) {
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
  } else {
    if (n >= MAX) __builtin_amdgcn_s_waitcnt(waitcnt_imm(MAX * KL));
    else wait_whole_tiles<KL, MAX - 1>(n);
  }
}

}  // namespace
}  // namespace dtas

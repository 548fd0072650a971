// Dynamic-M GEMM for gfx950: C[M,N] = A[M,K] . W[N,K]^T (+ bias[N]); fp16 in/out, fp32
// accumulation on the MFMA matrix cores.  The fused-epilogue GEMMs and the two batched
// attention matmuls run on the same kernels.
//
// Replaces the kernels DTAS's WMMA rule generates (python/dtas/schedule/tir_wmma.py:20-222:
// pad M to a tile multiple, block tile (i*micro_x*16) x (j*micro_y*16), k tile micro_k*16,
// A/B staged in shared.dyn by cooperative_fetch (python/dtas/schedule/tir_base.py:37-97),
// two-stage software pipeline, accumulators through shared memory to a guarded vector
// store; example output experiment/testIR/GEMM/m_n2560_k10240/wmma/16x16x16/i2j4_x7y2_in8.py).
//
// MFMA kernel (M > 64)
//   tile     : BM x BN x 64 per workgroup; WM x WN wavefronts (8 for 256x256 and, on request, 256x128 /
//              128x256; else 4), each owning (BM/WM) x (BN/WN) as 32x32 blocks of
//              v_mfma_f32_32x32x16_f16 (16x16 blocks of v_mfma_f32_16x16x32_f16 on the 8-wavefront
//              tiles), fp32 accumulators in registers.  Both operands are K-contiguous, so a tile row
//              is one 128-byte line = 8 chunks of 16 bytes.
//   global   : 128-bit buffer loads that write LDS directly (no register staging, no
//              ds_write): one wavefront instruction fills one 1 KiB block = 8 tile rows; which
//              (row, chunk) a lane fetches is the inverse of the LDS swizzle.  Rows past M / N
//              and chunks past K fall outside the buffer's range and arrive as zeros.
//   LDS      : two to four stages of (BM + BN) x 128 B (256x256: a ring of five 32 KiB operand
//              units).  Chunk c of row r sits at a swizzled slot so
//              that the MFMA operand reads (a column of 32 rows per half-wavefront, 128 bit
//              per lane) spread over all 64 banks.
//   pipeline : 4-wavefront tiles: fragments of step s+1 are read from LDS while the MFMAs of step
//              s issue (two register sets); the tile barrier sits before the last step of a k
//              tile, the loads of tile k+2 are issued right after it into the stage just
//              vacated, and the first fragments of tile k+1 are read under the last MFMAs of
//              tile k.  The interleaving is pinned with scheduling barriers.
//              8-wavefront tiles: v_mfma_f32_16x16x32_f16 (more flops per watt than 32x32x16,
//              and the card is power-limited on random operands), a whole k32 step of fragments in
//              registers, one barrier per k tile; wavefronts w and w+4 share a SIMD, the older one
//              wins the MFMA pipe, and each requests its share of the next units while the other
//              multiplies (a wavefront that issues a load stalls until the load path takes it).
//   epilogue : accumulators -> fp16 -> wavefront-private LDS region (xor-swizzled 8-byte
//              slots) -> coalesced stores of whole tile rows (8 bytes per lane, 16 on the
//              8-wavefront tiles) with the bias added on the way out.
//   launch   : workgroup ids are remapped so that each XCD (own L2) works on a compact patch of
//              the tile grid.
//   split K  : few output tiles -> several workgroups share a tile and meet in a workspace.
//   epilogues: bias; bias + two residuals (optionally widened to fp32); bias + erf-GELU; the
//              attention scores' scale / clamp / mask -- every step an fp16 value, as the fused
//              PrimFuncs spell them.
//   batches  : the attention matmuls run all heads in one launch (strides in GemmEpilogue).
//   k-major W: for P.V the V tiles are transposed on their way into the LDS (template flag WT).
// SKINNY kernel (M <= 80): the work is streaming W once; a workgroup owns 16 columns of C and
//              all of M, its wavefronts split K, v_mfma_f32_16x16x32_f16 operands are loaded
//              straight from global memory, partial tiles are folded through LDS.
// STREAM kernel (M <= 64; the built-in choice for M <= 16): W rows come in as 1 KiB direct-to-LDS
//              loads, everything a workgroup needs requested at once; K slices meet in the workspace.
//              With 8-bit weights (M <= 32) the bytes ride the same loads and are widened between
//              the LDS and the MFMA.  For a W with many rows (4096 < N <= 16384, K <= 4096) the looping
//              form: a workgroup keeps its columns over the whole of K, walked through a ring of LDS stages.
// ROWS kernel (M <= 4; the built-in choice for M = 2): W streamed in whole rows on the vector ALU.
// Also here: attn_scores_kernel (Q.K^T for head dimensions up to 128, walking tiles; attn_scores_pipe_kernel: its two-deep
//              pipeline for head dimensions 80 and 96), attn_scores_rows_kernel (a handful
//              of query rows: a workgroup sweeps a run of the head's keys), attn_pv_rows_kernel (P.V for one or two query
//              rows) and attn_pv_whole_row_kernel (P.V for a few query rows: a workgroup sweeps the head's V, the keys
//              shared between workgroups when they are many).
#include "dtas_device.h"
#include "dtas_host.h"

#include <mutex>
#include <type_traits>

// Scratch memory of dtas_gemm_f16_static, the entry point that allocates nothing: arrival counters first, fp32
// partial tiles behind them.  Every device the library runs on holds its own copy of this array from the moment
// the code object is loaded until the process ends.  In host code the array's name is not a device address:
// resolve_static_scratch() asks the runtime for the address, once per device, and everything below uses that pointer.
static __device__ __align__(256) unsigned char scratch[DTAS_STATIC_SCRATCH_COUNTERS * 4 + DTAS_STATIC_SCRATCH_PARTIAL_BYTES];

namespace dtas {
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
};

// Attention scores, fused_NT_matmul1_divide_maximum_minimum_cast2 (before_dl.py:116-160):
// fp32(min(max(fp16(mm * fp16(scale)), -65504), mask)), mask = res1 shared by all heads.
constexpr int kEpiScores = 100;

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

// WT: W is given k-major ([K][N], N contiguous -- the V operand of attention's P.V); its tiles are
// then transposed on the way into the LDS (two stages, 4 wavefronts only).
// WQ: W is 8-bit with an fp16 scale per 32 elements of a row (Wq bytes [N][K], ep.wscale [N][K/32]); its
// tiles are dequantised on their way into the LDS by the same register path.
// M16: 8 wavefronts (256x256, 256x128, 128x256) on v_mfma_f32_16x16x32_f16 with one barrier per k tile (see the main loop).
template <int BM, int BN, int WM, int WN, int NS, bool WT = false, bool WQ = false, bool M16 = false>
__global__ void __launch_bounds__(64 * WM * WN) gemm_mfma_kernel(const half_t* __restrict__ A,
                                                                 const half_t* __restrict__ W,
                                                                 GemmEpilogue ep, void* __restrict__ C, int64_t M,
                                                                 int64_t N,
                                                                 int64_t K, unsigned tiles_m, unsigned tiles_n,
                                                                 unsigned nsplit, float* __restrict__ ws,
                                                                 unsigned* __restrict__ arrivals) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;  // wavefront tile
  constexpr int MT = WTM / 32, NT = WTN / 32;  // 32x32 blocks per wavefront
  constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;  // 1 KiB block loads per wavefront per k tile
  constexpr int kABytes = BM * kRowBytes, kStage = (BM + BN) * kRowBytes;
  static_assert(NW % 2 == 0 && LA >= 1 && LB >= 1 && MT >= 1 && NT >= 1, "tile / wavefront split");
  static_assert(NS >= 2 && NS <= 4 && (NW != 8 || NS == 2), "stage count");
  static_assert((NS - 1) * (LA + LB) <= 63, "outstanding loads must fit the vmcnt field");
  constexpr bool WREG = WT || WQ;  // W tiles pass through registers (transposed or dequantised), not the direct-to-LDS path
  static_assert(!WREG || (NS <= 3 && NW == 4), "the register W path is written for two or three stages and 4 wavefronts");
  static_assert(!(WT && WQ), "k-major 8-bit weights are not served");
  static_assert(M16 == (NW == 8) && (!M16 || !WREG), "8 wavefronts run the 16x16x32 loop, and only they");
  // 256x256 and every 8-wavefront tile: a ring of 5 operand units, each the larger operand's rows of a k tile
  constexpr bool kRing = BM + BN == 512 || M16;
  constexpr int kRingUnit = (BM > BN ? BM : BN) * kRowBytes;
  constexpr int kLdsAlloc = kRing ? 5 * kRingUnit : NS * kStage;
  static_assert(BM * BN * 2 <= kLdsAlloc, "epilogue staging must fit the operand stages");
  static_assert(kLdsAlloc <= kLdsBytes, "stages exceed the LDS");
  __shared__ __attribute__((aligned(1024))) char lds[kLdsAlloc];

  const unsigned t = threadIdx.x, l = t & 63u;
  const unsigned wv = __builtin_amdgcn_readfirstlane(t >> 6), wm = wv / WN, wn = wv % WN;

  // ---- which problem of a batched launch, which tile.  Workgroup ids are dealt round-robin over the
  // XCDs; xcd_contiguous_id gives each XCD a contiguous span of (problem, tile) instead, so the tiles of
  // one problem (which share its W -- the keys or values of an attention head) meet in one L2.
  // With ep.tiles_pinned (the scores: every problem reads the same mask) an XCD instead keeps one
  // span of tiles and walks the problems, so its part of the shared operand stays in its L2.
  // With ep.tiles_unsplit (one problem): the first tiles_unsplit tiles -- whole rounds of the chip -- are computed by
  // one workgroup each; only the tiles of the last, partly filled round are shared by nsplit workgroups, which are
  // launched after the whole ones.
  const unsigned total = tiles_m * tiles_n, unsplit = ep.tiles_unsplit;
  const unsigned per_batch = unsplit + (total - unsplit) * nsplit;
  // (divisions run on the vector ALU; pinning the results to scalar registers keeps every address
  // and buffer descriptor derived from them scalar -- a descriptor left in vector registers turns
  // each load into a loop over its distinct values)
  unsigned batch_u, wgid;
  bool whole = false;
  if (unsplit > 0) {
    batch_u = 0;
    whole = blockIdx.x < unsplit;
    wgid = whole ? xcd_contiguous_id(blockIdx.x, unsplit) : unsplit * nsplit + xcd_contiguous_id(blockIdx.x - unsplit, per_batch - unsplit);
  } else if (ep.tiles_pinned && per_batch % kNumXCD == 0) {
    const unsigned span = per_batch / kNumXCD, xcd = blockIdx.x % kNumXCD, local = blockIdx.x / kNumXCD;
    batch_u = __builtin_amdgcn_readfirstlane(local / span);
    wgid = xcd * span + local % span;
  } else {
    const unsigned gid = xcd_contiguous_id(blockIdx.x, per_batch * ep.batches);
    batch_u = __builtin_amdgcn_readfirstlane(gid / per_batch);
    wgid = gid - batch_u * per_batch;
  }
  const int64_t batch = batch_u;
  A += batch * ep.stride_a;
  W += batch * ep.stride_w;
  C = static_cast<char*>(C) + batch * ep.stride_c * (ep.out_f32 ? 4 : 2);
  if (ep.res1) ep.res1 += batch * ep.stride_res;
  if (ep.res2) ep.res2 += batch * ep.stride_res;

  // ---- tiles in groups of 8 tile rows walked column-wise
  // nsplit > 1: nsplit consecutive workgroups (same XCD) share a tile and split its k tiles
  const unsigned my_split = __builtin_amdgcn_readfirstlane(whole ? 1u : nsplit);
  const unsigned pid = __builtin_amdgcn_readfirstlane(whole ? wgid : wgid / nsplit), z = __builtin_amdgcn_readfirstlane(whole ? 0u : wgid % nsplit);
  constexpr unsigned kGroup = 8;
  const unsigned width = kGroup * tiles_n;
  const unsigned first_m = (pid / width) * kGroup;
  const unsigned gsize = tiles_m - first_m < kGroup ? tiles_m - first_m : kGroup;
  const unsigned tm = __builtin_amdgcn_readfirstlane(first_m + (pid % width) % gsize);
  const unsigned tn = __builtin_amdgcn_readfirstlane((pid % width) / gsize);
  const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;

  // ---- global side.  Lane p of a block load fills 16-byte slot p of the block, so it fetches
  // the (row, chunk) that lds_chunk_offset places there; the block index of wavefront w's i-th
  // load is i*NW + w, whose parity is w's (NW is even).
  const int64_t rows_a = M - m0 < BM ? M - m0 : BM, rows_w = N - n0 < BN ? N - n0 : BN;
  const int64_t lda = WT && ep.lda ? ep.lda : K;  // (with a row-major W both operands' rows are K long)
  const unsigned row_bytes = static_cast<unsigned>(lda) * 2u;
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(A + m0 * lda, static_cast<unsigned>(rows_a) * row_bytes);
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(W + n0 * K, static_cast<unsigned>(rows_w) * row_bytes);
  const unsigned r_in = 2u * (l >> 4) + (((l >> 3) & 1u) ^ (wv & 1u));  // row inside the 8-row block
  const unsigned c_in = (l & 7u) ^ r_in;                                // chunk of that row
  const unsigned g_off = (8u * wv + r_in) * row_bytes + c_in * 16u;
  const unsigned g_step = 8u * NW * row_bytes;

  // ---- LDS -> MFMA operands: lane l supplies row (l & 31), chunk 2*ks + (l >> 5)
  unsigned lds_rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) lds_rd[ks] = lds_chunk_offset(l & 31u, 2u * ks + (l >> 5));
  const unsigned a_base = wm * WTM * 128u, b_base = kABytes + wn * WTN * 128u;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  // M16: 16x16 blocks, 4 accumulator registers each
  constexpr int MT16 = M16 ? WTM / 16 : 1, NT16 = M16 ? WTN / 16 : 1;
  f32x4 acc16[MT16][NT16];
#pragma unroll
  for (int i = 0; i < MT16; ++i)
#pragma unroll
    for (int j = 0; j < NT16; ++j) acc16[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // this workgroup's k tiles: kt0 .. kt0 + ktiles - 1 of the matrix (none, if the split runs out)
  const int ktiles_all = static_cast<int>((K + kBK - 1) / kBK);
  const int kt_per = (ktiles_all + static_cast<int>(my_split) - 1) / static_cast<int>(my_split);
  const int kt0 = static_cast<int>(z) * kt_per;
  const int ktiles = ktiles_all - kt0 < kt_per ? (ktiles_all - kt0 > 0 ? ktiles_all - kt0 : 0) : kt_per;

  // tile kt -> LDS stage kt % NS, asynchronously (completion is counted by vmcnt)
  auto fetch = [&](int kt) {
    // a chunk past K is pointed out of range; K % 8 == 0, so chunks are all-in or all-out
    const unsigned off = (static_cast<int64_t>(kt0 + kt) * kBK + c_in * 8 < K)
                             ? g_off + static_cast<unsigned>(kt0 + kt) * kRowBytes : kOob;
    char* base = lds + (kt % NS) * kStage + wv * 1024;
    // (the block's row offset rides in the scalar offset operand: no vector add per load)
#pragma unroll
    for (int i = 0; i < LA; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + i * NW * 1024), 16, off, i * g_step, 0, 0);
    if constexpr (!WREG) {
#pragma unroll
      for (int i = 0; i < LB; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(base + kABytes + i * NW * 1024), 16, off, i * g_step, 0, 0);
    }
  };

  // ---- k-major W.  A tile is 64 k x BN columns of W[K][N]; an item is 8 columns of two
  // consecutive k rows: a lane loads the two 16-byte pieces into registers (wt_load, issued just
  // before the tile's A blocks) and later (wt_commit, once the tile is next in line) stores eight
  // 4-byte words {W[k][c], W[k+1][c]} to where the row-major path would have put them.  Item -> lane
  // is chosen so that a wavefront's 64 stores hit 64 distinct banks: 32 k pairs x 2 adjacent column
  // chunks.  The pieces come through buffer loads (out of range -> zeros), so every lane issues the
  // same number of loads per tile whatever its columns: the waits below count them.  Columns past N
  // are never written: the W parts of all stages are zeroed once, up front.
  // 8-bit W: an item is 16 weights of a row (16 bytes -> two 16-byte chunks of fp16) and their scale; lane
  // t takes piece t % 4 of row t / 4 (+ 64 rows per further item), so a wavefront reads 64 contiguous bytes
  // of each of 16 rows.  Every row of the tile is written every time (rows past N as zeros): nothing to clear.
  constexpr int kWtItems = WREG ? 4 * BN / (64 * NW) : 1;
  constexpr int kWtSlots = WREG ? NS - 1 : 1;  // register sets: one per tile in flight
  constexpr int kWtLoads = 2 * kWtItems;  // per lane and tile: k-major two pieces per item, 8-bit a piece and its scale
  u32x4 wt_reg[kWtSlots][kWtItems][WQ ? 1 : 2];
  unsigned short wq_scale[kWtSlots][kWtItems];
  const __amdgpu_buffer_rsrc_t rv = make_rsrc(W, WT ? static_cast<unsigned>(K * N * 2) : WQ ? static_cast<unsigned>(K * N) : 0u);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(ep.wscale, WQ ? static_cast<unsigned>((K / 32) * N * 2) : 0u);
  auto wt_item = [&](int i, unsigned& cc, unsigned& kp) {
    const unsigned item = t + i * 64 * NW;
    cc = ((item >> 6) << 1) | (item & 1u);
    kp = (item >> 1) & 31u;
  };
  auto wt_load = [&](int kt, auto slot_tag) {
    constexpr int SLOT = decltype(slot_tag)::value;
    if constexpr (WQ) {
#pragma unroll
      for (int i = 0; i < kWtItems; ++i) {
        const unsigned item = t + i * 64 * NW, r = item >> 2, c4 = item & 3u;
        const int64_t row = n0 + r, k = static_cast<int64_t>(kt0 + kt) * kBK + c4 * 16;
        const bool in = row < N && k < K;  // K % 32 == 0: a piece and its scale group are all-in or all-out
        wt_reg[SLOT][i][0] = __builtin_amdgcn_raw_buffer_load_b128(rv, in ? static_cast<unsigned>(row * K + k) : kOob, 0, 0);
        wq_scale[SLOT][i] = __builtin_amdgcn_raw_buffer_load_b16(rs, in ? static_cast<unsigned>((row * (K >> 5) + (k >> 5)) * 2) : kOob, 0, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < kWtItems; ++i) {
        unsigned cc, kp;
        wt_item(i, cc, kp);
        const int64_t col = n0 + cc * 8, k = static_cast<int64_t>(kt0 + kt) * kBK + 2 * kp;
        const unsigned at = static_cast<unsigned>((k * N + col) * 2), row = static_cast<unsigned>(N) * 2u;
        wt_reg[SLOT][i][0] = __builtin_amdgcn_raw_buffer_load_b128(rv, (col < N && k < K) ? at : kOob, 0, 0);
        wt_reg[SLOT][i][1] = __builtin_amdgcn_raw_buffer_load_b128(rv, (col < N && k + 1 < K) ? at + row : kOob, 0, 0);
      }
    }
  };
  auto wt_commit = [&](int kt, auto slot_tag) {
    constexpr int SLOT = decltype(slot_tag)::value;
    char* base = lds + (kt % NS) * kStage + kABytes;
    if constexpr (WQ) {
#pragma unroll
      for (int i = 0; i < kWtItems; ++i) {
        const unsigned item = t + i * 64 * NW, r = item >> 2, c4 = item & 3u;
        const half_t sc = __builtin_bit_cast(half_t, wq_scale[SLOT][i]);
        const f16x2 s2 = {sc, sc};
        u32x4 out[2];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          f16x2 lo, hi;
          const unsigned word = wt_reg[SLOT][i][0][w];
          dequant_q8_word(word, s2, lo, hi);
          out[w >> 1][(w & 1) * 2] = __builtin_bit_cast(unsigned, lo);
          out[w >> 1][(w & 1) * 2 + 1] = __builtin_bit_cast(unsigned, hi);
        }
        *reinterpret_cast<u32x4*>(base + lds_chunk_offset(r, 2 * c4)) = out[0];
        *reinterpret_cast<u32x4*>(base + lds_chunk_offset(r, 2 * c4 + 1)) = out[1];
      }
    } else {
#pragma unroll
      for (int i = 0; i < kWtItems; ++i) {
        unsigned cc, kp;
        wt_item(i, cc, kp);
        if (n0 + cc * 8 >= N) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned a = wt_reg[SLOT][i][0][j], b = wt_reg[SLOT][i][1][j];
          const unsigned r = cc * 8 + 2 * j;
          *reinterpret_cast<unsigned*>(base + lds_chunk_offset(r, kp >> 2) + (kp & 3u) * 4u) = (a & 0xffffu) | (b << 16);
          *reinterpret_cast<unsigned*>(base + lds_chunk_offset(r + 1, kp >> 2) + (kp & 3u) * 4u) = (a >> 16) | (b & 0xffff0000u);
        }
      }
    }
  };
  if constexpr (WT) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (int s = 0; s < NS; ++s)
      for (unsigned at = t * 16u; at < static_cast<unsigned>(BN * kRowBytes); at += 64 * NW * 16)
        *reinterpret_cast<u32x4*>(lds + s * kStage + kABytes + at) = zero;
    __syncthreads();
  }

  f16x8 fa[2][MT], fb[2][NT];
  auto read_a = [&](int set, int i, const char* stage, int ks) {
    fa[set][i] = *reinterpret_cast<const f16x8*>(stage + a_base + i * 4096 + lds_rd[ks]);
  };
  auto read_b = [&](int set, int j, const char* stage, int ks) {
    fb[set][j] = *reinterpret_cast<const f16x8*>(stage + b_base + j * 4096 + lds_rd[ks]);
  };
  // The MT*NT MFMAs of register set `set`, with the MT+NT fragment reads of the next step (from
  // `stage`, step `ks`, into the other set) spread evenly between them.  W rows are the first MFMA
  // operand, so a lane ends up with 4 consecutive columns of one C row per accumulator quad.
  auto step = [&](int set, const char* stage, int ks, bool reads) {
    constexpr int kReads = MT + NT, kMfma = MT * NT;
#pragma unroll
    for (int q = 0; q < kMfma; ++q) {
      if (reads) {
#pragma unroll
        for (int r = 0; r < kReads; ++r) {
          if (r * kMfma / kReads == q) {
            if (r < MT) read_a(set ^ 1, r, stage, ks); else read_b(set ^ 1, r - MT, stage, ks);
          }
        }
      }
      const int i = q / NT, j = q % NT;
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
      DTAS_SCHED_FENCE();
    }
  };

  if constexpr (WREG) {
    // ---- W through registers (k-major or 8-bit): NS stages, NS-1 tiles requested ahead (W pieces to registers, then the A blocks
    // to the LDS, so the loads of a tile are contiguous in the order they complete in).  This path
    // is bound by the bytes of A in flight, not by MFMA issue: loads go out in one burst per tile.
    constexpr int AH = NS - 1;
    constexpr int kTileLoads = LA + kWtLoads;  // per lane and tile
    static_assert((AH - 1) * kTileLoads <= 63, "outstanding loads must fit the vmcnt field");
    using Slot0 = std::integral_constant<int, 0>;
    using Slot1 = std::integral_constant<int, (AH > 1 ? 1 : 0)>;
    if (0 < ktiles) { wt_load(0, Slot0{}); fetch(0); }
    if (AH > 1 && 1 < ktiles) { wt_load(1, Slot1{}); fetch(1); }
    if (AH > 1 && 1 < ktiles) __builtin_amdgcn_s_waitcnt(waitcnt_imm(kTileLoads));
    else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
    if (0 < ktiles) wt_commit(0, Slot0{});
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the transposed words are in the LDS
    __builtin_amdgcn_s_barrier();
    DTAS_SCHED_FENCE();
    if (ktiles > 0) {
#pragma unroll
      for (int i = 0; i < MT; ++i) read_a(0, i, lds, 0);
#pragma unroll
      for (int j = 0; j < NT; ++j) read_b(0, j, lds, 0);
    }
    DTAS_SCHED_FENCE();
    // tile kt: its W sits in register slot kt % AH until committed, which frees the slot for tile kt + AH.
    // `steady`: tiles kt+1 .. kt+AH all exist -- no conditions in the body (a conditional load leaves the
    // compiler merging old and new register values, which it resolves with copies that wait for the loads)
    auto k_tile = [&](int kt, auto slot_tag, auto next_slot_tag, auto steady_tag) {
      constexpr bool kSteady = decltype(steady_tag)::value;
      const char* cur = lds + (kt % NS) * kStage;
      const char* nxt = lds + ((kt + 1) % NS) * kStage;
      if (kSteady || kt + AH < ktiles) {  // into the stage tile kt-1 occupied: free since the last barrier
        wt_load(kt + AH, slot_tag);
        fetch(kt + AH);
      }
      DTAS_SCHED_FENCE();
      step(0, cur, 1, true);
      step(1, cur, 2, true);
      step(0, cur, 3, true);
      if (kSteady || kt + 1 < ktiles) {
        // tile kt+1 must be complete; a tile requested after it may stay in flight
        if (AH > 1 && (kSteady || kt + 2 < ktiles)) __builtin_amdgcn_s_waitcnt(waitcnt_imm(kTileLoads));
        else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
        wt_commit(kt + 1, next_slot_tag);
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();        // tile kt+1 is whole, and every wavefront has finished reading tile kt
      DTAS_SCHED_FENCE();
      step(1, nxt, 0, kSteady || kt + 1 < ktiles);
    };
    int kt = 0;
    for (; kt + 2 * AH - 1 < ktiles; kt += AH) {  // the AH tiles of a round and the AH after them exist
      k_tile(kt, Slot0{}, Slot1{}, std::true_type{});
      if constexpr (AH > 1) k_tile(kt + 1, Slot1{}, Slot0{}, std::true_type{});
    }
    for (; kt < ktiles; kt += AH) {
      k_tile(kt, Slot0{}, Slot1{}, std::false_type{});
      if (AH > 1 && kt + 1 < ktiles) k_tile(kt + 1, Slot1{}, Slot0{}, std::false_type{});
    }
  } else if constexpr (M16) {
    // ---- 8 wavefronts, v_mfma_f32_16x16x32_f16, one barrier per k tile.
    // What the measurements on MI355X said, and what this loop is built around:
    //  * with random operands the card is power-limited, and the 16x16x32 instruction holds ~15 % more flops per
    //    watt than 32x32x16 (half the accumulator traffic per flop): 1.94 against 1.68 PFLOP/s for bare MFMA loops;
    //  * a wavefront that issues a direct-to-LDS load stalls until the texture addresser takes it (tens of
    //    cycles per instruction while data comes from the L2), and cannot issue its MFMAs behind it; of the two
    //    wavefronts of a SIMD the older one wins the MFMA pipe, so between two barriers w multiplies first and w+4
    //    second.  Each therefore issues its loads while the other one multiplies: w+4 (W units) right after the
    //    barrier, w (A units) after its own MFMAs;
    //  * loads are whole 128-byte lines (half lines cost the L2 path twice the requests), and the barrier sits
    //    where every wavefront holds all fragments of the tile in registers, so both units of tile kt are free
    //    from that barrier on.
    // The whole LDS is a ring of five 32 KiB operand units, A(0) W(0) A(1) W(1) A(2) ...: unit u sits in slot u % 5;
    // a k tile is two k32 steps.
    // (a 256x128 or 128x256 tile leaves half of every other slot unused)
    constexpr int kUnit = kRingUnit;
    constexpr int kLoadsA = BM / 32, kLoadsW = BN / 32;  // 1 KiB block loads per wavefront and unit
    static_assert(5 * kUnit <= kLdsAlloc && BM % 32 == 0 && BN % 32 == 0, "ring exceeds the LDS");
    auto wrap5 = [](int v) { return v >= 5 ? v - 5 : v; };
    const bool hi = wv >= 4;
    if (hi) __builtin_amdgcn_s_setprio(0); else __builtin_amdgcn_s_setprio(2);
    // wavefronts 0-3 load A units, 4-7 W units; block b (8 rows) of a unit goes to wavefront b % 4 of the group,
    // whose parity is the block's (the lane -> (row, chunk) map depends on it)
    const unsigned r16 = 2u * (l >> 4) + (((l >> 3) & 1u) ^ (wv & 1u));
    const unsigned c16 = (l & 7u) ^ r16;
    const unsigned g16 = (8u * (wv & 3u) + r16) * row_bytes + c16 * 16u;
    const unsigned g16_step = 32u * row_bytes;
    auto lane_off16 = [&](int kt) -> unsigned {
      return (static_cast<int64_t>(kt0 + kt) * kBK + c16 * 8 < K && kt < ktiles) ? g16 + static_cast<unsigned>(kt0 + kt) * kRowBytes : kOob;
    };
    auto fetch16 = [&](int slot, unsigned voff) {
      char* base = lds + slot * kUnit + (wv & 3u) * 1024;
      if (hi) {
#pragma unroll
        for (int q = 0; q < kLoadsW; ++q) __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(base + q * 4096), 16, voff, q * g16_step, 0, 0);
      } else {
#pragma unroll
        for (int q = 0; q < kLoadsA; ++q) __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + q * 4096), 16, voff, q * g16_step, 0, 0);
      }
    };
    // fragment of 16 rows x 32 k: lane l supplies row (l & 15) and the 8 k of lane group l >> 4.  Which chunk of the
    // step a lane group holds is free as long as both operands agree: groups 0..3 take chunks 0, 2, 1, 3, so that
    // lanes l and l + 32, which the LDS serves together, read neighbouring chunks -- the pairing the swizzle keeps
    // free of bank conflicts (chunks 0 and 2 of the same rows collide: measured, half of the LDS cycles)
    unsigned rd16[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) rd16[ks] = lds_chunk_offset(l & 15u, 4u * ks + (((l >> 4) & 1u) << 1 | (l >> 5)));
    const unsigned a_frag = wm * WTM * 128u, b_frag = wn * WTN * 128u;
    f16x8 ga[2][MT16], gb[2][NT16];
    if (hi) {
      fetch16(1, lane_off16(0));
      fetch16(3, lane_off16(1));
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(kLoadsW));
    } else {
      fetch16(0, lane_off16(0));
      fetch16(2, lane_off16(1));
      fetch16(4, lane_off16(2));
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * kLoadsA));
    }
    __builtin_amdgcn_s_barrier();
    DTAS_SCHED_FENCE();
#pragma unroll
    for (int j = 0; j < NT16; ++j) gb[0][j] = *reinterpret_cast<const f16x8*>(lds + kUnit + b_frag + j * 2048 + rd16[0]);
#pragma unroll
    for (int i = 0; i < MT16; ++i) ga[0][i] = *reinterpret_cast<const f16x8*>(lds + a_frag + i * 2048 + rd16[0]);
    DTAS_SCHED_FENCE();
    // the MFMAs of fragment set `set`; the fragment reads of (pa, pw, ks) into the other set, one before every
    // other MFMA (a burst of reads backs up the LDS queue, and the wavefront's MFMAs wait behind it)
    // (a 64x32 wavefront tile has 8 MFMAs for 6 reads: then one before every MFMA)
    constexpr int kReadEvery = 2 * (MT16 + NT16) <= MT16 * NT16 ? 2 : 1;
    auto step16 = [&](int set, const char* pa, const char* pw, int ks) {
      constexpr int kReads = MT16 + NT16;
#pragma unroll
      for (int i = 0; i < MT16; ++i)
#pragma unroll
        for (int j = 0; j < NT16; ++j) {
          const int q = i * NT16 + j;
          if (q % kReadEvery == 0 && q / kReadEvery < kReads) {
            const int r = q / kReadEvery;
            if (r < NT16) gb[set ^ 1][r] = *reinterpret_cast<const f16x8*>(pw + b_frag + r * 2048 + rd16[ks]);
            else ga[set ^ 1][r - NT16] = *reinterpret_cast<const f16x8*>(pa + a_frag + (r - NT16) * 2048 + rd16[ks]);
          }
          acc16[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(gb[set][j], ga[set][i], acc16[i][j], 0, 0, 0);
          DTAS_SCHED_FENCE();
        }
    };
    static_assert(kReadEvery * (MT16 + NT16) <= MT16 * NT16, "fragment reads must fit between the MFMAs of a step");
    int slot_a = 0, slot_w = 1;  // slots of A(kt), W(kt)
    for (int kt = 0; kt < ktiles; ++kt) {
      const char* pa = lds + slot_a * kUnit;
      const char* pw = lds + slot_w * kUnit;
      const int next_a = wrap5(slot_a + 2), next_w = wrap5(slot_w + 2);
      step16(0, pa, pw, 1);
      // wavefronts 0-3: A(kt+2) into the slot W(kt-1) left at the previous barrier
      if (!hi && kt > 0) fetch16(wrap5(slot_w + 3), lane_off16(kt + 2));
      // every fragment of tile kt is in registers and tile kt+1 has landed (0-3: all but the unit just requested)
      if (hi) __builtin_amdgcn_s_waitcnt(waitcnt_imm(0)); else __builtin_amdgcn_s_waitcnt(waitcnt_imm(kLoadsA));
      DTAS_SCHED_FENCE();
      __builtin_amdgcn_s_barrier();
      DTAS_SCHED_FENCE();
      if (hi) fetch16(slot_a, lane_off16(kt + 2));  // W(kt+2) into the slot of A(kt)
      DTAS_SCHED_FENCE();
      step16(1, lds + next_a * kUnit, lds + next_w * kUnit, 0);
      slot_a = next_a;
      slot_w = next_w;
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));  // (loads past the last tile are out of range: zeros, but they do write the LDS)
    __builtin_amdgcn_s_setprio(0);
  } else if constexpr (MT * NT == 16) {
    // ---- four wavefronts with 128x128 tiles each (256 accumulator registers): every k step reads
    // 8 KiB of fragments per wavefront for 16 MFMAs, two thirds of the LDS traffic per flop of the
    // 8-wavefront split -- the LDS port (fragment reads plus the direct-to-LDS writes) is what the
    // 8-wavefront kernel saturates.  One wavefront per SIMD has nobody to hide behind, so everything
    // is interleaved with the MFMAs of the running step: the next step's 8 fragment reads before its
    // first 8 MFMAs, 4 block loads between the last 8 (their per-lane offset is computed once per
    // k tile, the block's offset rides in the scalar offset operand).  Same ring of five operand units.
    static_assert(BM == BN && NW == 4, "ring units are one operand's rows of a k tile");
    constexpr int kUnit = BM * kRowBytes;
    static_assert(5 * kUnit <= kLdsAlloc && LA % 2 == 0 && 8 % (LA / 2) == 0, "ring exceeds the LDS");
    constexpr int kHalf = LA / 2;  // block loads per wavefront and half unit
    auto wrap5 = [](int v) { return v >= 5 ? v - 5 : v; };
    const unsigned a_frag = wm * WTM * 128u, b_frag = wn * WTN * 128u;
    // per-lane byte offset of this lane's chunk in k tile kt of either operand (out of range past K)
    auto lane_off = [&](int kt) -> unsigned {
      return (static_cast<int64_t>(kt0 + kt) * kBK + c_in * 8 < K) ? g_off + static_cast<unsigned>(kt0 + kt) * kRowBytes : kOob;
    };
    // block load b of a unit (the descriptor is named here, not passed down through the lambdas)
    auto fetch_one = [&](bool is_w, unsigned voff, int slot, int b) {
      lds_ptr_t dst = (lds_ptr_t)(lds + slot * kUnit + wv * 1024 + b * NW * 1024);
      if (is_w) __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, dst, 16, voff, b * g_step, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, dst, 16, voff, b * g_step, 0, 0);
    };
    // MFMAs of register set `set`; reads of step `ks_next` of (pa, pw) into the other set; half `dpart`
    // of a unit's loads.  DMA: 0 = none, 1 = always, 2 = if `cond`.
    auto step4 = [&](int set, const char* pa, const char* pw, int ks_next, bool reads, int dma, bool cond, bool is_w,
                     unsigned voff, int dslot, int dpart) {
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        if (reads && q < 8) {
          if (q < 4) fa[set ^ 1][q] = *reinterpret_cast<const f16x8*>(pa + q * 4096 + lds_rd[ks_next]);
          else fb[set ^ 1][q - 4] = *reinterpret_cast<const f16x8*>(pw + (q - 4) * 4096 + lds_rd[ks_next]);
        }
        const int i = q / 4, j = q % 4;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
        if (dma != 0 && q >= 8 && (q - 8) % (8 / kHalf) == 0) {
          if (dma == 1 || cond) fetch_one(is_w, voff, dslot, dpart * kHalf + (q - 8) / (8 / kHalf));
        }
        DTAS_SCHED_FENCE();
      }
    };
    if (ktiles > 0) {
      const unsigned v0 = lane_off(0);
#pragma unroll
      for (int b = 0; b < LA; ++b) fetch_one(false, v0, 0, b);
#pragma unroll
      for (int b = 0; b < LA; ++b) fetch_one(true, v0, 1, b);
    }
    if (ktiles > 1) {
      const unsigned v1 = lane_off(1);
#pragma unroll
      for (int b = 0; b < LA; ++b) fetch_one(false, v1, 2, b);
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(LA));
    } else {
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
    }
    __builtin_amdgcn_s_barrier();
    DTAS_SCHED_FENCE();
    if (ktiles > 0) {
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[0][i] = *reinterpret_cast<const f16x8*>(lds + a_frag + i * 4096 + lds_rd[0]);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb[0][j] = *reinterpret_cast<const f16x8*>(lds + kUnit + b_frag + j * 4096 + lds_rd[0]);
    }
    DTAS_SCHED_FENCE();
    int slot_a = 0, slot_w = 1;  // slots of A(kt) and W(kt)
    // one k tile; `steady`: tiles kt+1 and kt+2 exist (no conditions in the instruction stream)
    auto k_tile = [&](int kt, bool steady) {
      const char* pa = lds + slot_a * kUnit + a_frag;
      const char* pw = lds + slot_w * kUnit + b_frag;
      const int next_a = wrap5(slot_a + 2), next_w = wrap5(slot_w + 2), far_a = wrap5(slot_a + 4);
      const bool w1 = kt + 1 < ktiles, a2 = kt + 2 < ktiles;
      const int mode = steady ? 1 : 2;
      const unsigned vw = lane_off(kt + 1), va = lane_off(kt + 2);
      // W(kt+1) goes where A(kt-1) was, A(kt+2) where W(kt-1) was: free since the previous barrier
      step4(0, pa, pw, 1, true, mode, w1, true, vw, next_w, 0);
      step4(1, pa, pw, 2, true, mode, w1, true, vw, next_w, 1);
      step4(0, pa, pw, 3, true, mode, a2, false, va, far_a, 0);
      // tile kt+1 has landed: everything but the half unit of A(kt+2) just requested
      if (steady || a2) __builtin_amdgcn_s_waitcnt(waitcnt_imm(kHalf)); else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
      __builtin_amdgcn_s_barrier();  // ... for every wavefront, and all of them are done reading tile kt
      DTAS_SCHED_FENCE();
      step4(1, lds + next_a * kUnit + a_frag, lds + next_w * kUnit + b_frag, 0, steady || w1, mode, a2, false, va, far_a, 1);
      slot_a = next_a;
      slot_w = next_w;
    };
    int kt = 0;
    for (; kt + 2 < ktiles; ++kt) k_tile(kt, true);
    for (; kt < ktiles; ++kt) k_tile(kt, false);
  } else if constexpr (NS >= 3) {
    // ---- NS >= 3 whole-tile stages, for grids with about one workgroup (one wavefront per SIMD) per
    // CU: nothing hides a burst of loads or a run of scalar bookkeeping, so the kL block loads of a
    // tile are issued in four parts between the MFMAs of four consecutive steps (part 0 right after
    // the barrier that frees the stage, parts 1-3 in the next tile's first three steps), with their
    // per-lane offset computed once and the block offsets in the scalar operand; the steady-state
    // loop carries no conditions.
    constexpr int kL = LA + LB;
    auto lane_off = [&](int kt) -> unsigned {
      return (static_cast<int64_t>(kt0 + kt) * kBK + c_in * 8 < K) ? g_off + static_cast<unsigned>(kt0 + kt) * kRowBytes : kOob;
    };
    // block load l (0 .. kL-1: A blocks, then W blocks) of a tile into `stage`
    auto fetch_one = [&](int l_, unsigned voff, char* stage) {
      if (l_ < LA)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(stage + wv * 1024 + l_ * NW * 1024), 16, voff, l_ * g_step, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(stage + kABytes + wv * 1024 + (l_ - LA) * NW * 1024), 16, voff,
                                                 (l_ - LA) * g_step, 0, 0);
    };
    // MFMAs of `set`, the next step's fragment reads, and part `part` of a tile's loads (if `dma`)
    auto step_dma = [&](int set, const char* stage, int ks, bool reads, bool dma, int part, unsigned voff, char* dst) {
      constexpr int kReads = MT + NT, kMfma = MT * NT;
#pragma unroll
      for (int q = 0; q < kMfma; ++q) {
        if (reads) {
#pragma unroll
          for (int r = 0; r < kReads; ++r)
            if (r * kMfma / kReads == q) {
              if (r < MT) read_a(set ^ 1, r, stage, ks); else read_b(set ^ 1, r - MT, stage, ks);
            }
        }
        const int i = q / NT, j = q % NT;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
        if (dma) {
          // loads part*kL/4 .. (part+1)*kL/4 - 1, spread over the step's MFMAs
          const int lo = part * kL / 4, hi = (part + 1) * kL / 4;
#pragma unroll
          for (int l_ = 0; l_ < kL; ++l_)
            if (l_ >= lo && l_ < hi && (l_ - lo) * kMfma / (hi - lo) == q) fetch_one(l_, voff, dst);
        }
        DTAS_SCHED_FENCE();
      }
    };
    // every stage is free: tile 0, tiles 1 .. NS-2 whole and part 0 of tile NS-1 are requested together, and only
    // tile 0 is waited for (loads complete in order: whole tiles requested after it may stay outstanding)
    if (ktiles > 0) {
      const unsigned v0 = lane_off(0);
#pragma unroll
      for (int l_ = 0; l_ < kL; ++l_) fetch_one(l_, v0, lds);
    }
#pragma unroll
    for (int p = 1; p < NS; ++p) {
      if (p < ktiles) {
        const unsigned vp = lane_off(p);
#pragma unroll
        for (int l_ = 0; l_ < (p < NS - 1 ? kL : kL / 4); ++l_) fetch_one(l_, vp, lds + p * kStage);
      }
    }
    wait_whole_tiles<kL, NS - 2>(ktiles - 1);
    __builtin_amdgcn_s_barrier();
    DTAS_SCHED_FENCE();
    if (ktiles > 0) {
#pragma unroll
      for (int i = 0; i < MT; ++i) read_a(0, i, lds, 0);
#pragma unroll
      for (int j = 0; j < NT; ++j) read_b(0, j, lds, 0);
    }
    DTAS_SCHED_FENCE();
    int cur_s = 0;  // stage of tile kt
    auto wrap = [](int v) { return v >= NS ? v - NS : v; };
    auto k_tile = [&](int kt, bool steady) {
      char* cur = lds + cur_s * kStage;
      char* nxt = lds + wrap(cur_s + 1) * kStage;
      char* late = lds + wrap(cur_s + NS - 1) * kStage;  // stage of tile kt-1 = of tile kt+NS-1
      const bool have_late = steady || kt + NS - 1 < ktiles, have_new = steady || kt + NS < ktiles;
      const unsigned v_late = lane_off(kt + NS - 1), v_new = lane_off(kt + NS);
      step_dma(0, cur, 1, true, have_late, 1, v_late, late);
      step_dma(1, cur, 2, true, have_late, 2, v_late, late);
      step_dma(0, cur, 3, true, have_late, 3, v_late, late);
      // tile kt+1 must have landed; later tiles (at most NS-2 of them) may stay in flight.  Loads
      // complete in order, so it is enough to allow that many tiles' worth of loads outstanding.
      if (steady) {
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 2) * kL));
      } else {
        wait_whole_tiles<kL, NS - 2>(ktiles - 2 - kt);  // tiles after kt+1 that have been requested
      }
      __builtin_amdgcn_s_barrier();  // ... and every wavefront has finished reading tile kt
      DTAS_SCHED_FENCE();
      step_dma(1, nxt, 0, steady || kt + 1 < ktiles, have_new, 0, v_new, cur);
      cur_s = wrap(cur_s + 1);
    };
    static_assert((NS - 2) * kL <= 63, "outstanding loads must fit the vmcnt field");
    int kt = 0;
    for (; kt + NS < ktiles; ++kt) k_tile(kt, true);
    for (; kt < ktiles; ++kt) k_tile(kt, false);
  } else {
  // two stages: tile 0 resident, tile 1 in flight, fragments of (tile 0, step 0) in registers
  // (row-major W: tile 1 is requested together with tile 0 -- both stages are free -- and only tile 0
  // is waited for; with two k tiles in all, as in the attention scores, that is one round trip less)
  if (ktiles > 0) fetch(0);
  if (1 < ktiles) {
    fetch(1);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(LA + LB));  // tile 1's loads may stay outstanding
  } else {
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  }
  __builtin_amdgcn_s_barrier();
  DTAS_SCHED_FENCE();
  if (ktiles > 0) {
#pragma unroll
    for (int i = 0; i < MT; ++i) read_a(0, i, lds, 0);
#pragma unroll
    for (int j = 0; j < NT; ++j) read_b(0, j, lds, 0);
  }
  DTAS_SCHED_FENCE();
  for (int kt = 0; kt < ktiles; ++kt) {
    const char* cur = lds + (kt % NS) * kStage;
    const char* nxt = lds + ((kt + 1) % NS) * kStage;
    step(0, cur, 1, true);
    step(1, cur, 2, true);
    step(0, cur, 3, true);
    __builtin_amdgcn_s_waitcnt(0x0070);  // tile kt+1 has landed
    __builtin_amdgcn_s_barrier();        // ... and every wavefront has finished reading tile kt
    DTAS_SCHED_FENCE();
    if (kt + NS < ktiles) fetch(kt + NS);  // into the stage tile kt occupied
    DTAS_SCHED_FENCE();
    step(1, nxt, 0, kt + 1 < ktiles);
  }
  }

  // ---- epilogue.  acc[i][j][v] of lane l is C row i*32 + (l & 31), column
  // j*32 + 8*(v/4) + 4*(l >> 5) + v%4 of the wavefront tile.  Each wavefront stages its tile in a
  // private LDS region of WTM rows x WTN fp16 (8-byte slots, xor-swizzled by the row) and writes
  // it out as 8-byte accesses that are contiguous along the row.
  // ---- split K: every workgroup of a tile parks its fp32 partial tile in the workspace (in
  // accumulator layout: 8 bytes per lane and register pair, lane-contiguous); the one that arrives
  // last adds the nsplit partials in split order, so the sum does not depend on who was last, and
  // goes on to the epilogue.  Nobody waits for anybody.
  // The XCDs' L2 caches are not coherent with each other.  Partials and the arrival counter are
  // therefore moved with device-scope accesses (they pass the L2), ordered by explicit waits for the
  // store count plus the barriers, rather than with device-scope fences, which write back and
  // invalidate a whole L2 on every use (measured: that made a two-way split slower than no split).
  if constexpr (WT) {
    // the last k_tail k: 16-byte pieces of A's rows end at K (a piece across the end of a row would bring in the next
    // row's elements), so these few products are added here, element by element, in fp32
    if (ep.k_tail > 0 && z == 0) {
      const int64_t lda_t = ep.lda ? ep.lda : K;
      // kTB k at a time (four; two on the small tiles, whose register count decides how many workgroups a CU holds), every
      // element of A and piece of W requested before the first is used: one round trip to memory per kTB k instead of one per k
      constexpr int kTB = MT * NT >= 4 ? 4 : 2;
      for (unsigned e0 = 0; e0 < ep.k_tail; e0 += kTB) {
        half_t pa[kTB][MT];
        f16x4 vv[kTB][NT][4];
        const half_t hz = static_cast<half_t>(0.f);
#pragma unroll
        for (int e = 0; e < kTB; ++e) {
          const bool k_in = e0 + e < ep.k_tail;
#pragma unroll
          for (int i = 0; i < MT; ++i) {
            const int64_t row = m0 + wm * WTM + i * 32 + (l & 31u);
            pa[e][i] = k_in && row < M ? A[row * lda_t + K + e0 + e] : hz;
          }
          const half_t* vrow = W + (K + e0 + e) * N;
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const int64_t col = n0 + wn * WTN + j * 32 + 8 * g + 4 * (l >> 5);
              const f16x4 none = {hz, hz, hz, hz};
              vv[e][j][g] = k_in && col < N ? *reinterpret_cast<const f16x4*>(vrow + col) : none;  // (N % 8 == 0: four columns are all-in or all-out)
            }
        }
#pragma unroll
        for (int e = 0; e < kTB; ++e)
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
              for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[i][j][g * 4 + c] += static_cast<float>(pa[e][i]) * static_cast<float>(vv[e][j][g][c]);
      }
    }
  }
  if (my_split > 1) {
    // (the flag lives in the operand stages, free by now: a second LDS object would make the
    // compiler order every fragment read behind the outstanding direct-to-LDS loads)
    volatile unsigned* is_last = reinterpret_cast<volatile unsigned*>(lds);
    constexpr int kTilePairs = BM * BN / 2;  // 8-byte units per partial tile
    const unsigned tile_g = batch_u * total + pid - unsplit;  // this tile among all problems' tiles
    unsigned long long* tile_ws = reinterpret_cast<unsigned long long*>(ws) + static_cast<size_t>(tile_g) * nsplit * kTilePairs;
    unsigned long long* mine = tile_ws + static_cast<size_t>(z) * kTilePairs + wv * (MT * NT * 8 * 64);
    // pair q of a lane's accumulators (in whatever order the main loop keeps them)
    constexpr int kPer = MT * NT * 8;  // 8-byte units per lane and partial tile
    auto pair_get = [&](int q, int e) -> float {
      if constexpr (M16) return acc16[q / (NT16 * 2)][(q / 2) % NT16][2 * (q % 2) + e];
      else return acc[q / (NT * 8)][(q / 8) % NT][2 * (q % 8) + e];
    };
    auto pair_set = [&](int q, int e, float v) {
      if constexpr (M16) acc16[q / (NT16 * 2)][(q / 2) % NT16][2 * (q % 2) + e] = v;
      else acc[q / (NT * 8)][(q / 8) % NT][2 * (q % 8) + e] = v;
    };
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
      const f32x2v pr = {pair_get(q, 0), pair_get(q, 1)};
      __hip_atomic_store(mine + q * 64 + l, __builtin_bit_cast(unsigned long long, pr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // The partials are device-scope stores (write-through): once a wavefront's store count has drained they are
    // visible to every XCD.  The barrier alone does not wait for that (a workgroup-scope barrier lets stores stay
    // in flight), and the counter below must not be seen before the partials it announces.
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
    __syncthreads();  // every store of this workgroup has completed; nobody reads the stages any more
    if (t == 0) {
      const unsigned before = __hip_atomic_fetch_add(arrivals + tile_g, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *is_last = before == my_split - 1 ? 1u : 0u;
      if (before == my_split - 1)  // re-armed for the next launch
        __hip_atomic_store(arrivals + tile_g, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const bool last = *is_last != 0;
    if (!last) return;
    // The sum is p0 + p1 + ... in split order whoever arrived last.  The last arriver's own partial is still in its
    // registers: as split 0 it is the first term, and of two splits the sum is the same in either order (a + b = b + a
    // exactly) -- then only the others' partials are read back; otherwise all of them, from zero.
    const bool keep_own = z == 0 || my_split == 2;
    if (!keep_own) {
#pragma unroll
      for (int q = 0; q < kPer; ++q) {
        pair_set(q, 0, 0.f);
        pair_set(q, 1, 0.f);
      }
    }
    // The partials are added in split order, but requested kGroup tiles at a time (up to 64 loads per lane):
    // one tile per round trip made the combine cost ~1.2 us per split, which capped useful splits at 4.
    constexpr int kGroup = kPer >= 64 ? 1 : 64 / kPer;
    auto add_partials = [&](unsigned k0, auto count_tag) {
      constexpr int COUNT = decltype(count_tag)::value;
      unsigned long long raw[COUNT][kPer];
#pragma unroll
      for (int g = 0; g < COUNT; ++g) {
        const unsigned long long* part = tile_ws + static_cast<size_t>(k0 + g) * kTilePairs + wv * (kPer * 64);
#pragma unroll
        for (int q = 0; q < kPer; ++q)
          raw[g][q] = __hip_atomic_load(part + q * 64 + l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
#pragma unroll
      for (int g = 0; g < COUNT; ++g)
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
          const f32x2v pr = __builtin_bit_cast(f32x2v, raw[g][q]);
          pair_set(q, 0, pair_get(q, 0) + pr[0]);
          pair_set(q, 1, pair_get(q, 1) + pr[1]);
        }
    };
    unsigned k = keep_own && z == 0 ? 1u : 0u;
    const unsigned k_end = keep_own && z != 0 ? 1u : my_split;  // (two splits, the second one last: p0 alone)
    for (; k + kGroup <= k_end; k += kGroup) add_partials(k, std::integral_constant<int, kGroup>{});
    for (; k < k_end; ++k) add_partials(k, std::integral_constant<int, 1>{});
  }

  // The sums go through the LDS so that the stores are whole rows of the wavefront tile: staged as 8-byte slots of
  // 4 columns (what a lane holds), read back kVecC columns per lane.  With 8 wavefronts a lane takes 16 bytes: half
  // the store instructions for the same lines.
  constexpr int kVecC = M16 ? 8 : 4;
  constexpr int kSlots = WTN / 4, kLaneSlots = WTN / kVecC, kRowB = WTN * 2, kRowsPerPass = 64 / kLaneSlots;
  using cvec_t = std::conditional_t<kVecC == 8, f16x8, f16x4>;
  typedef cvec_t __attribute__((aligned(2))) cvec_a2;
  // staging offset of 8-byte slot `s` of row m: the xor keeps a wavefront's writes (16 or 32 rows of one slot) and
  // its reads (whole rows) on distinct banks; with 16-byte reads it leaves slot pairs together
  auto stage_off = [](unsigned m, unsigned s) -> unsigned {
    const unsigned x = M16 ? ((m >> 1) & (kSlots / 2 - 1)) << 1 : m & (kSlots - 1);
    return m * kRowB + ((s ^ x) * 8);
  };
  char* region = lds + wv * (WTM * kRowB);
  __syncthreads();  // every wavefront is done with the operand stages
  if constexpr (M16) {
    // acc16[i][j][v] of lane l is C row i*16 + (l & 15), column j*16 + 4*(l >> 4) + v of the wavefront tile
#pragma unroll
    for (int i = 0; i < MT16; ++i) {
      const unsigned m = i * 16 + (l & 15u);
#pragma unroll
      for (int j = 0; j < NT16; ++j) {
        f16x4 hv;
#pragma unroll
        for (int e = 0; e < 4; ++e) hv[e] = static_cast<half_t>(acc16[i][j][e]);
        *reinterpret_cast<f16x4*>(region + stage_off(m, j * 4 + (l >> 4))) = hv;
      }
    }
  } else {
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const unsigned m = i * 32 + (l & 31u);
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f16x4 hv;
#pragma unroll
        for (int e = 0; e < 4; ++e) hv[e] = static_cast<half_t>(acc[i][j][g * 4 + e]);
        *reinterpret_cast<f16x4*>(region + stage_off(m, j * 8 + g * 2 + (l >> 5))) = hv;
      }
  }
  }
  // no barrier: a wavefront reads back only what it wrote itself
  const unsigned slot = l % kLaneSlots, rsub = l / kLaneSlots;
  const int64_t col = n0 + wn * WTN + slot * kVecC;
  // one access per lane to C and the residuals for every lane whose columns lie inside the row, at whatever
  // alignment the row has
  const bool vec_store = col + kVecC - 1 < N;
  float bv[kVecC];
  cvec_t bvh;
#pragma unroll
  for (int e = 0; e < kVecC; ++e) {
    bvh[e] = ep.bias && col + e < N ? ep.bias[col + e] : static_cast<half_t>(0.f);
    bv[e] = static_cast<float>(bvh[e]);
  }
  // one store loop per epilogue kind, chosen once (kind is uniform)
  auto store_tile = [&](auto kind_tag) {
    constexpr int KIND = decltype(kind_tag)::value;
    constexpr bool kAdd2 = KIND == DTAS_EPI_BIAS_ADD2 || KIND == DTAS_EPI_BIAS_ADD2_CAST_F32;
    constexpr bool kUseR1 = kAdd2 || KIND == kEpiScores;
    constexpr bool kOutF32 = KIND == DTAS_EPI_BIAS_ADD2_CAST_F32 || KIND == kEpiScores;
    const bool has_bias = ep.bias != nullptr;
    // passes in groups of G: the group's residual / mask vectors are requested together, before the
    // first of them is needed (one at a time, every pass would wait out a memory round trip)
    constexpr int kPasses = WTM / kRowsPerPass;
    // as many as the registers hold (kVecC / 2 per vector): 128 registers for one operand, 64 each for two
    constexpr int kWant = (KIND == DTAS_EPI_BIAS_GELU ? 16 : kAdd2 ? 64 : kUseR1 ? 128 : 16) / kVecC;
    constexpr int G = kPasses <= kWant ? kPasses : kPasses % kWant == 0 ? kWant : (kPasses % 8 == 0 && kWant >= 8 ? 8 : (kPasses % 4 == 0 && kWant >= 4 ? 4 : 1));
#pragma unroll 1
    for (int p0 = 0; p0 < kPasses; p0 += G) {
      cvec_t r1v[G] = {}, r2v[G] = {};
      if (kUseR1) {
#pragma unroll
        for (int u = 0; u < G; ++u) {
          const int64_t row = m0 + wm * WTM + (p0 + u) * kRowsPerPass + rsub;
          if (row >= M) continue;
          const int64_t at = row * N + col;
          if (vec_store) {
            r1v[u] = *reinterpret_cast<const cvec_a2*>(ep.res1 + at);
            if (kAdd2) r2v[u] = *reinterpret_cast<const cvec_a2*>(ep.res2 + at);
          } else {
#pragma unroll
            for (int e = 0; e < kVecC; ++e)
              if (col + e < N) {
                r1v[u][e] = ep.res1[at + e];
                if (kAdd2) r2v[u][e] = ep.res2[at + e];
              }
          }
        }
      }
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const unsigned m = (p0 + u) * kRowsPerPass + rsub;
        cvec_t hv = *reinterpret_cast<const cvec_t*>(region + stage_off(m, slot * (kVecC / 4)));
        const int64_t row = m0 + wm * WTM + m;
        if (row >= M) continue;
        const int64_t at = row * N + col;
        if constexpr (KIND == DTAS_EPI_BIAS_GELU) {
          hv = gelu_erf_f16_steps_vec<cvec_t, kVecC>(hv, has_bias, bvh);
        } else if constexpr (KIND == DTAS_EPI_BIAS || kAdd2) {
          // "+ bias", "+ residual" act on the sum already rounded to fp16, each step rounded to fp16: as packed fp16
          // additions (an fp16 sum rounded once is what the step computed through fp32 and rounded gives: the same bits)
          hv = add_steps_vec<cvec_t, kAdd2>(hv, has_bias, bvh, r1v[u], r2v[u]);
        } else if constexpr (KIND == kEpiScores) {
#pragma unroll
          for (int h4 = 0; h4 < kVecC / 4; ++h4) {
            const f16x4 part = scores_steps_vec(f16x4{hv[4 * h4], hv[4 * h4 + 1], hv[4 * h4 + 2], hv[4 * h4 + 3]}, ep.scale,
                                                f16x4{r1v[u][4 * h4], r1v[u][4 * h4 + 1], r1v[u][4 * h4 + 2], r1v[u][4 * h4 + 3]});
#pragma unroll
            for (int e = 0; e < 4; ++e) hv[4 * h4 + e] = part[e];
          }
        } else {
#pragma unroll
          for (int e = 0; e < kVecC; ++e)
            hv[e] = epilogue_value_k<KIND>(hv[e], has_bias, ep.scale, bv[e], static_cast<float>(r1v[u][e]),
                                           static_cast<float>(r2v[u][e]));
        }
        if (kOutF32) {
          float* dst = static_cast<float*>(C) + at;
          if (vec_store) {
            // 4*heads*n*m bytes of scores: streamed (rows of whole sectors)
            const bool stream = KIND == kEpiScores && N % 16 == 0 && (reinterpret_cast<uintptr_t>(C) & 63u) == 0;
#pragma unroll
            for (int h = 0; h < kVecC / 4; ++h) {
              const f32x4v wide = {static_cast<float>(hv[4 * h]), static_cast<float>(hv[4 * h + 1]), static_cast<float>(hv[4 * h + 2]),
                                   static_cast<float>(hv[4 * h + 3])};
              if (stream) __builtin_nontemporal_store(wide, reinterpret_cast<f32x4v*>(dst + 4 * h));
              else *reinterpret_cast<f32x4v_a4*>(dst + 4 * h) = wide;
            }
          } else {
#pragma unroll
            for (int e = 0; e < kVecC; ++e)
              if (col + e < N) dst[e] = static_cast<float>(hv[e]);
          }
        } else {
          half_t* dst = static_cast<half_t*>(C) + at;
          if (vec_store) {
            *reinterpret_cast<cvec_a2*>(dst) = hv;
          } else {
#pragma unroll
            for (int e = 0; e < kVecC; ++e)
              if (col + e < N) dst[e] = hv[e];
          }
        }
      }
    }
  };
  switch (ep.kind) {
    case DTAS_EPI_BIAS_ADD2: store_tile(std::integral_constant<int, DTAS_EPI_BIAS_ADD2>{}); break;
    case DTAS_EPI_BIAS_ADD2_CAST_F32: store_tile(std::integral_constant<int, DTAS_EPI_BIAS_ADD2_CAST_F32>{}); break;
    case DTAS_EPI_BIAS_GELU: store_tile(std::integral_constant<int, DTAS_EPI_BIAS_GELU>{}); break;
    case kEpiScores: store_tile(std::integral_constant<int, kEpiScores>{}); break;
    default: store_tile(std::integral_constant<int, DTAS_EPI_BIAS>{}); break;
  }
}

// Attention scores for head dimensions up to 128 (two k tiles): out[h] = epilogue(Q[h] . K[h]^T).
// What the op moves is its fp32 output, and a workgroup of the general kernel lives mostly in two
// waits -- for its operands, then for its stores to drain -- while its LDS keeps further workgroups
// off the CU.  Here a workgroup walks tiles (stride = grid): it requests the whole Q and K tiles and
// its part of the mask at once, multiplies, stages the result through the LDS and issues the stores;
// the next tile's loads are then in flight together with those stores.  Tiles are numbered as the
// batched launches of gemm_mfma_kernel number their workgroups; with `pinned` an XCD keeps one span of
// tiles (spans differ by at most one tile) and walks the heads, so its part of the mask stays in its L2.
// Operand layout in the LDS as there.
template <int BM, int BN>
__global__ void __launch_bounds__(256) attn_scores_kernel(const half_t* __restrict__ Q, const half_t* __restrict__ Kmat,
                                                          const half_t* __restrict__ mask, float* __restrict__ out,
                                                          int64_t n, int64_t m, int64_t d, float scale, unsigned tiles_m,
                                                          unsigned tiles_n, unsigned heads, unsigned pinned) {
  constexpr int NW = 4, WN = 2, WTM = BM / 2, WTN = BN / 2, MT = WTM / 32, NT = WTN / 32;
  constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;
  constexpr int kABytes = BM * kRowBytes, kStage = (BM + BN) * kRowBytes;
  static_assert(BM * BN * 2 <= 2 * kStage, "epilogue staging must fit the operand tiles");
  __shared__ __attribute__((aligned(1024))) char lds[2 * kStage];

  const unsigned t = threadIdx.x, l = t & 63u;
  const unsigned wv = __builtin_amdgcn_readfirstlane(t >> 6), wm = wv / WN, wn = wv % WN;
  const int ktiles = static_cast<int>((d + kBK - 1) / kBK);  // 1 or 2
  const unsigned row_bytes = static_cast<unsigned>(d) * 2u;
  const unsigned r_in = 2u * (l >> 4) + (((l >> 3) & 1u) ^ (wv & 1u));
  const unsigned c_in = (l & 7u) ^ r_in;
  const unsigned g_off = (8u * wv + r_in) * row_bytes + c_in * 16u;
  const unsigned g_step = 8u * NW * row_bytes;
  unsigned lds_rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) lds_rd[ks] = lds_chunk_offset(l & 31u, 2u * ks + (l >> 5));
  const unsigned a_base = wm * WTM * 128u, b_base = kABytes + wn * WTN * 128u;

  constexpr int kSlots = WTN / 4, kRowB = WTN * 2, kRowsPerPass = 64 / kSlots, kPasses = WTM / kRowsPerPass;
  const unsigned slot = l % kSlots, rsub = l / kSlots;
  char* region = lds + wv * (WTM * kRowB);
  const bool ptr_ok = true;  // rows of any length: vector accesses at the rows' own alignment
  const bool stream_out = m % 16 == 0 && (reinterpret_cast<uintptr_t>(out) & 63u) == 0;  // (then every access is 16-byte aligned)

  const unsigned per_batch = tiles_m * tiles_n, total = per_batch * heads;
  const unsigned span_base = per_batch / kNumXCD, span_rem = per_batch % kNumXCD;
  const unsigned walk_end = pinned ? kNumXCD * heads * (span_base + (span_rem ? 1u : 0u)) : total;
  for (unsigned tix = blockIdx.x; tix < walk_end; tix += gridDim.x) {
    unsigned batch, pid;
    if (pinned) {
      const unsigned xcd = tix % kNumXCD, local = tix / kNumXCD;
      const unsigned span = span_base + (xcd < span_rem ? 1u : 0u), first = xcd * span_base + (xcd < span_rem ? xcd : span_rem);
      if (local >= span * heads) continue;  // (the shorter spans end earlier; uniform over the workgroup)
      batch = __builtin_amdgcn_readfirstlane(local / span);
      pid = __builtin_amdgcn_readfirstlane(first + local % span);
    } else {
      const unsigned gid = xcd_contiguous_id(tix, total);
      batch = __builtin_amdgcn_readfirstlane(gid / per_batch);
      pid = __builtin_amdgcn_readfirstlane(gid % per_batch);
    }
    const unsigned tm = __builtin_amdgcn_readfirstlane(pid / tiles_n), tn = __builtin_amdgcn_readfirstlane(pid % tiles_n);
    const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;
    const int64_t rows_a = n - m0 < BM ? n - m0 : BM, rows_w = m - n0 < BN ? m - n0 : BN;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Q + (static_cast<int64_t>(batch) * n + m0) * d, static_cast<unsigned>(rows_a) * row_bytes);
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(Kmat + (static_cast<int64_t>(batch) * m + n0) * d, static_cast<unsigned>(rows_w) * row_bytes);
    // ---- every k tile of both operands, asynchronously (rows past the extents and the K tail read as zeros)
    for (int kt = 0; kt < ktiles; ++kt) {
      const unsigned off = (static_cast<int64_t>(kt) * kBK + c_in * 8 < d) ? g_off + static_cast<unsigned>(kt) * kRowBytes : kOob;
      char* base = lds + kt * kStage + wv * 1024;
#pragma unroll
      for (int i = 0; i < LA; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + i * NW * 1024), 16, off, i * g_step, 0, 0);
#pragma unroll
      for (int i = 0; i < LB; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(base + kABytes + i * NW * 1024), 16, off, i * g_step, 0, 0);
    }
    // ---- this lane's part of the mask tile
    const int64_t col = n0 + wn * WTN + slot * 4;
    const bool vec_ok = ptr_ok && col + 3 < m;
    f16x4 mk[kPasses];
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int64_t row = m0 + wm * WTM + p * kRowsPerPass + rsub;
      const f16x4 zero = {};
      mk[p] = zero;
      if (row >= n) continue;
      if (vec_ok) {
        mk[p] = *reinterpret_cast<const f16x4_a2*>(mask + row * m + col);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (col + e < m) mk[p][e] = mask[row * m + col + e];
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // the operands have landed (and the previous tile's stores have left)
    __builtin_amdgcn_s_barrier();

    f32x16 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    for (int kt = 0; kt < ktiles; ++kt) {
      const char* stage = lds + kt * kStage;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        f16x8 fa[MT], fb[NT];
#pragma unroll
        for (int i = 0; i < MT; ++i) fa[i] = *reinterpret_cast<const f16x8*>(stage + a_base + i * 4096 + lds_rd[ks]);
#pragma unroll
        for (int j = 0; j < NT; ++j) fb[j] = *reinterpret_cast<const f16x8*>(stage + b_base + j * 4096 + lds_rd[ks]);
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
      }
    }
    __syncthreads();  // every wavefront is done with the operand tiles

    // ---- epilogue: acc[i][j][v] of lane l is row i*32 + (l & 31), column j*32 + 8*(v/4) + 4*(l >> 5) + v%4 of
    // the wavefront tile; staged in a wavefront-private LDS region (8-byte slots, xor-swizzled by the row)
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const unsigned mr = i * 32 + (l & 31u);
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f16x4 hv;
#pragma unroll
          for (int e = 0; e < 4; ++e) hv[e] = static_cast<half_t>(acc[i][j][g * 4 + e]);
          const unsigned sl = j * 8 + g * 2 + (l >> 5);
          *reinterpret_cast<f16x4*>(region + mr * kRowB + ((sl ^ (mr & (kSlots - 1))) * 8)) = hv;
        }
    }
    // no barrier: a wavefront reads back only what it wrote itself
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const unsigned mr = p * kRowsPerPass + rsub;
      f16x4 hv = *reinterpret_cast<const f16x4*>(region + mr * kRowB + ((slot ^ (mr & (kSlots - 1))) * 8));
      const int64_t row = m0 + wm * WTM + mr;
      if (row >= n) continue;
      hv = scores_steps_vec(hv, scale, mk[p]);
      float* dst = out + (static_cast<int64_t>(batch) * n + row) * m + col;
      if (vec_ok) {
        const f32x4v wide = {static_cast<float>(hv[0]), static_cast<float>(hv[1]), static_cast<float>(hv[2]), static_cast<float>(hv[3])};
        // 4*heads*n*m bytes: streamed -- unless a row is not a whole number of 64-byte sectors: then the tiles
        // left and right of a column boundary each write part of a sector, and only the cache can join the parts
        if (stream_out) __builtin_nontemporal_store(wide, reinterpret_cast<f32x4v*>(dst));
        else *reinterpret_cast<f32x4v_a4*>(dst) = wide;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (col + e < m) dst[e] = static_cast<float>(hv[e]);
      }
    }
    __syncthreads();  // the staging regions are free: the next tile's operands may land
  }
}

// The walking scores kernel for head dimensions 64 + 8 TC (TC = 2: the model's 80; 4: 96), rows of whole sectors, as a
// two-deep pipeline.  In attn_scores_kernel a workgroup's tile is a chain -- request the operands, wait for them,
// multiply, stage, store, and wait for the stores to drain before the next operands may land -- hidden only by the
// other two workgroups of the CU.  Here the tail of the head dimension (k = 64 ..) is kept in rows of its own 16 TC bytes
// instead of a second 128-byte k tile, so a tile's operands take 24 KiB + 192 x 16 TC bytes and two sets fit twice per
// CU: the next tile's operands and mask are requested as soon as the MFMAs of the current one are done, and land while
// it is staged and its epilogue computed; the results wait in registers and are stored after the next tile's operands
// have been waited for, so that no wait for loads ever waits for stores issued just before (loads and stores share one
// counter, in order).  Tile numbering, mask, staging and epilogue as in attn_scores_kernel<128, 64>.
template <int TC>
__global__ void __launch_bounds__(256) attn_scores_pipe_kernel(const half_t* __restrict__ Q, const half_t* __restrict__ Kmat,
                                                               const half_t* __restrict__ mask, float* __restrict__ out,
                                                               int64_t n, int64_t m, int64_t d, float scale, unsigned tiles_m,
                                                               unsigned tiles_n, unsigned heads, unsigned pinned) {
  constexpr int BM = 128, BN = 64, NW = 4, WN = 2, WTM = BM / 2, WTN = BN / 2, MT = WTM / 32, NT = WTN / 32;
  constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;
  constexpr int kTB = 16 * TC;                                // bytes of a row's tail
  constexpr int kABytes = BM * kRowBytes, kMain = (BM + BN) * kRowBytes;
  constexpr int kTailA = kMain, kTailW = kMain + BM * kTB, kSet = kMain + (BM + BN) * kTB;
  constexpr int kRowsPerTailLoad = 64 / TC;                   // rows a 1 KiB load of tails covers
  static_assert(TC == 2 || TC == 4, "tails of 16 or 32 elements");
  static_assert(BM % (kRowsPerTailLoad * NW) == 0 || BM / kRowsPerTailLoad <= NW, "tail loads per wavefront");
  static_assert(BM * BN * 2 <= kSet, "epilogue staging must fit an operand set");
  __shared__ __attribute__((aligned(1024))) char lds[2 * kSet];

  const unsigned t = threadIdx.x, l = t & 63u;
  const unsigned wv = __builtin_amdgcn_readfirstlane(t >> 6), wm = wv / WN, wn = wv % WN;
  const unsigned row_bytes = static_cast<unsigned>(d) * 2u;
  const unsigned r_in = 2u * (l >> 4) + (((l >> 3) & 1u) ^ (wv & 1u));
  const unsigned c_in = (l & 7u) ^ r_in;
  const unsigned g_off = (8u * wv + r_in) * row_bytes + c_in * 16u;
  const unsigned g_step = 8u * NW * row_bytes;
  const unsigned t_row = l / TC, t_off = t_row * row_bytes + 128u + (l % TC) * 16u;  // this lane's piece of a tail load
  unsigned lds_rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) lds_rd[ks] = lds_chunk_offset(l & 31u, 2u * ks + (l >> 5));
  const unsigned a_base = wm * WTM * 128u, b_base = kABytes + wn * WTN * 128u;

  constexpr int kSlots = WTN / 4, kRowB = WTN * 2, kRowsPerPass = 64 / kSlots, kPasses = WTM / kRowsPerPass;
  const unsigned slot = l % kSlots, rsub = l / kSlots;

  const unsigned per_batch = tiles_m * tiles_n, total = per_batch * heads;
  const unsigned span_base = per_batch / kNumXCD, span_rem = per_batch % kNumXCD;
  const unsigned walk_end = pinned ? kNumXCD * heads * (span_base + (span_rem ? 1u : 0u)) : total;
  // tile index -> (head, tile row, tile column); false: nothing at this index (a shorter span has ended)
  auto locate = [&](unsigned tix, unsigned& batch, unsigned& tm, unsigned& tn) -> bool {
    unsigned pid;
    if (pinned) {
      const unsigned xcd = tix % kNumXCD, local = tix / kNumXCD;
      const unsigned span = span_base + (xcd < span_rem ? 1u : 0u), first = xcd * span_base + (xcd < span_rem ? xcd : span_rem);
      if (local >= span * heads) return false;
      batch = __builtin_amdgcn_readfirstlane(local / span);
      pid = __builtin_amdgcn_readfirstlane(first + local % span);
    } else {
      const unsigned gid = xcd_contiguous_id(tix, total);
      batch = __builtin_amdgcn_readfirstlane(gid / per_batch);
      pid = __builtin_amdgcn_readfirstlane(gid % per_batch);
    }
    tm = __builtin_amdgcn_readfirstlane(pid / tiles_n);
    tn = __builtin_amdgcn_readfirstlane(pid % tiles_n);
    return true;
  };
  // every operand piece of a tile into set `base`, asynchronously (rows past the extents read as zeros), and this lane's
  // part of the mask tile into `mk`
  auto request = [&](unsigned batch, unsigned tm, unsigned tn, char* base, f16x4 (&mk)[kPasses]) {
    const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;
    const int64_t rows_a = n - m0 < BM ? n - m0 : BM, rows_w = m - n0 < BN ? m - n0 : BN;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Q + (static_cast<int64_t>(batch) * n + m0) * d, static_cast<unsigned>(rows_a) * row_bytes);
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(Kmat + (static_cast<int64_t>(batch) * m + n0) * d, static_cast<unsigned>(rows_w) * row_bytes);
#pragma unroll
    for (int i = 0; i < LA; ++i) __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + wv * 1024 + i * NW * 1024), 16, g_off, i * g_step, 0, 0);
#pragma unroll
    for (int i = 0; i < LB; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(base + kABytes + wv * 1024 + i * NW * 1024), 16, g_off, i * g_step, 0, 0);
    // tails: load j covers rows j * kRowsPerTailLoad ..; wavefront w takes loads w, w + 4, ... of A and of W
#pragma unroll
    for (int j = 0; j < BM / kRowsPerTailLoad; ++j)
      if (static_cast<unsigned>(j % NW) == wv)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + kTailA + j * 1024), 16, t_off, j * kRowsPerTailLoad * row_bytes, 0, 0);
#pragma unroll
    for (int j = 0; j < BN / kRowsPerTailLoad; ++j)
      if (static_cast<unsigned>(j % NW) == wv)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(base + kTailW + j * 1024), 16, t_off, j * kRowsPerTailLoad * row_bytes, 0, 0);
    const int64_t col = n0 + wn * WTN + slot * 4;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int64_t row = m0 + wm * WTM + p * kRowsPerPass + rsub;
      const f16x4 zero = {};
      mk[p] = row < n && col + 3 < m ? *reinterpret_cast<const f16x4_a2*>(mask + row * m + col) : zero;  // (m % 16 == 0: whole vectors)
    }
  };
  // the results of a tile, held until the next tile's operands have been waited for
  f32x4v held[kPasses];
  int64_t held_at[kPasses];  // element offset of each vector; -1: nothing to store
  auto store_held = [&]() {
#pragma unroll
    for (int p = 0; p < kPasses; ++p)
      if (held_at[p] >= 0) __builtin_nontemporal_store(held[p], reinterpret_cast<f32x4v*>(out + held_at[p]));
  };
#pragma unroll
  for (int p = 0; p < kPasses; ++p) held_at[p] = -1;

  f16x4 mk_cur[kPasses], mk_nxt[kPasses];
  unsigned batch = 0, tm = 0, tn = 0;
  unsigned tix = blockIdx.x;
  bool have = false;
  for (; tix < walk_end && !have; tix += have ? 0u : gridDim.x) have = locate(tix, batch, tm, tn);
  int cur = 0;
  if (have) request(batch, tm, tn, lds, mk_cur);
  while (have) {
    // the next tile of this workgroup, if any
    unsigned nbatch = 0, ntm = 0, ntn = 0;
    bool more = false;
    unsigned nix = tix + gridDim.x;
    for (; nix < walk_end && !more; nix += more ? 0u : gridDim.x) more = locate(nix, nbatch, ntm, ntn);
    char* set = lds + cur * kSet;
    __builtin_amdgcn_s_waitcnt(0x0070);  // this tile's operands have landed (the stores before them left long ago)
    __builtin_amdgcn_s_barrier();
    store_held();                         // the previous tile's results: they drain while this tile is computed
    f32x16 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      f16x8 fa[MT], fb[NT];
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[i] = *reinterpret_cast<const f16x8*>(set + a_base + i * 4096 + lds_rd[ks]);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb[j] = *reinterpret_cast<const f16x8*>(set + b_base + j * 4096 + lds_rd[ks]);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int ks = 0; ks < TC / 2; ++ks) {  // the tail: lane l supplies row l & 31, piece 2 ks + (l >> 5) of it
      f16x8 fa[MT], fb[NT];
      const unsigned at = (l & 31u) * kTB + (2u * ks + (l >> 5)) * 16u;
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[i] = *reinterpret_cast<const f16x8*>(set + kTailA + (wm * WTM + i * 32) * kTB + at);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb[j] = *reinterpret_cast<const f16x8*>(set + kTailW + (wn * WTN + j * 32) * kTB + at);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    // every wavefront is done with this set (its fragments are in registers: the MFMAs above consumed them): it becomes
    // the staging area; the other set is free as well.  (A bare barrier: a wait for the stores just issued is what this
    // kernel is built to avoid.)
    DTAS_SCHED_FENCE();
    __builtin_amdgcn_s_barrier();
    DTAS_SCHED_FENCE();
    if (more) request(nbatch, ntm, ntn, lds + (cur ^ 1) * kSet, mk_nxt);
    // ---- epilogue, as in attn_scores_kernel: staged in a wavefront-private region of this set
    char* region = set + wv * (WTM * kRowB);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const unsigned mr = i * 32 + (l & 31u);
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f16x4 hv;
#pragma unroll
          for (int e = 0; e < 4; ++e) hv[e] = static_cast<half_t>(acc[i][j][g * 4 + e]);
          const unsigned sl = j * 8 + g * 2 + (l >> 5);
          *reinterpret_cast<f16x4*>(region + mr * kRowB + ((sl ^ (mr & (kSlots - 1))) * 8)) = hv;
        }
    }
    const int64_t m0 = static_cast<int64_t>(tm) * BM, col = static_cast<int64_t>(tn) * BN + wn * WTN + slot * 4;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const unsigned mr = p * kRowsPerPass + rsub;
      f16x4 hv = *reinterpret_cast<const f16x4*>(region + mr * kRowB + ((slot ^ (mr & (kSlots - 1))) * 8));
      const int64_t row = m0 + wm * WTM + mr;
      hv = scores_steps_vec(hv, scale, mk_cur[p]);
      held[p] = f32x4v{static_cast<float>(hv[0]), static_cast<float>(hv[1]), static_cast<float>(hv[2]), static_cast<float>(hv[3])};
      held_at[p] = row < n && col + 3 < m ? (static_cast<int64_t>(batch) * n + row) * m + col : -1;
    }
#pragma unroll
    for (int p = 0; p < kPasses; ++p) mk_cur[p] = mk_nxt[p];
    have = more;
    batch = nbatch; tm = ntm; tn = ntn;
    tix = nix;
    cur ^= 1;
  }
  store_held();
}

// M <= 16 * MT.  Workgroup = 16 columns of C; wavefront w takes k steps w, w + nwaves, ...
// of 32 elements.  Lane l supplies row (l & 15), elements 8*(l >> 4) .. +8 of the step, for both
// operands, loaded straight from global memory.  Result register v of lane l is row
// 4*(l >> 4) + v, column l & 15 of the 16x16 block.
template <int MT>
__global__ void __launch_bounds__(1024) gemm_skinny_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W,
                                                          GemmEpilogue ep, void* __restrict__ C, int64_t M, int64_t N,
                                                          int64_t K) {
  __shared__ f32x4v part[16][MT][64];
  const unsigned t = threadIdx.x, l = t & 63u, wv = t >> 6, nwaves = blockDim.x >> 6;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * 16;
  const int64_t wrow = n0 + (l & 15u) < N ? n0 + (l & 15u) : N - 1;  // clamped rows are never stored
  const half_t* wp = W + wrow * K + 8 * (l >> 4);
  const half_t* ap[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int64_t arow = i * 16 + (l & 15u) < M ? i * 16 + (l & 15u) : M - 1;
    ap[i] = A + arow * K + 8 * (l >> 4);
  }
  f32x4v acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = f32x4v{0.f, 0.f, 0.f, 0.f};

  const int64_t steps = K >> 5;  // whole 32-element steps; K % 32 is handled below
  // A wavefront takes pairs of consecutive steps (2p, 2p+1) for p = wv, wv + nwaves, ...: the two
  // 64-byte pieces a lane row contributes per pair are the halves of one 128-byte line.  G pairs
  // at a time, so that 2 * G * (1 + MT) independent 1 KiB loads are in flight before the first
  // MFMA: the loop is a chain of memory round trips, and K = 4096 over 16 wavefronts is one of them.
  constexpr int G = MT == 1 ? 4 : 2;
  const int64_t pairs = steps >> 1;
  const int64_t mine = pairs > wv ? (pairs - wv + nwaves - 1) / nwaves : 0;
  int64_t q = 0;
  for (; q + G <= mine; q += G) {
    f16x8 fw[2 * G], fa[2 * G][MT];
#pragma unroll
    for (int u = 0; u < 2 * G; ++u) {
      const int64_t off = ((wv + (q + (u >> 1)) * nwaves) * 2 + (u & 1)) * 32;
      fw[u] = __builtin_bit_cast(f16x8, load_stream(reinterpret_cast<const u32x4*>(wp + off)));
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[u][i] = *reinterpret_cast<const f16x8*>(ap[i] + off);
    }
#pragma unroll
    for (int u = 0; u < 2 * G; ++u)
#pragma unroll
      for (int i = 0; i < MT; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[u][i], fw[u], acc[i], 0, 0, 0);
  }
  for (; q < mine; ++q) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int64_t off = ((wv + q * nwaves) * 2 + u) * 32;
      const f16x8 fw = __builtin_bit_cast(f16x8, load_stream(reinterpret_cast<const u32x4*>(wp + off)));
#pragma unroll
      for (int i = 0; i < MT; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const f16x8*>(ap[i] + off), fw, acc[i], 0, 0, 0);
    }
  }
  // an odd number of whole steps: the last one goes to the wavefront after the last pair's
  if ((steps & 1) && wv == pairs % nwaves) {
    const int64_t off = (steps - 1) * 32;
    const f16x8 fw = __builtin_bit_cast(f16x8, load_stream(reinterpret_cast<const u32x4*>(wp + off)));
#pragma unroll
    for (int i = 0; i < MT; ++i)
      acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const f16x8*>(ap[i] + off), fw, acc[i], 0, 0, 0);
  }
  // K % 32 (a multiple of 8): the last partial step, chunks past K contribute zeros
  if ((K & 31) != 0 && wv == steps % nwaves) {
    const bool in = steps * 32 + 8 * (l >> 4) < K;
    f16x8 fw, zero;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero[e] = static_cast<half_t>(0.f);
    fw = in ? *reinterpret_cast<const f16x8*>(wp + steps * 32) : zero;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const f16x8 fa = in ? *reinterpret_cast<const f16x8*>(ap[i] + steps * 32) : zero;
      acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, fw, acc[i], 0, 0, 0);
    }
  }

#pragma unroll
  for (int i = 0; i < MT; ++i) part[wv][i][l] = acc[i];
  __syncthreads();
  // MT * 64 lanes' worth of 4-row column strips; thread t folds strip t over the wavefronts
  for (unsigned idx = t; idx < MT * 64u; idx += blockDim.x) {
    const unsigned i = idx >> 6, ll = idx & 63u;
    f32x4v s = part[0][i][ll];
    for (unsigned w = 1; w < nwaves; ++w) s += part[w][i][ll];
    const int64_t col = n0 + (ll & 15u);
    if (col < N) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int64_t row = i * 16 + 4 * (ll >> 4) + v;
        if (row < M) finish(s[v], ep, C, row, col, N);
      }
    }
  }
}

// M <= 16 * MT against a W that is streamed once: with few rows of A the launch is a read of W from HBM, and what
// the measurements on MI355X say about that read decides the shape.  A wavefront access of 1 KiB of one row
// sustains 7.0 TB/s over the chip; 4 rows x 256 bytes 6.0; 8 rows x 128 bytes -- the block loads of the MFMA
// tiles -- 4.5; 16 rows x 64 bytes -- operands loaded in MFMA layout, as gemm_skinny_kernel does -- 5.0, and A
// fetched per wavefront from the L2 in that layout costs a further quarter.  Deeper LDS pipelines of the tile
// kernel (up to all of a workgroup's k tiles in flight) changed nothing: the access shape is the limit.
// So here a workgroup of WAVES wavefronts owns 16 * WAVES columns of C and a K slice of SEG x 512 elements;
// wavefront w brings in its own 16 rows of W, each row's slice as SEG direct-to-LDS loads of 1 KiB, and its share
// of the slice's A rows (1 KiB accesses as well, from the L2), all requested before anything is waited for.  Only
// the A rows are shared, so one barrier, after they have landed; W is waited for per 512-element segment.
// In the LDS the 16-byte chunk c of row r sits in slot c ^ f(r), f(r) = 2 * (r & 7) + ((r >> 3) & 1), and lane
// groups 0..3 of a fragment read take chunks 0, 2, 1, 3 of the k step: the 16 rows of a lane group land in 16
// different 16-byte bank groups, and so do the 8 rows x 2 chunks of lanes l, l + 32, which the LDS serves together.
// K slices meet in the workspace as in the tile kernel: partials in accumulator layout, added in slice order by
// the workgroup that arrives last.  Result register v of lane l is row 4 * (l >> 4) + v, column l & 15 of a 16x16
// block (A is the first MFMA operand).
__device__ __forceinline__ unsigned stream_swizzle(unsigned r) { return ((r & 7u) << 1) | ((r >> 3) & 1u); }

//
// Q8: W is 8-bit with an fp16 scale per 32 elements of a row (bytes [N][K], ep.wscale [N][K/32], K % 256 == 0).  A
// 512-element segment of a row is 512 bytes, so a 1 KiB load brings in two rows; the bytes sit in the LDS per
// (wavefront, segment) as 16 rows of 512 bytes, 16-byte chunk c of row r in slot c ^ f(r) as above; a wavefront's
// 16 x SEG x 16 scales arrive with one more load.  A lane's 8 weights of a k step are 8 consecutive bytes (lane
// groups 0..3 take bytes 0-7, 16-23, 8-15, 24-31 of the step, matching the chunk order of the A fragments: lanes l
// and l + 32 then read the two halves of one chunk) and are widened and scaled in registers, rounded as the
// dequantiser rounds them.
template <int MT, int SEG, int WAVES, bool Q8 = false>
__global__ void __launch_bounds__(64 * WAVES) gemm_stream_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W,
                                                                GemmEpilogue ep, void* __restrict__ C, int64_t M, int64_t N,
                                                                int64_t K, unsigned nsplit, float* __restrict__ ws,
                                                                unsigned* __restrict__ arrivals) {
  constexpr int kCols = 16 * WAVES, kRowsA = 16 * MT, kSegBytes = 1024, kRowLds = SEG * kSegBytes;
  constexpr int kWSlab = Q8 ? kCols * SEG * 512 : kCols * kRowLds, kScaleSlab = Q8 ? WAVES * 1024 : 0;
  constexpr int kALoads = kRowsA / WAVES * SEG, kWLoads = Q8 ? 8 * SEG + 1 : 16 * SEG;
  static_assert(kRowsA % WAVES == 0 && kWSlab + kRowsA * kRowLds + kScaleSlab <= kLdsBytes && kALoads + kWLoads <= 63, "slab / LDS / vmcnt");
  __shared__ __attribute__((aligned(1024))) char lds[kWSlab + kRowsA * kRowLds + kScaleSlab];
  const unsigned t = threadIdx.x, l = t & 63u;
  const unsigned wv = __builtin_amdgcn_readfirstlane(t >> 6);
  // (the K slices of a column tile, which share lines of the scales, run on one XCD)
  const unsigned item = Q8 ? xcd_contiguous_id(blockIdx.x, gridDim.x) : blockIdx.x;
  const unsigned tn = __builtin_amdgcn_readfirstlane(item / nsplit), z = __builtin_amdgcn_readfirstlane(item % nsplit);
  const int64_t n0 = static_cast<int64_t>(tn) * kCols;
  const int64_t rows_w = N - n0 < kCols ? N - n0 : kCols;
  const unsigned row_bytes = static_cast<unsigned>(K) * 2u;
  const unsigned w_row_bytes = Q8 ? static_cast<unsigned>(K) : row_bytes;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(reinterpret_cast<const char*>(W) + n0 * w_row_bytes, static_cast<unsigned>(rows_w) * w_row_bytes);
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(A, static_cast<unsigned>(M) * row_bytes);
  // lane l of the load of (row, segment s) fetches the chunk that belongs in slot l: chunk l ^ f(row); past K: out of range
  auto voff = [&](unsigned row, int s) -> unsigned {
    const unsigned c = l ^ stream_swizzle(row);
    const int64_t k = (static_cast<int64_t>(z) * SEG + s) * 512 + c * 8;
    return k < K ? row * row_bytes + static_cast<unsigned>(k) * 2u : kOob;
  };
  ColumnOperands<MT> colop;
  load_column_operands<MT>(colop, ep, l >> 4, n0 + wv * 16u + (l & 15u), M, N);
  char* lds_a = lds + kWSlab;
#pragma unroll
  for (int i = 0; i < kRowsA / WAVES; ++i) {
    const unsigned a = i * WAVES + wv;
#pragma unroll
    for (int s = 0; s < SEG; ++s) {
      const unsigned at = voff(a, s);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(lds_a + a * kRowLds + s * kSegBytes), 16, at, 0, 0, 0);
    }
  }
  char* lds_w8 = lds + wv * (SEG * 8192);          // Q8: this wavefront's bytes, [segment][row][512]
  char* lds_sc = lds + kWSlab + kRowsA * kRowLds + wv * 1024;  // Q8: ... and scales, [row][16 * SEG]
  if constexpr (Q8) {
    {  // scales: lane l takes 8 of row l / (2 SEG)
      const unsigned r = l / (2 * SEG), part = l % (2 * SEG);
      const unsigned sc_row_bytes = static_cast<unsigned>(K >> 5) * 2u;
      const __amdgpu_buffer_rsrc_t rs = make_rsrc(reinterpret_cast<const char*>(ep.wscale) + n0 * sc_row_bytes, static_cast<unsigned>(rows_w) * sc_row_bytes);
      const int64_t k = static_cast<int64_t>(z) * (SEG * 512) + part * 256;
      const unsigned at = (l < 32u * SEG && k < K) ? (wv * 16u + r) * sc_row_bytes + static_cast<unsigned>(k >> 5) * 2u : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)lds_sc, 16, at, 0, 0, 0);
    }
#pragma unroll
    for (int s = 0; s < SEG; ++s)
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const unsigned r = 2u * q + (l >> 5), c = (l & 31u) ^ stream_swizzle(r);
        const int64_t k = (static_cast<int64_t>(z) * SEG + s) * 512 + c * 16;
        const unsigned at = k < K ? (wv * 16u + r) * w_row_bytes + static_cast<unsigned>(k) : kOob;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(lds_w8 + s * 8192 + q * 1024), 16, at, 0, 0, 0);
      }
  } else {
#pragma unroll
  for (int s = 0; s < SEG; ++s)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const unsigned row = wv * 16u + r, at = voff(row, s);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(lds + row * kRowLds + s * kSegBytes), 16, at, 0, 0, 0);
    }
  }
  f32x4v acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = f32x4v{0.f, 0.f, 0.f, 0.f};
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(kWLoads));  // this wavefront's A rows have landed
  __builtin_amdgcn_s_barrier();                       // ... and everybody's
  pin_column_operands<MT>(colop);
  DTAS_SCHED_FENCE();
  // fragment reads: row l & 15 of a 16-row block, chunk 4 * ks + perm(l >> 4) -> slot (4 * ks) ^ x, x = perm ^ f(row)
  const unsigned i16 = l & 15u, g = l >> 4;
  const unsigned x16 = ((((g & 1u) << 1) | (g >> 1)) ^ stream_swizzle(i16)) * 16u;
  const char* w_lane = lds + (wv * 16u + i16) * kRowLds;
  const char* a_lane = lds_a + i16 * kRowLds;
  // Q8: bytes 8 p .. 8 p + 7 of the step, p = 0, 2, 1, 3 for lane groups 0..3: chunk 2 ks + (p >> 1), half p & 1
  const unsigned p8 = ((g & 1u) << 1) | (g >> 1);
  const unsigned x8 = (((p8 >> 1) ^ stream_swizzle(i16)) * 16u);
  const char* w8_lane = lds_w8 + i16 * 512u + (p8 & 1u) * 8u;
  f16x8 scales[Q8 ? 2 * SEG : 1];
#pragma unroll
  for (int s = 0; s < SEG; ++s) {
    if (s == 0) __builtin_amdgcn_s_waitcnt(waitcnt_imm((Q8 ? 8 : 16) * (SEG - 1)));
    else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
    DTAS_SCHED_FENCE();
    if constexpr (Q8) {
      if (s == 0) {
#pragma unroll
        for (int h = 0; h < 2 * SEG; ++h) scales[h] = *reinterpret_cast<const f16x8*>(lds_sc + i16 * (32 * SEG) + h * 16);
      }
    }
#pragma unroll
    for (int ks = 0; ks < 16; ++ks) {
      const unsigned at = s * kSegBytes + (x16 ^ (ks * 64u));
      f16x8 fw;
      if constexpr (Q8) {
        const u32x2 raw = *reinterpret_cast<const u32x2*>(w8_lane + s * 8192 + (x8 ^ (ks * 32u)));
        // (a step past K multiplies zeros of A: its scale is made zero too, whatever lies behind the row's scales)
        const bool in = (static_cast<int64_t>(z) * SEG + s) * 512 + ks * 32 < K;
        const half_t sc = in ? scales[2 * s + ks / 8][ks % 8] : static_cast<half_t>(0.f);
        const f16x2 s2 = {sc, sc};
        f16x2 d0, d1, d2, d3;
        dequant_q8_word(raw[0], s2, d0, d1);
        dequant_q8_word(raw[1], s2, d2, d3);
        fw = f16x8{d0[0], d0[1], d1[0], d1[1], d2[0], d2[1], d3[0], d3[1]};
      } else {
        fw = *reinterpret_cast<const f16x8*>(w_lane + at);
      }
#pragma unroll
      for (int i = 0; i < MT; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const f16x8*>(a_lane + i * 16 * kRowLds + at), fw, acc[i], 0, 0, 0);
    }
    DTAS_SCHED_FENCE();
  }
  static_assert(SEG <= 2, "the waits above are written for one or two segments");

  if (nsplit > 1) {
    __syncthreads();  // nobody reads the slab any more: its first word becomes the flag
    volatile unsigned* is_last = reinterpret_cast<volatile unsigned*>(lds);
    constexpr int kPer = 2 * MT;                    // 8-byte units per lane
    constexpr int kPartial = kPer * 64 * WAVES;     // ... per workgroup
    unsigned long long* tile_ws = reinterpret_cast<unsigned long long*>(ws) + static_cast<size_t>(tn) * nsplit * kPartial;
    unsigned long long* mine = tile_ws + static_cast<size_t>(z) * kPartial + wv * (kPer * 64);
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
      const f32x2v pr = {acc[q / 2][2 * (q % 2)], acc[q / 2][2 * (q % 2) + 1]};
      __hip_atomic_store(mine + q * 64 + l, __builtin_bit_cast(unsigned long long, pr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));  // (device-scope stores: drained = visible to every XCD; the barrier does not wait for them)
    __syncthreads();  // every store of this workgroup has completed
    if (t == 0) {
      const unsigned before = __hip_atomic_fetch_add(arrivals + tn, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *is_last = before == nsplit - 1 ? 1u : 0u;
      if (before == nsplit - 1)  // re-armed for the next launch
        __hip_atomic_store(arrivals + tn, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (*is_last == 0) return;
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = f32x4v{0.f, 0.f, 0.f, 0.f};
    // slices are added in slice order whoever arrived last, up to 8 of them requested per round trip
    constexpr int kGroup = MT <= 2 ? 8 : 4;
    for (unsigned k0 = 0; k0 < nsplit; k0 += kGroup) {
      unsigned long long raw[kGroup][kPer];
#pragma unroll
      for (int gk = 0; gk < kGroup; ++gk) {
        const unsigned k = k0 + gk < nsplit ? k0 + gk : nsplit - 1;  // (past the last slice: re-read it, not added)
        const unsigned long long* part = tile_ws + static_cast<size_t>(k) * kPartial + wv * (kPer * 64);
#pragma unroll
        for (int q = 0; q < kPer; ++q) raw[gk][q] = __hip_atomic_load(part + q * 64 + l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
#pragma unroll
      for (int gk = 0; gk < kGroup; ++gk) {
        if (k0 + gk < nsplit) {
#pragma unroll
          for (int q = 0; q < kPer; ++q) {
            const f32x2v pr = __builtin_bit_cast(f32x2v, raw[gk][q]);
            acc[q / 2][2 * (q % 2)] += pr[0];
            acc[q / 2][2 * (q % 2) + 1] += pr[1];
          }
        }
      }
    }
  }
  finish_column<MT>(acc, colop, ep, C, g, n0 + wv * 16u + i16, M, N);
}

// The W-streaming kernel with a loop over K instead of K slices: for a W with many rows (enough column tiles to fill the
// chip without splitting K) a workgroup of WAVES wavefronts owns 16 * WAVES columns of C over the whole of K and walks it
// in segments of 256 elements through a ring of NSTG LDS stages, NSTG - 1 segments requested ahead; the sums stay in
// registers, nothing is handed over.  A segment of a row is 512 bytes, so every 1 KiB load brings in two rows (a
// wavefront its own 16 rows of W with 8 loads, and its share of the 16 * MT rows of A); layout, swizzle and fragment
// order as in gemm_stream_kernel.  One barrier per segment: it makes the segment's A rows visible and says that
// everybody has read the stage that the next request overwrites.
template <int MT, int WAVES, int NSTG>
__global__ void __launch_bounds__(64 * WAVES) gemm_stream_loop_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W,
                                                                     GemmEpilogue ep, void* __restrict__ C, int64_t M, int64_t N,
                                                                     int64_t K) {
  constexpr int kCols = 16 * WAVES, kRowsA = 16 * MT, kSegK = 256, kRowLds = 2 * kSegK;
  constexpr int kStage = (kCols + kRowsA) * kRowLds;
  constexpr int kALoads = kRowsA / 2 / WAVES;  // 1 KiB loads (two rows each) per wavefront and segment
  constexpr int kL = 8 + kALoads;
  static_assert((kRowsA / 2) % WAVES == 0 && NSTG >= 2 && NSTG * kStage <= kLdsBytes && (NSTG - 1) * kL <= 63, "stages / LDS / vmcnt");
  __shared__ __attribute__((aligned(1024))) char lds[NSTG * kStage];
  const unsigned t = threadIdx.x, l = t & 63u;
  const unsigned wv = __builtin_amdgcn_readfirstlane(t >> 6);
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * kCols;
  const int64_t rows_w = N - n0 < kCols ? N - n0 : kCols;
  const unsigned row_bytes = static_cast<unsigned>(K) * 2u;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(W + n0 * K, static_cast<unsigned>(rows_w) * row_bytes);
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(A, static_cast<unsigned>(M) * row_bytes);
  const int nseg = static_cast<int>((K + kSegK - 1) / kSegK);
  ColumnOperands<MT> colop;
  load_column_operands<MT>(colop, ep, l >> 4, n0 + wv * 16u + (l & 15u), M, N);
  // lane l of load q of a 16-row group fills slot l & 31 of row 2 q + (l >> 5): it fetches chunk (l & 31) ^ f(row)
  const unsigned lr = l >> 5;
  auto request = [&](int seg, char* stage) {
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const unsigned q = wv * kALoads + i, r = 2u * q + lr, c = (l & 31u) ^ stream_swizzle(r);
      const int64_t k = static_cast<int64_t>(seg) * kSegK + c * 8;
      const unsigned at = k < K ? r * row_bytes + static_cast<unsigned>(k) * 2u : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(stage + kCols * kRowLds + q * 1024), 16, at, 0, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const unsigned r = 2u * q + lr, c = (l & 31u) ^ stream_swizzle(r);
      const int64_t k = static_cast<int64_t>(seg) * kSegK + c * 8;
      const unsigned at = k < K ? (wv * 16u + r) * row_bytes + static_cast<unsigned>(k) * 2u : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(stage + wv * (16 * kRowLds) + q * 1024), 16, at, 0, 0, 0);
    }
  };
#pragma unroll
  for (int p = 0; p < NSTG - 1; ++p)
    if (p < nseg) request(p, lds + p * kStage);
  f32x4v acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = f32x4v{0.f, 0.f, 0.f, 0.f};
  const unsigned i16 = l & 15u, g = l >> 4;
  const unsigned x16 = ((((g & 1u) << 1) | (g >> 1)) ^ stream_swizzle(i16)) * 16u;
  int cur = 0;  // stage of segment s
  for (int s = 0; s < nseg; ++s) {
    // segment s has landed; later ones (at most NSTG - 2 of those requested) may stay in flight
    wait_whole_tiles<kL, NSTG - 2>(nseg - 1 - s);
    __builtin_amdgcn_s_barrier();
    if (s == 0) pin_column_operands<MT>(colop);
    DTAS_SCHED_FENCE();
    const int into = cur == 0 ? NSTG - 1 : cur - 1;  // the stage of segment s - 1, read by everybody before this barrier
    if (s + NSTG - 1 < nseg) request(s + NSTG - 1, lds + into * kStage);
    DTAS_SCHED_FENCE();
    const char* w_lane = lds + cur * kStage + (wv * 16u + i16) * kRowLds;
    const char* a_lane = lds + cur * kStage + (kCols + i16) * kRowLds;
#pragma unroll
    for (int ks = 0; ks < kSegK / 32; ++ks) {
      const unsigned at = x16 ^ (ks * 64u);
      const f16x8 fw = *reinterpret_cast<const f16x8*>(w_lane + at);
#pragma unroll
      for (int i = 0; i < MT; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const f16x8*>(a_lane + i * 16 * kRowLds + at), fw, acc[i], 0, 0, 0);
    }
    DTAS_SCHED_FENCE();
    cur = cur + 1 == NSTG ? 0 : cur + 1;
  }
  // result register v of lane l: row 4 * (l >> 4) + v, column l & 15 of a 16x16 block
  finish_column<MT>(acc, colop, ep, C, g, n0 + wv * 16u + i16, M, N);
}

// A few rows of A (M <= MV <= 4) against a W that is streamed once: R rows of W per wavefront, lane l
// takes the 16-byte chunks l, l + 64, ... of each (a wavefront access is 1 KiB of one W row, non-temporal,
// as in the GEMV kernel), multiplies each with the matching chunks of the MV rows of A (re-read per
// wavefront; they stay in L1 / L2) by v_dot2_f32_f16, and holds R * MV fp32 sums.  At the end the sums are
// added across the lanes by a reduce-scatter: in each of the first log2(R * MV) butterfly steps a lane hands
// half of its values to its partner and keeps the other half, so the fold costs R * MV - 1 exchanges in all
// instead of six per value; lane l ends with value l >> (6 - log2(R * MV)).  No LDS, no barrier: wavefronts
// are independent.  This pays for two rows of A only (8.1 against 10.1 us at 4096 x 4096, 40 against 60 at
// 32000 x 4096): every 16 bytes of W meet MV * 16 bytes of A from the L1, whose 64 bytes per clock bound
// the kernel from four rows on (16 rows: 3x slower than the MFMA tiles), so the instantiations stop at MV = 4.
template <int R, int MV>
__global__ void __launch_bounds__(256) gemm_rows_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W,
                                                        GemmEpilogue ep, void* __restrict__ C, int64_t M, int64_t N,
                                                        int64_t K) {
  constexpr int NV = R * MV;
  static_assert(NV >= 2 && NV <= 64 && (NV & (NV - 1)) == 0, "R * MV must be a power of two in [2, 64]");
  const unsigned l = threadIdx.x & 63u;
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
  if (row0 >= N) return;  // whole wavefronts leave together; nothing below synchronises across wavefronts
  const int64_t chunks = K >> 3;
  const u32x4* wv[R];
  const u32x4* av[MV];
#pragma unroll
  for (int r = 0; r < R; ++r) wv[r] = reinterpret_cast<const u32x4*>(W + (row0 + r < N ? row0 + r : N - 1) * K);  // rows past N: re-read, never stored
#pragma unroll
  for (int m = 0; m < MV; ++m) av[m] = reinterpret_cast<const u32x4*>(A + (m < M ? m : M - 1) * K);                // likewise rows past M
  float v[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = 0.f;
  // the lane that will store value idx = r * MV + m requests its bias and residual elements now and keeps them as loaded
  // (read after the reduction they cost the launch a round trip to memory of their own)
  constexpr int kShift = NV == 64 ? 0 : NV == 32 ? 1 : NV == 16 ? 2 : NV == 8 ? 3 : NV == 4 ? 4 : 5;
  const unsigned idx = l >> kShift;  // = r * MV + m
  const int64_t out_row = row0 + idx / MV, out_m = idx % MV;
  const bool stores = (l & ((1u << kShift) - 1u)) == 0 && out_row < N && out_m < M;
  const bool add2 = ep.kind == DTAS_EPI_BIAS_ADD2 || ep.kind == DTAS_EPI_BIAS_ADD2_CAST_F32;
  const half_t hz = static_cast<half_t>(0.f);
  const half_t e_bias = stores && ep.bias ? ep.bias[out_row] : hz;
  const half_t e_r1 = stores && add2 ? ep.res1[out_m * N + out_row] : hz;
  const half_t e_r2 = stores && add2 ? ep.res2[out_m * N + out_row] : hz;
  auto dot8 = [](u32x4 a, u32x4 b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned ai = a[i], bi = b[i];
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, ai), __builtin_bit_cast(f16x2, bi), acc, false);
    }
    return acc;
  };
  constexpr int U = R >= 4 ? 2 : 4;  // steps requested together: U * R KiB of W per wavefront in flight
  int64_t i = l;
  for (; i + (U - 1) * 64 < chunks; i += U * 64) {
    u32x4 wr[U][R];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < R; ++r) wr[u][r] = load_stream(wv[r] + i + u * 64);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int m = 0; m < MV; ++m) {
        const u32x4 xr = av[m][i + u * 64];
#pragma unroll
        for (int r = 0; r < R; ++r) v[r * MV + m] = dot8(xr, wr[u][r], v[r * MV + m]);
      }
  }
  for (; i < chunks; i += 64) {
    u32x4 wr[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wr[r] = load_stream(wv[r] + i);
#pragma unroll
    for (int m = 0; m < MV; ++m) {
      const u32x4 xr = av[m][i];
#pragma unroll
      for (int r = 0; r < R; ++r) v[r * MV + m] = dot8(xr, wr[r], v[r * MV + m]);
    }
  }
  asm volatile("" ::"v"(e_bias), "v"(e_r1), "v"(e_r2));  // (they exist by now: their loads stay where they were written)
  // reduce-scatter over the 64 lanes
  int n = NV;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    if (n > 1) {
      const int half = n >> 1;
      const bool upper = (l & d) != 0;
#pragma unroll
      for (int j = 0; j < half; ++j) {
        const float send = upper ? v[j] : v[j + half];
        const float keep = upper ? v[j + half] : v[j];
        v[j] = keep + __shfl_xor(send, d, 64);
      }
      n = half;
    } else {
      v[0] += __shfl_xor(v[0], d, 64);
    }
  }
  if (stores) {
    const half_t r = epilogue_value(round_h(v[0]), ep, static_cast<float>(e_bias), static_cast<float>(e_r1), static_cast<float>(e_r2));
    if (ep.out_f32) static_cast<float*>(C)[out_m * N + out_row] = static_cast<float>(r);
    else static_cast<half_t*>(C)[out_m * N + out_row] = r;
  }
}

// Any K and alignment: one thread per element of C.  blockIdx.y = problem of a batched launch;
// w_kmajor: W is [K][N] instead of [N][K]; ep.wscale set: W is 8-bit with group scales.
__global__ void __launch_bounds__(256) gemm_scalar_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W,
                                                          GemmEpilogue ep, void* __restrict__ C, int64_t M, int64_t N,
                                                          int64_t K, bool w_kmajor) {
  const int64_t batch = blockIdx.y;
  A += batch * ep.stride_a;
  W += batch * ep.stride_w;
  C = static_cast<char*>(C) + batch * ep.stride_c * (ep.out_f32 ? 4 : 2);
  if (ep.res1) ep.res1 += batch * ep.stride_res;
  if (ep.res2) ep.res2 += batch * ep.stride_res;
  const int64_t total = M * N;
  for (int64_t ij = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; ij < total;
       ij += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const half_t* a = A + (ij / N) * K;
    float acc = 0.f;
    if (ep.wscale) {  // 8-bit W: bytes [N][K], one fp16 scale per 32
      const unsigned char* wq = reinterpret_cast<const unsigned char*>(W) + (ij % N) * K;
      const half_t* sc = ep.wscale + (ij % N) * (K >> 5);
      for (int64_t k = 0; k < K; ++k) {
        const half_t q = static_cast<half_t>(static_cast<float>(wq[k])) - static_cast<half_t>(127.f);
        acc += static_cast<float>(a[k]) * static_cast<float>(q * sc[k >> 5]);
      }
    } else {
      const half_t* w = w_kmajor ? W + ij % N : W + (ij % N) * K;
      const int64_t wk = w_kmajor ? N : 1;
      for (int64_t k = 0; k < K; ++k) acc += static_cast<float>(a[k]) * static_cast<float>(w[k * wk]);
    }
    finish(acc, ep, C, ij / N, ij % N, N);
  }
}

// P.V for a handful of query rows (decoding): out[h, r, :] = sum_k P[h, r, k] * V[h, k, :].
// Workgroup = (head, 8 columns of V, R rows of P); thread t takes k = t, t + 256, ...: a 16-byte piece
// of V's row k and P[h, r, k] of each row, eight k at a time with every load requested before the
// first is used -- with m <= 2048 that is the whole job in one memory round trip, and round trips
// are what this op costs.  The pieces of one row of V are 16 bytes out of every 2*d, so the d/8
// workgroups of a head are given consecutive ids on one XCD and share the lines in its L2.
template <int R>
__global__ void __launch_bounds__(256) attn_pv_rows_kernel(const half_t* __restrict__ P, const half_t* __restrict__ V,
                                                           half_t* __restrict__ out, int64_t n, int64_t m, int64_t d) {
  __shared__ float part[4][R][8];
  const unsigned chunks = static_cast<unsigned>(d / 8);
  const unsigned id = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const unsigned h = id / chunks, cc = id % chunks, t = threadIdx.x;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * R;
  const int rows = n - r0 < R ? static_cast<int>(n - r0) : R;
  const half_t* p = P + (static_cast<int64_t>(h) * n + r0) * m;
  const half_t* v = V + static_cast<int64_t>(h) * m * d + cc * 8;
  float acc[R][8];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;
  for (int64_t kb = t; kb < m; kb += 8 * 256) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    u32x4 vraw[8];
    half_t pk[8][R];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t k = kb + u * 256;
      vraw[u] = k < m ? *reinterpret_cast<const u32x4*>(v + k * d) : zero;  // (cached: the head's other workgroups want the line too)
#pragma unroll
      for (int r = 0; r < R; ++r) pk[u][r] = (k < m && r < rows) ? p[r * m + k] : static_cast<half_t>(0.f);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const f16x8 vv = __builtin_bit_cast(f16x8, vraw[u]);
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][e] += static_cast<float>(pk[u][r]) * static_cast<float>(vv[e]);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float sum = wave_sum(acc[r][e]);
      if ((t & 63u) == 0) part[t >> 6][r][e] = sum;
    }
  __syncthreads();
  if (t < static_cast<unsigned>(rows) * 8u) {
    const unsigned r = t / 8, e = t % 8;
    out[(static_cast<int64_t>(h) * n + r0 + r) * d + cc * 8 + e] =
        static_cast<half_t>(part[0][r][e] + part[1][r][e] + part[2][r][e] + part[3][r][e]);
  }
}

// Scores for a handful of query rows (decoding): out[h, r, k] = epilogue(Q[h, r] . K[h, k]).  What the op moves is the
// head's K, m rows of d fp16 = d / 8 16-byte pieces each, contiguous in memory; a workgroup of 1024 threads takes a run of
// keys and sweeps it as attn_pv_whole_row_kernel sweeps V: thread t holds piece t % (d / 8) of the R query rows and
// multiplies it with that piece of keys t / (d / 8), + per-pass, ... (consecutive threads, consecutive 16 bytes, kU
// passes in flight), 8 products per row; the d / 8 threads of a key are neighbours, their sums meet in the LDS and the
// first R * per-pass threads add them in piece order, apply the epilogue and store a row's scores side by side.
template <int R>
__global__ void __launch_bounds__(1024) attn_scores_rows_kernel(const half_t* __restrict__ Q, const half_t* __restrict__ Kmat,
                                                               const half_t* __restrict__ mask, float* __restrict__ out, int64_t n,
                                                               int64_t m, int64_t d, float scale, unsigned keys_per_wg) {
  constexpr int kU = 4;
  __shared__ float part[R][1024];
  const unsigned chunks = static_cast<unsigned>(d / 8), per_pass = 1024u / chunks, t = threadIdx.x;
  const int64_t h = blockIdx.y, r0 = static_cast<int64_t>(blockIdx.z) * R;
  const int64_t k_lo = static_cast<int64_t>(blockIdx.x) * keys_per_wg;
  const int64_t k_hi = k_lo + keys_per_wg < m ? k_lo + keys_per_wg : m;
  const bool active = t < per_pass * chunks;
  const unsigned key0 = t / chunks, c = t - key0 * chunks;
  const u32x4* kp = reinterpret_cast<const u32x4*>(Kmat + h * m * d);
  f16x8 q[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    q[r] = __builtin_bit_cast(f16x8, active && r0 + r < n ? *(reinterpret_cast<const u32x4*>(Q + (h * n + r0 + r) * d) + c) : zero);
  }
  for (int64_t kb = k_lo; kb < k_hi; kb += static_cast<int64_t>(kU) * per_pass) {
    u32x4 raw[kU];
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const int64_t k = kb + static_cast<int64_t>(u) * per_pass + key0;
      // (K is read this once and streamed past the caches, unless further blocks of rows come for it)
      raw[u] = !(active && k < k_hi) ? zero : n <= R ? load_stream(kp + k * chunks + c) : kp[k * chunks + c];
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (kb + static_cast<int64_t>(u) * per_pass >= k_hi) break;  // (uniform)
      const f16x8 kv = __builtin_bit_cast(f16x8, raw[u]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += static_cast<float>(q[r][e]) * static_cast<float>(kv[e]);
        part[r][t] = sum;
      }
      __syncthreads();
      for (unsigned idx = t; idx < R * per_pass; idx += 1024u) {
        const unsigned r = idx / per_pass, j = idx - r * per_pass;
        const int64_t k = kb + static_cast<int64_t>(u) * per_pass + j, row = r0 + r;
        if (k < k_hi && row < n) {
          float sum = 0.f;
          for (unsigned cc = 0; cc < chunks; ++cc) sum += part[r][j * chunks + cc];
          const half_t v = epilogue_value_k<kEpiScores>(round_h(sum), false, scale, 0.f, static_cast<float>(mask[row * m + k]), 0.f);
          out[(h * n + row) * m + k] = static_cast<float>(v);
        }
      }
      __syncthreads();
    }
  }
}

// P.V for one query row per workgroup, the whole of V's head read in one sweep (decoding: n = 1, a few heads' worth of
// workgroups on the chip).  A head's V is m rows of d fp16 = d / 8 16-byte pieces each, contiguous in memory: thread t of
// 1024 takes piece t % (d / 8) of the rows t / (d / 8), + rows-per-pass, ... -- consecutive threads read consecutive
// 16 bytes, a wavefront 1 KiB, eight passes in flight -- and multiplies each piece with its row's P.  The 8 sums of a
// thread are those of its 8 columns; threads with the same piece index meet in the LDS and are added in thread order.
__global__ void __launch_bounds__(1024) attn_pv_whole_row_kernel(const half_t* __restrict__ P, const half_t* __restrict__ V,
                                                                half_t* __restrict__ out, int64_t n, int64_t m, int64_t d, unsigned cols,
                                                                unsigned nsplit, float* __restrict__ ws, unsigned* __restrict__ arrivals) {
  __shared__ float red[1024][8];
  __shared__ unsigned is_last;
  // (cols < d: the workgroups of a (head, row) share the pieces of a key, cols / 8 consecutive ones each)
  const unsigned row_chunks = static_cast<unsigned>(d / 8), chunks = cols / 8, groups = row_chunks / chunks;
  const unsigned per_pass = blockDim.x / chunks, t = threadIdx.x;
  const int64_t h = blockIdx.x / groups, r = blockIdx.y;
  const unsigned first = (blockIdx.x % groups) * chunks;
  const half_t* p = P + (h * n + r) * m;
  const u32x4* v = reinterpret_cast<const u32x4*>(V + h * m * d) + first;
  const bool active = t < per_pass * chunks;
  const unsigned row0 = t / chunks;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  // nsplit > 1: the workgroups blockIdx.z = 0 .. nsplit - 1 of a (head, row) share the keys, a run each, and meet in the
  // split-K workspace as the GEMM kernels' K slices do (partials added in run order by whoever arrives last)
  const int64_t run = (m + nsplit - 1) / nsplit;
  const int64_t k_lo = static_cast<int64_t>(blockIdx.z) * run, k_hi = k_lo + run < m ? k_lo + run : m;
  if (active) {
    constexpr int kU = 8;
    for (int64_t k0 = k_lo + row0; k0 < k_hi; k0 += static_cast<int64_t>(kU) * per_pass) {
      u32x4 vraw[kU];
      half_t pk[kU];
      const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t k = k0 + static_cast<int64_t>(u) * per_pass;
        // (piece index of thread t in pass u: t + u * per_pass * chunks -- the passes continue where the last thread stopped)
        // (one row: V is read this once and streamed past the caches; more rows: their workgroups share it)
        vraw[u] = k >= k_hi ? zero : n == 1 ? load_stream(v + k * row_chunks + (t - row0 * chunks)) : v[k * row_chunks + (t - row0 * chunks)];
        pk[u] = k < k_hi ? p[k] : static_cast<half_t>(0.f);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const f16x8 vv = __builtin_bit_cast(f16x8, vraw[u]);
        const float pf = static_cast<float>(pk[u]);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += pf * static_cast<float>(vv[e]);
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[t][e] = active ? acc[e] : 0.f;
  __syncthreads();
  // column j of the row: piece j / 8, element j % 8, summed over the per_pass threads that hold that piece
  const bool holds = t < chunks * 8u;
  float sum = 0.f;
  if (holds) {
    const unsigned c = t >> 3, e = t & 7u;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    unsigned q = 0;
    for (; q + 3 < per_pass; q += 4) {
      s0 += red[(q + 0) * chunks + c][e];
      s1 += red[(q + 1) * chunks + c][e];
      s2 += red[(q + 2) * chunks + c][e];
      s3 += red[(q + 3) * chunks + c][e];
    }
    for (; q < per_pass; ++q) s0 += red[q * chunks + c][e];
    sum = (s0 + s1) + (s2 + s3);
  }
  if (nsplit > 1) {
    const size_t tile = static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x;  // (row, head, columns)
    float* tile_ws = ws + tile * nsplit * cols;
    if (holds) __hip_atomic_store(tile_ws + static_cast<size_t>(blockIdx.z) * cols + t, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));  // (device-scope stores: drained = visible to every XCD)
    __syncthreads();
    if (t == 0) {
      const unsigned before = __hip_atomic_fetch_add(arrivals + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last = before == nsplit - 1 ? 1u : 0u;
      if (before == nsplit - 1) __hip_atomic_store(arrivals + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // re-armed for the next launch
    }
    __syncthreads();
    if (is_last == 0 || !holds) return;
    sum = 0.f;
    for (unsigned z = 0; z < nsplit; ++z) sum += __hip_atomic_load(tile_ws + static_cast<size_t>(z) * cols + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (holds) out[(h * n + r) * d + first * 8u + t] = static_cast<half_t>(sum);
}

// Library-owned scratch memory, one set per (device, stream):
//  * the split-K workspace: nsplit fp32 partial tiles per shared output tile and one arrival counter per tile
//    (zero between launches: the last arriver of a tile re-arms it);
//  * the operand buffer: the fp16 copy of an 8-bit weight matrix (dtas_gemm_q8_f16_fused's two-pass route).
// Allocated on first use by a stream and grown on demand -- the only allocations in the library.  Launches on one
// stream are ordered by it and share its set; launches on different streams use different sets, so they may overlap.
// g_ws_mutex is held from the lookup until the launches that use the set are enqueued: a set is never grown (freed
// and re-allocated: hipFree waits for the device, hence for every launch that may still use it) between a lookup
// and its launch, also with several host threads.  At most kMaxWsStreams streams per device hold a set; beyond
// that the set used longest ago is released first.
constexpr size_t kMaxSplitWsBytes = size_t{1} << 30;
constexpr int kMaxDevices = 64;
constexpr int kMaxWsStreams = 16;
struct StreamWorkspace {
  bool used = false;
  hipStream_t stream = nullptr;
  uint64_t stamp = 0;
  float* partials = nullptr;
  size_t partial_bytes = 0;
  unsigned* arrivals = nullptr;
  size_t tiles = 0;
  void* operand = nullptr;
  size_t operand_bytes = 0;
};
struct DeviceWorkspaces {
  StreamWorkspace slot[kMaxWsStreams];
  uint64_t clock = 0;
};
DeviceWorkspaces g_ws[kMaxDevices];
std::recursive_mutex g_ws_mutex;

int release_workspace(StreamWorkspace& w) {
  // kernels of earlier launches may still use the buffers: hipFree waits for the device
  if (w.partials && hipFree(w.partials) != hipSuccess) return fail("workspace: hipFree of the split-K partials failed");
  if (w.arrivals && hipFree(w.arrivals) != hipSuccess) return fail("workspace: hipFree of the split-K counters failed");
  if (w.operand && hipFree(w.operand) != hipSuccess) return fail("workspace: hipFree of the operand buffer failed");
  w = StreamWorkspace{};
  return 0;
}

// The set of `stream` on the current device (g_ws_mutex held by the caller).
int stream_workspace(hipStream_t stream, StreamWorkspace** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail("workspace: cannot identify the current device");
  DeviceWorkspaces& d = g_ws[dev];
  StreamWorkspace* free_slot = nullptr;
  StreamWorkspace* oldest = nullptr;
  for (StreamWorkspace& w : d.slot) {
    if (w.used && w.stream == stream) {
      w.stamp = ++d.clock;
      *out = &w;
      return 0;
    }
    if (!w.used && !free_slot) free_slot = &w;
    if (w.used && (!oldest || w.stamp < oldest->stamp)) oldest = &w;
  }
  if (!free_slot) {
    if (release_workspace(*oldest) != 0) return -1;
    free_slot = oldest;
  }
  free_slot->used = true;
  free_slot->stream = stream;
  free_slot->stamp = ++d.clock;
  *out = free_slot;
  return 0;
}

int split_workspace(hipStream_t stream, size_t partial_bytes, size_t tiles, float** partials, unsigned** arrivals) {
  StreamWorkspace* w = nullptr;
  if (stream_workspace(stream, &w) != 0) return -1;
  if (partial_bytes > w->partial_bytes) {
    if (w->partials && hipFree(w->partials) != hipSuccess) return fail("gemm: hipFree of the split-K workspace failed");
    w->partials = nullptr;
    w->partial_bytes = 0;
    const size_t want = partial_bytes < (size_t{32} << 20) ? (size_t{32} << 20) : partial_bytes;
    if (hipMalloc(reinterpret_cast<void**>(&w->partials), want) != hipSuccess) {
      (void)hipGetLastError();
      return fail("gemm: cannot allocate %zu bytes of split-K workspace", want);
    }
    w->partial_bytes = want;
  }
  if (tiles > w->tiles) {
    if (w->arrivals && hipFree(w->arrivals) != hipSuccess) return fail("gemm: hipFree of the split-K counters failed");
    w->arrivals = nullptr;
    w->tiles = 0;
    const size_t want = tiles < 4096 ? 4096 : tiles;
    // (cleared on the stream that will use them: a memset on the default stream is not ordered with a non-blocking stream)
    if (hipMalloc(reinterpret_cast<void**>(&w->arrivals), want * sizeof(unsigned)) != hipSuccess ||
        hipMemsetAsync(w->arrivals, 0, want * sizeof(unsigned), stream) != hipSuccess) {
      (void)hipGetLastError();
      return fail("gemm: cannot allocate the split-K arrival counters");
    }
    w->tiles = want;
  }
  *partials = w->partials;
  *arrivals = w->arrivals;
  return 0;
}

int operand_workspace(hipStream_t stream, size_t bytes, void** out) {
  StreamWorkspace* w = nullptr;
  if (stream_workspace(stream, &w) != 0) return -1;
  if (bytes > w->operand_bytes) {
    if (bytes > kMaxSplitWsBytes) return fail("operand buffer: a rewritten operand needs %zu bytes (limit %zu)", bytes, kMaxSplitWsBytes);
    if (w->operand && hipFree(w->operand) != hipSuccess) return fail("operand buffer: hipFree failed");
    w->operand = nullptr;
    w->operand_bytes = 0;
    const size_t want = bytes < (size_t{64} << 20) ? (size_t{64} << 20) : bytes;
    if (hipMalloc(&w->operand, want) != hipSuccess) {
      (void)hipGetLastError();
      return fail("operand buffer: cannot allocate %zu bytes", want);
    }
    w->operand_bytes = want;
  }
  *out = w->operand;
  return 0;
}

// Where a launch that splits K keeps its partial tiles when the caller must not allocate: set (per host thread) by
// dtas_gemm_f16_static around its call into the common code, read by launch_mfma.
struct FixedScratch {
  float* partials;
  size_t partial_bytes;
  unsigned* arrivals;
  size_t tiles;
};
thread_local const FixedScratch* t_fixed_scratch = nullptr;

void* g_static_scratch[kMaxDevices];  // device address of `scratch` on each device, once resolved
std::mutex g_static_scratch_mutex;

__global__ void zero_u32_kernel(unsigned* p, size_t count) {
  const size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
  if (i < count) p[i] = 0u;
}

// Partial tiles and arrival counters of a launch that splits K over `nsplit` workgroups per tile: the static scratch
// if the calling thread is inside dtas_gemm_f16_static, else the stream's workspace, whose lock `lock` then holds
// (the caller keeps it until its kernel is enqueued).
int split_scratch(hipStream_t s, size_t bytes, size_t split_tiles, int nsplit, float** partials, unsigned** arrivals,
                  std::unique_lock<std::recursive_mutex>* lock) {
  if (t_fixed_scratch) {
    const FixedScratch& f = *t_fixed_scratch;
    if (bytes > f.partial_bytes || split_tiles > f.tiles)
      return fail("gemm: K split over %d workgroups needs %zu bytes of partial tiles and %zu counters; the static scratch "
                  "holds %zu bytes and %zu counters (a cfg with split_k = 1 needs none)", nsplit, bytes, split_tiles, f.partial_bytes, f.tiles);
    *partials = f.partials;
    *arrivals = f.arrivals;
    // every call on this device shares the array and finds what the last one left: the counters of this launch are
    // cleared first (by a kernel, not a memset node: the caller may be capturing a graph)
    hipLaunchKernelGGL(zero_u32_kernel, dim3(static_cast<unsigned>(ceil_div(static_cast<int64_t>(split_tiles), 256))), dim3(256), 0, s, *arrivals,
                       split_tiles);
    return check_launch("gemm");
  }
  if (bytes > kMaxSplitWsBytes) return fail("gemm: split_k %d needs %zu bytes of workspace (limit %zu)", nsplit, bytes, kMaxSplitWsBytes);
  *lock = std::unique_lock<std::recursive_mutex>(g_ws_mutex);
  return split_workspace(s, bytes, split_tiles, partials, arrivals);
}

template <int BM, int BN, int WM, int WN, int NS, bool WT = false, bool WQ = false, bool M16 = false>
int launch_mfma(hipStream_t s, const half_t* A, const half_t* W, const GemmEpilogue& ep, void* C, int64_t M, int64_t N,
                int64_t K, int nsplit, int batch = 1, unsigned unsplit = 0) {
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(M, BM)), tiles_n = static_cast<unsigned>(ceil_div(N, BN));
  const size_t tiles = static_cast<size_t>(tiles_m) * tiles_n;
  float* partials = nullptr;
  unsigned* arrivals = nullptr;
  if (batch < 1 || batch > 65535) return fail("gemm: batch must be in [1, 65535], got %d", batch);
  if (unsplit > 0 && (batch != 1 || unsplit >= tiles || nsplit < 2)) return fail("gemm: a partly split launch takes one problem and a split");
  const size_t split_tiles = (tiles - unsplit) * batch;  // tiles shared by nsplit workgroups
  std::unique_lock<std::recursive_mutex> ws_lock;  // held until the launch is enqueued
  if (nsplit > 1 && split_scratch(s, split_tiles * nsplit * BM * BN * sizeof(float), split_tiles, nsplit, &partials, &arrivals, &ws_lock) != 0)
    return -1;
  const size_t wgs = unsplit + split_tiles * nsplit;
  if (wgs > 0x7fffffffu) return fail("gemm: too many workgroups");
  GemmEpilogue batched = ep;
  batched.batches = static_cast<unsigned>(batch);
  batched.tiles_unsplit = unsplit;
  hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, WM, WN, NS, WT, WQ, M16>), dim3(static_cast<unsigned>(wgs)), dim3(64 * WM * WN), 0,
                     s, A, W, batched, C, M, N, K, tiles_m, tiles_n, static_cast<unsigned>(nsplit), partials, arrivals);
  return check_launch("gemm");
}

// The W-streaming kernel: 16 * WAVES columns and SEG * 512 elements of K per workgroup, K slices met in the workspace.
template <int MT, int SEG, int WAVES, bool Q8 = false>
int launch_stream(hipStream_t s, const half_t* A, const half_t* W, const GemmEpilogue& ep, void* C, int64_t M, int64_t N, int64_t K) {
  const size_t tiles = static_cast<size_t>(ceil_div(N, 16 * WAVES));
  const int nsplit = static_cast<int>(ceil_div(K, SEG * 512));
  float* partials = nullptr;
  unsigned* arrivals = nullptr;
  std::unique_lock<std::recursive_mutex> ws_lock;  // held until the launch is enqueued
  if (nsplit > 1 && split_scratch(s, tiles * nsplit * (16 * MT) * (16 * WAVES) * sizeof(float), tiles, nsplit, &partials, &arrivals, &ws_lock) != 0)
    return -1;
  if (tiles * nsplit > 0x7fffffffu) return fail("gemm: too many workgroups");
  hipLaunchKernelGGL((gemm_stream_kernel<MT, SEG, WAVES, Q8>), dim3(static_cast<unsigned>(tiles * nsplit)), dim3(64 * WAVES), 0, s, A, W, ep,
                     C, M, N, K, static_cast<unsigned>(nsplit), partials, arrivals);
  return check_launch("gemm");
}

template <int MT, int WAVES, int NSTG>
int launch_stream_loop(hipStream_t s, const half_t* A, const half_t* W, const GemmEpilogue& ep, void* C, int64_t M, int64_t N, int64_t K) {
  const int64_t tiles = ceil_div(N, 16 * WAVES);
  if (tiles > 0x7fffffff) return fail("gemm: too many workgroups");
  hipLaunchKernelGGL((gemm_stream_loop_kernel<MT, WAVES, NSTG>), dim3(static_cast<unsigned>(tiles)), dim3(64 * WAVES), 0, s, A, W, ep, C, M, N, K);
  return check_launch("gemm");
}

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

// threads per workgroup of the MFMA kernel for a tile: 8 wavefronts for 256x256, else 4
inline int mfma_threads(int bm, int bn) { return bm == 256 && bn == 256 ? 512 : 256; }
// LDS stages a launch uses unless told otherwise: 2 for 256x256, 3 for 256x128, 4 below that
inline int mfma_max_stages(int bm, int bn) { return bm + bn >= 512 ? 2 : bm + bn >= 384 ? 3 : 4; }

}  // namespace

// The device address of the static scratch array on the current device.  hipGetSymbolAddress is asked once per
// device, with that device current (each GPU holds its own copy of the array at its own address).
int resolve_static_scratch(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail("static scratch: cannot identify the current device");
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (!g_static_scratch[dev]) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return fail("static scratch: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
    }
    g_static_scratch[dev] = ptr;
  }
  if (out) *out = g_static_scratch[dev];
  return 0;
}

// The 8-wavefront 256x256 tile when the library chooses: whole rounds of the chip run one workgroup per tile; the
// tiles of a last, partly filled round are shared by 2..4 workgroups each (as many as still fit the chip at once),
// which split K and meet in the workspace -- a round of half or a third the length instead of a whole one.
// Fewer tiles than CUs in all: every tile is split that way.
void tail_split_256(int64_t M, int64_t N, int64_t K, int* nsplit, unsigned* unsplit) {
  const int64_t tiles = ceil_div(M, 256) * ceil_div(N, 256), ktiles = ceil_div(K, kBK);
  const int64_t rem = tiles % kNumCU;
  *nsplit = 1;
  *unsplit = 0;
  if (rem == 0) return;
  int64_t split = kNumCU / rem;
  if (split > 4) split = 4;
  while (split >= 2 && ktiles / split < 8) --split;  // (a part should still be long against its prologue and the combine)
  // a round that fills only part of the chip runs at a higher clock; against that, parts that fill it again gain
  // only when K is long (measured: 128 tiles in two parts each break even at K = 4096 and win 20 % at K = 11008)
  if (split >= 2 && rem * split > 3 * kNumCU / 4 && ktiles < 128) return;
  if (split < 2) return;
  *nsplit = static_cast<int>(split);
  *unsplit = static_cast<unsigned>(tiles - rem);
}

// launch_args: {grid, 1, 1, block, static LDS bytes, tiles along M, tiles along N}
int describe_gemm(int64_t M, int64_t N, int64_t K, const dtas_config& cfg, int64_t la[7]) {
  for (int i = 0; i < 7; ++i) la[i] = 0;
  la[1] = la[2] = 1;
  if (cfg.vec == 1) {  // element-access fallback
    int64_t grid = ceil_div(M * N, 256);
    la[0] = grid > 65536 ? 65536 : (grid < 1 ? 1 : grid);
    la[3] = 256;
    return 0;
  }
  if (cfg.vec != 8) return fail("gemm: vector width must be 8 (128 bit) or 1, got %d", cfg.vec);
  if (cfg.variant == DTAS_GEMM_MFMA) {
    const int bm = cfg.tile[0], bn = cfg.tile[1];
    const bool known = (bm == 256 && bn == 256) || (bm == 256 && bn == 128) || (bm == 128 && bn == 256) ||
                       (bm == 128 && bn == 128) || (bm == 64 && bn == 128) || (bm == 128 && bn == 64) ||
                       (bm == 64 && bn == 64);
    if (!known || cfg.tile[2] != kBK) return fail("gemm: no MFMA kernel for tile %dx%dx%d", bm, bn, cfg.tile[2]);
    // 256x256 comes as 8 wavefronts (two per SIMD, 128x64 each) or 4 (one per SIMD, 128x128 each); 256x128 and
    // 128x256 as 4 wavefronts on whole-tile stages or 8 (64x64 each) on the 16x16x32 ring loop (128x128 on that
    // loop, 64x32 per wavefront, measured slower than on 4 wavefronts at every M: not instantiated)
    const bool four_waves = bm == 256 && bn == 256 && cfg.block == 256;
    const bool eight_waves = bm + bn == 384 && cfg.block == 512;
    if (cfg.block != mfma_threads(bm, bn) && !four_waves && !eight_waves)
      return fail("gemm: the %dx%d MFMA kernel uses %d threads, got %d", bm, bn, mfma_threads(bm, bn), cfg.block);
    if (K * 2 * (bm > bn ? bm : bn) >= (int64_t{1} << 31)) return fail("gemm: K=%lld too large for 32-bit tile offsets", (long long)K);
    const int64_t tm = ceil_div(M, bm), tn = ceil_div(N, bn);
    if (tm * tn > 0x7fffffff) return fail("gemm: too many tiles");
    // cfg.unroll = LDS stages (the depth of the load pipeline); 0 or 1 = as many as fit
    if (cfg.unroll < 0 || cfg.unroll > mfma_max_stages(bm, bn))
      return fail("gemm: the %dx%d tile holds at most %d LDS stages, got %d", bm, bn, mfma_max_stages(bm, bn), cfg.unroll);
    int nsplit = cfg.split_k < 1 ? 1 : cfg.split_k;
    if (nsplit > 16) return fail("gemm: split_k must be in [1, 16], got %d", cfg.split_k);
    // split_k = 0 on the 8-wavefront 256x256 tile: only the tiles of a last, partly filled round are split
    unsigned unsplit = 0;
    if (cfg.split_k == 0 && bm == 256 && bn == 256 && !four_waves) tail_split_256(M, N, K, &nsplit, &unsplit);
    if (tm * tn * nsplit > 0x7fffffff) return fail("gemm: too many workgroups");
    la[0] = unsplit + (tm * tn - unsplit) * nsplit;
    la[3] = four_waves ? 256 : eight_waves ? 512 : mfma_threads(bm, bn);
    // 256x256 and the 8-wavefront tiles: a ring of five operand units; else whole-tile stages
    la[4] = (bm == 256 && bn == 256) || eight_waves ? 5 * (bm > bn ? bm : bn) * kRowBytes
                                                    : (cfg.unroll >= 2 ? cfg.unroll : mfma_max_stages(bm, bn)) * (bm + bn) * kRowBytes;
    la[5] = tm;
    la[6] = tn;
    return 0;
  }
  if (cfg.variant == DTAS_GEMM_ROWS) {
    const int mv = cfg.tile[0], r = cfg.tile[1];
    if ((mv != 2 && mv != 4) || (r != 1 && r != 2 && r != 4))
      return fail("gemm: the row kernel takes tile {2,4} rows of A x {1,2,4} rows of W, got %dx%d", mv, r);
    if (M > mv) return fail("gemm: a row tile of %d rows cannot hold M=%lld", mv, (long long)M);
    if (cfg.block != 64 && cfg.block != 128 && cfg.block != 256) return fail("gemm: the row kernel uses 64, 128 or 256 threads, got %d", cfg.block);
    la[0] = ceil_div(N, static_cast<int64_t>(r) * (cfg.block / 64));
    la[3] = cfg.block;
    la[5] = 1;
    la[6] = la[0];
    if (la[0] > 0x7fffffff) return fail("gemm: too many workgroups");
    return 0;
  }
  if (cfg.variant == DTAS_GEMM_SKINNY) {
    const int mt = cfg.tile[0] / 16;
    if (cfg.tile[0] % 16 != 0 || mt < 1 || mt > 5 || cfg.tile[1] != 16)
      return fail("gemm: skinny tile must be {16,32,48,64,80}x16, got %dx%d", cfg.tile[0], cfg.tile[1]);
    if (M > cfg.tile[0]) return fail("gemm: skinny tile of %d rows cannot hold M=%lld", cfg.tile[0], (long long)M);
    if (cfg.block < 64 || cfg.block > 1024 || cfg.block % 64 != 0)
      return fail("gemm: block must be a multiple of 64 in [64, 1024], got %d", cfg.block);
    la[0] = ceil_div(N, 16);
    la[3] = cfg.block;
    la[4] = 16 * mt * 64 * 16;
    la[5] = 1;
    la[6] = la[0];
    return 0;
  }
  if (cfg.variant == DTAS_GEMM_STREAM && cfg.tile[2] == 256) {  // the looping form: the whole of K per workgroup
    const int stages = stream_loop_stages(cfg.tile[0], cfg.tile[1]);
    if (stages == 0)
      return fail("gemm: the looping W-streaming kernel takes tiles 16x64x256 and 16x16x256, got %dx%dx%d", cfg.tile[0], cfg.tile[1],
                  cfg.tile[2]);
    if (M > cfg.tile[0]) return fail("gemm: a streaming tile of %d rows cannot hold M=%lld", cfg.tile[0], (long long)M);
    if (cfg.block != 4 * cfg.tile[1]) return fail("gemm: the %d-column streaming tile uses %d threads, got %d", cfg.tile[1], 4 * cfg.tile[1], cfg.block);
    if (K * 2 * cfg.tile[1] >= (int64_t{1} << 31)) return fail("gemm: K=%lld too large for 32-bit tile offsets", (long long)K);
    const int64_t tn = ceil_div(N, cfg.tile[1]);
    if (tn > 0x7fffffff) return fail("gemm: too many workgroups");
    la[0] = tn;
    la[3] = cfg.block;
    la[4] = stages * (cfg.tile[0] + cfg.tile[1]) * 512;
    la[5] = 1;
    la[6] = tn;
    return 0;
  }
  if (cfg.variant == DTAS_GEMM_STREAM) {
    const int mt = cfg.tile[0] / 16, waves = cfg.tile[1] / 16, seg = cfg.tile[2] / 512;
    if (!stream_shape_ok(cfg.tile[0], cfg.tile[1], cfg.tile[2]))
      return fail("gemm: the W-streaming kernel takes tiles {16,32,64}x{64,128}x{512,1024} that fit the LDS, got %dx%dx%d", cfg.tile[0],
                  cfg.tile[1], cfg.tile[2]);
    if (M > cfg.tile[0]) return fail("gemm: a streaming tile of %d rows cannot hold M=%lld", cfg.tile[0], (long long)M);
    if (cfg.block != 64 * waves) return fail("gemm: the %d-column streaming tile uses %d threads, got %d", cfg.tile[1], 64 * waves, cfg.block);
    if (K * 2 * cfg.tile[1] >= (int64_t{1} << 31)) return fail("gemm: K=%lld too large for 32-bit tile offsets", (long long)K);
    const int64_t tn = ceil_div(N, cfg.tile[1]), slices = ceil_div(K, cfg.tile[2]);
    if (slices < 1 || tn * slices > 0x7fffffff) return fail("gemm: too many workgroups");
    la[0] = tn * slices;
    la[3] = cfg.block;
    la[4] = (16 * mt + 16 * waves) * seg * 1024;
    la[5] = 1;
    la[6] = tn;
    return 0;
  }
  return fail("gemm: unknown variant %d", cfg.variant);
}

}  // namespace dtas

extern "C" int dtas_gemm_f16(const void* A, const void* W, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                             const dtas_config* user, void* stream) {
  return dtas_gemm_f16_fused(A, W, bias, nullptr, nullptr, C, M, N, K, DTAS_EPI_BIAS, user, stream);
}

extern "C" int dtas_gemm_f16_static(const void* A, const void* W, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                                    const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  void* base = nullptr;
  if (resolve_static_scratch(&base) != 0) return -1;  // (a table lookup after the first call on a device, or after dtas_init)
  const FixedScratch fixed = {reinterpret_cast<float*>(static_cast<unsigned char*>(base) + DTAS_STATIC_SCRATCH_COUNTERS * 4),
                              DTAS_STATIC_SCRATCH_PARTIAL_BYTES, static_cast<unsigned*>(base), DTAS_STATIC_SCRATCH_COUNTERS};
  struct Scope {
    explicit Scope(const FixedScratch* f) { t_fixed_scratch = f; }
    ~Scope() { t_fixed_scratch = nullptr; }
  } scope(&fixed);
  return dtas_gemm_f16_fused(A, W, bias, nullptr, nullptr, C, M, N, K, DTAS_EPI_BIAS, user, stream);
}

extern "C" int dtas_gemm_f16_fused(const void* A, const void* W, const void* bias, const void* res1, const void* res2,
                                   void* C, int64_t M, int64_t N, int64_t K, int32_t epilogue, const dtas_config* user,
                                   void* stream) {
  using namespace dtas;
  clear_error();
  if (epilogue < DTAS_EPI_BIAS || epilogue > DTAS_EPI_BIAS_GELU) return fail("gemm: unknown epilogue %d", epilogue);
  const bool add2 = epilogue == DTAS_EPI_BIAS_ADD2 || epilogue == DTAS_EPI_BIAS_ADD2_CAST_F32;
  const int out_bytes = epilogue == DTAS_EPI_BIAS_ADD2_CAST_F32 ? 4 : 2;
  if (M < 0 || N < 0 || K < 0) return fail("gemm: negative extent M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (M == 0 || N == 0) return 0;
  if ((K != 0 && (M > INT64_MAX / 4 / K || N > INT64_MAX / 4 / K)) || M > INT64_MAX / 4 / N) return fail("gemm: extents overflow");
  if (!C || (K > 0 && (!A || !W))) return fail("gemm: NULL buffer");
  if (add2 && (!res1 || !res2)) return fail("gemm: the add-add epilogue needs both residual buffers");
  if (!add2 && (res1 || res2)) return fail("gemm: residual buffers given for an epilogue that takes none");
  if (overlaps(C, M * N * out_bytes, A, M * K * 2) || overlaps(C, M * N * out_bytes, W, N * K * 2) ||
      (add2 && (overlaps(C, M * N * out_bytes, res1, M * N * 2) || overlaps(C, M * N * out_bytes, res2, M * N * 2))))
    return fail("gemm: output overlaps an input");
  // one row of A is the decode GEMV: same PrimFunc shape, dedicated kernel (every epilogue)
  if (!user && M == 1) return dtas_gemv_f16_fused(A, W, bias, res1, res2, C, N, K, epilogue, nullptr, stream);
  const GemmEpilogue ep = {static_cast<const half_t*>(bias), static_cast<const half_t*>(res1),
                           static_cast<const half_t*>(res2), epilogue, out_bytes == 4 ? 1 : 0, 0.f, 0, 0, 0, 0};
  dtas_config cfg = user ? *user : builtin_config(DTAS_OP_GEMM_F16, M, N, K).cfg;
  const bool vec_ok = K % 8 == 0 && aligned(A, 16) && aligned(W, 16);
  // two rows of A (the first bucket's table row is sized for 16): W streamed in whole rows, as the GEMV does
  if (!user && M == 2 && vec_ok) cfg = dtas_config{DTAS_GEMM_ROWS, 64, 8, 1, {2, 2, 8}, 1, 0};
  if (cfg.vec == 8 && !vec_ok) cfg.vec = 1;  // K % 8 != 0 or odd pointers: element accesses
  int64_t la[7];
  if (describe_gemm(M, N, K, cfg, la) != 0) return -1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* a = static_cast<const half_t*>(A);
  const half_t* w = static_cast<const half_t*>(W);
  const GemmEpilogue& b = ep;
  void* c = C;
  if (cfg.vec == 1) {
    hipLaunchKernelGGL(gemm_scalar_kernel, dim3(static_cast<unsigned>(la[0])), dim3(256), 0, s, a, w, b, c, M, N, K, false);
    return check_launch("gemm");
  }
  if (cfg.variant == DTAS_GEMM_ROWS) {
    const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
#define DTAS_ROWS_CASE(MV_, R_) \
  if (cfg.tile[0] == MV_ && cfg.tile[1] == R_) hipLaunchKernelGGL((gemm_rows_kernel<R_, MV_>), grid, block, 0, s, a, w, b, c, M, N, K)
    DTAS_ROWS_CASE(2, 1); DTAS_ROWS_CASE(2, 2); DTAS_ROWS_CASE(2, 4);
    DTAS_ROWS_CASE(4, 1); DTAS_ROWS_CASE(4, 2); DTAS_ROWS_CASE(4, 4);
#undef DTAS_ROWS_CASE
    return check_launch("gemm");
  }
  if (cfg.variant == DTAS_GEMM_SKINNY) {
    const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
    switch (cfg.tile[0]) {
      case 16: hipLaunchKernelGGL(gemm_skinny_kernel<1>, grid, block, 0, s, a, w, b, c, M, N, K); break;
      case 32: hipLaunchKernelGGL(gemm_skinny_kernel<2>, grid, block, 0, s, a, w, b, c, M, N, K); break;
      case 48: hipLaunchKernelGGL(gemm_skinny_kernel<3>, grid, block, 0, s, a, w, b, c, M, N, K); break;
      case 64: hipLaunchKernelGGL(gemm_skinny_kernel<4>, grid, block, 0, s, a, w, b, c, M, N, K); break;
      case 80: hipLaunchKernelGGL(gemm_skinny_kernel<5>, grid, block, 0, s, a, w, b, c, M, N, K); break;
    }
    return check_launch("gemm");
  }
  if (cfg.variant == DTAS_GEMM_STREAM && cfg.tile[2] == 256) {
    if (cfg.tile[0] == 16 && cfg.tile[1] == 64) return launch_stream_loop<1, 4, 4>(s, a, w, b, c, M, N, K);
    if (cfg.tile[0] == 16 && cfg.tile[1] == 16) return launch_stream_loop<1, 1, 4>(s, a, w, b, c, M, N, K);
    return fail("gemm: no looping W-streaming kernel for tile %dx%d", cfg.tile[0], cfg.tile[1]);
  }
  if (cfg.variant == DTAS_GEMM_STREAM) {
#define DTAS_STREAM_CASE(BM_, BN_, BK_) \
  if (cfg.tile[0] == BM_ && cfg.tile[1] == BN_ && cfg.tile[2] == BK_) return launch_stream<BM_ / 16, BK_ / 512, BN_ / 16>(s, a, w, b, c, M, N, K)
    DTAS_STREAM_CASE(16, 64, 512); DTAS_STREAM_CASE(16, 64, 1024); DTAS_STREAM_CASE(16, 128, 512);
    DTAS_STREAM_CASE(32, 64, 512); DTAS_STREAM_CASE(32, 128, 512);
    DTAS_STREAM_CASE(64, 64, 512);
#undef DTAS_STREAM_CASE
    return fail("gemm: no W-streaming kernel for tile %dx%dx%d", cfg.tile[0], cfg.tile[1], cfg.tile[2]);
  }
  const int bm = cfg.tile[0], bn = cfg.tile[1];
  const int ns = cfg.unroll >= 2 ? cfg.unroll : 0;
  const int sk = cfg.split_k < 1 ? 1 : cfg.split_k;
  if (bm == 256 && bn == 256)
  {
    if (cfg.block == 256) return launch_mfma<256, 256, 2, 2, 2>(s, a, w, b, c, M, N, K, sk);
    int split = sk;
    unsigned unsplit = 0;
    if (cfg.split_k == 0) tail_split_256(M, N, K, &split, &unsplit);  // (split_k >= 1: that split for every tile)
    return launch_mfma<256, 256, 2, 4, 2, false, false, true>(s, a, w, b, c, M, N, K, split, 1, unsplit);
  }
  if (cfg.block == 512) {  // 8 wavefronts on the 16x16x32 ring loop
    if (bm == 256 && bn == 128) return launch_mfma<256, 128, 4, 2, 2, false, false, true>(s, a, w, b, c, M, N, K, sk);
    if (bm == 128 && bn == 256) return launch_mfma<128, 256, 2, 4, 2, false, false, true>(s, a, w, b, c, M, N, K, sk);
  }
  if (bm == 256 && bn == 128) return ns == 2 ? launch_mfma<256, 128, 2, 2, 2>(s, a, w, b, c, M, N, K, sk)
                                             : launch_mfma<256, 128, 2, 2, 3>(s, a, w, b, c, M, N, K, sk);
  if (bm == 128 && bn == 256) return ns == 2 ? launch_mfma<128, 256, 2, 2, 2>(s, a, w, b, c, M, N, K, sk)
                                             : launch_mfma<128, 256, 2, 2, 3>(s, a, w, b, c, M, N, K, sk);
  if (bm == 128 && bn == 128) return ns == 2   ? launch_mfma<128, 128, 2, 2, 2>(s, a, w, b, c, M, N, K, sk)
                                     : ns == 3 ? launch_mfma<128, 128, 2, 2, 3>(s, a, w, b, c, M, N, K, sk)
                                               : launch_mfma<128, 128, 2, 2, 4>(s, a, w, b, c, M, N, K, sk);
  if (bm == 64 && bn == 128) return ns == 2   ? launch_mfma<64, 128, 2, 2, 2>(s, a, w, b, c, M, N, K, sk)
                                    : ns == 3 ? launch_mfma<64, 128, 2, 2, 3>(s, a, w, b, c, M, N, K, sk)
                                              : launch_mfma<64, 128, 2, 2, 4>(s, a, w, b, c, M, N, K, sk);
  if (bm == 128 && bn == 64) return ns == 2   ? launch_mfma<128, 64, 2, 2, 2>(s, a, w, b, c, M, N, K, sk)
                                    : ns == 3 ? launch_mfma<128, 64, 2, 2, 3>(s, a, w, b, c, M, N, K, sk)
                                              : launch_mfma<128, 64, 2, 2, 4>(s, a, w, b, c, M, N, K, sk);
  if (bm == 64 && bn == 64) return ns == 2    ? launch_mfma<64, 64, 2, 2, 2>(s, a, w, b, c, M, N, K, sk)
                                   : ns == 3  ? launch_mfma<64, 64, 2, 2, 3>(s, a, w, b, c, M, N, K, sk)
                                              : launch_mfma<64, 64, 2, 2, 4>(s, a, w, b, c, M, N, K, sk);
  return fail("gemm: no MFMA kernel for tile %dx%d", bm, bn);
}

extern "C" int dtas_attn_scores_f16_f32(const void* Q, const void* Kmat, const void* mask, void* out, int64_t heads,
                                        int64_t n, int64_t m, int64_t d, float scale, const dtas_config* user,
                                        void* stream) {
  using namespace dtas;
  clear_error();
  if (heads < 0 || n < 0 || m < 0 || d < 0)
    return fail("attn_scores: negative extent heads=%lld n=%lld m=%lld d=%lld", (long long)heads, (long long)n, (long long)m, (long long)d);
  if (heads == 0 || n == 0 || m == 0) return 0;
  if (heads > 65535) return fail("attn_scores: at most 65535 heads, got %lld", (long long)heads);
  if (d > 0 && (n > INT64_MAX / 8 / d / heads || m > INT64_MAX / 8 / d / heads)) return fail("attn_scores: extents overflow");
  if (n > INT64_MAX / 8 / m / heads) return fail("attn_scores: extents overflow");
  if (!Q || !Kmat || !mask || !out) return fail("attn_scores: NULL buffer");
  if (d % 8 != 0 || !aligned(Q, 16) || !aligned(Kmat, 16))
    return fail("attn_scores: the head dimension must be a multiple of 8 and Q, K 16-byte aligned (d=%lld)", (long long)d);
  if (overlaps(out, heads * n * m * 4, Q, heads * n * d * 2) || overlaps(out, heads * n * m * 4, Kmat, heads * m * d * 2) ||
      overlaps(out, heads * n * m * 4, mask, n * m * 2))
    return fail("attn_scores: output overlaps an input");
  // the walking kernel: 128x64 tiles, at most three workgroups per CU (their LDS allows no more).  Up to 64 query
  // rows half of such a tile would be idle, and fewer tiles than CUs leave CUs idle: 64x64 tiles of the general
  // kernel then (n = 64 against 2048 keys: 6.9 us against 10.3)
  // a handful of query rows (decoding): the head's K in one sweep, R rows per workgroup (cfg: DTAS_GEMM_SKINNY, block 1024,
  // tile {1|2|4|8, 8, keys per workgroup or 0})
  auto launch_rows = [&](int R, int64_t keys_per_wg) -> int {
    const int64_t per_pass = 1024 / (d / 8);
    if (keys_per_wg <= 0) {
      // whole passes; enough workgroups to fill the chip twice, at least two passes each
      const int64_t want = ceil_div(m * heads * ceil_div(n, R), 2 * kNumCU);
      keys_per_wg = ceil_div(want < 2 * per_pass ? 2 * per_pass : want, per_pass) * per_pass;
    }
    const int64_t gx = ceil_div(m, keys_per_wg), gz = ceil_div(n, R);
    if (gx > 0x7fffffff || gz > 65535 || keys_per_wg > 0x7fffffff) return fail("attn_scores: too many workgroups for the row kernel");
    const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(heads), static_cast<unsigned>(gz));
    const half_t* q_ = static_cast<const half_t*>(Q);
    const half_t* k_ = static_cast<const half_t*>(Kmat);
    const half_t* m_ = static_cast<const half_t*>(mask);
    float* o_ = static_cast<float*>(out);
    const float sc = static_cast<float>(static_cast<half_t>(scale));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const unsigned kw = static_cast<unsigned>(keys_per_wg);
    switch (R) {
      case 1: hipLaunchKernelGGL(attn_scores_rows_kernel<1>, grid, dim3(1024), 0, st, q_, k_, m_, o_, n, m, d, sc, kw); break;
      case 2: hipLaunchKernelGGL(attn_scores_rows_kernel<2>, grid, dim3(1024), 0, st, q_, k_, m_, o_, n, m, d, sc, kw); break;
      case 4: hipLaunchKernelGGL(attn_scores_rows_kernel<4>, grid, dim3(1024), 0, st, q_, k_, m_, o_, n, m, d, sc, kw); break;
      default: hipLaunchKernelGGL(attn_scores_rows_kernel<8>, grid, dim3(1024), 0, st, q_, k_, m_, o_, n, m, d, sc, kw); break;
    }
    return check_launch("attn_scores");
  };
  if (user && user->variant == DTAS_GEMM_SKINNY) {
    const int R = user->tile[0];
    if (user->block != 1024 || user->vec != 8 || user->tile[1] != 8 || (R != 1 && R != 2 && R != 4 && R != 8))
      return fail("attn_scores: the row kernel takes block 1024, vec 8 and tile {1|2|4|8, 8, keys per workgroup}");
    if (d / 8 > 128) return fail("attn_scores: the row kernel holds head dimensions up to 1024, got %lld", (long long)d);
    if (user->tile[2] < 0 || user->tile[2] % (1024 / (d / 8)) != 0)
      return fail("attn_scores: keys per workgroup must be a multiple of the %lld keys a pass covers", (long long)(1024 / (d / 8)));
    return launch_rows(R, user->tile[2]);
  }
  // one or two rows always, three or four against many keys (with K from memory, 32 heads of 80, us: 1 row against 2048 /
  // 4096 / 8192 keys 4.7 / 7.0 / 11.6 where the 64x64 tiles take 6.0 / 10.5 / 18.8; 2 rows 5.6 / 8.3 / 14.5 against 6.1 /
  // 10.6 / 18.8; 4 rows 6.7 / 9.3 / 16.4 against 6.1 / 10.6 / 19.2; 8 rows lose: 11.1 against 6.2 at 2048)
  if (!user && d / 8 <= 128 && (n <= 2 || (n <= 4 && m >= 3072))) return launch_rows(n <= 1 ? 1 : n <= 2 ? 2 : 4, 0);
  const unsigned tm = static_cast<unsigned>(ceil_div(n, 128)), tn = static_cast<unsigned>(ceil_div(m, 64));
  const int64_t total = static_cast<int64_t>(tm) * tn * heads;
  const bool small = n <= 64 || total < kNumCU;
  if (!user && d <= 2 * kBK && !small) {
    if (total > 0x7fffffff) return fail("attn_scores: too many tiles");
    // Rows that are not whole 64-byte sectors (m % 16 != 0): neighbouring tiles each write part of the sector on their
    // common boundary, and the parts only meet in the L2 if they are written close together -- one workgroup per
    // tile, started in tile order, keeps them closer than workgroups that walk (n = m = 4097: 0.79 against 1.05 ms,
    // 3001: 0.43 / 0.53; whole sectors: walking is ahead, 122 against 135 us at 2048)
    const bool whole_sectors = m % 16 == 0 && aligned(out, 64);
    // head dimensions 80 and 96 on rows of whole sectors: the two-deep pipeline (two workgroups per CU), 2-8 % ahead
    // of three workgroups per CU that each wait out their own loads and stores (n = m = 512 / 1536 / 2048: 10.7 / 66.5 /
    // 110.5 against 11.6 / 70.0 / 113.3 us)
    if (whole_sectors && (d == 80 || d == 96)) {
      const int64_t grid_p = total < 2 * kNumCU ? total : 2 * kNumCU;
      const unsigned pin = n * m >= (int64_t{1} << 21) ? 1u : 0u;
      const half_t* q_ = static_cast<const half_t*>(Q);
      const half_t* k_ = static_cast<const half_t*>(Kmat);
      const half_t* m_ = static_cast<const half_t*>(mask);
      const float sc = static_cast<float>(static_cast<half_t>(scale));
      if (d == 80)
        hipLaunchKernelGGL(attn_scores_pipe_kernel<2>, dim3(static_cast<unsigned>(grid_p)), dim3(256), 0, static_cast<hipStream_t>(stream), q_, k_, m_,
                           static_cast<float*>(out), n, m, d, sc, tm, tn, static_cast<unsigned>(heads), pin);
      else
        hipLaunchKernelGGL(attn_scores_pipe_kernel<4>, dim3(static_cast<unsigned>(grid_p)), dim3(256), 0, static_cast<hipStream_t>(stream), q_, k_, m_,
                           static_cast<float*>(out), n, m, d, sc, tm, tn, static_cast<unsigned>(heads), pin);
      return check_launch("attn_scores");
    }
    const int64_t grid = !whole_sectors || total < 3 * kNumCU ? total : 3 * kNumCU;
    hipLaunchKernelGGL((attn_scores_kernel<128, 64>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const half_t*>(Q), static_cast<const half_t*>(Kmat), static_cast<const half_t*>(mask),
                       static_cast<float*>(out), n, m, d, static_cast<float>(static_cast<half_t>(scale)), tm, tn,
                       static_cast<unsigned>(heads), n * m >= (int64_t{1} << 21) ? 1u : 0u);
    return check_launch("attn_scores");
  }
  dtas_config cfg;
  if (user) {
    cfg = *user;
  } else {
    // the fp32 scores (4*n*m bytes per head) are what this op moves, and with two k tiles a workgroup
    // is mostly latency: measured best are 64x64 while 128x128 tiles do not give every CU a
    // workgroup, 128x128 up to ~1M scores per head, 128x64 (three workgroups per CU) beyond
    const int64_t t128 = heads * ceil_div(n, 128) * ceil_div(m, 128);
    const int bm = t128 >= kNumCU && !small ? 128 : 64, bn = t128 < kNumCU || small ? 64 : (n * m >= (int64_t{1} << 20) ? 64 : 128);
    cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 2, {bm, bn, kBK}, 1, 0};
  }
  if (cfg.variant != DTAS_GEMM_MFMA || cfg.vec != 8) return fail("attn_scores: only the MFMA kernels (vec 8) serve this op");
  if (cfg.split_k > 1) return fail("attn_scores: K is the head dimension, it is not split");
  int64_t la[7];
  if (describe_gemm(n, m, d, cfg, la) != 0) return -1;
  GemmEpilogue ep = {nullptr, static_cast<const half_t*>(mask), nullptr, kEpiScores, 1,
                     static_cast<float>(static_cast<half_t>(scale)), n * d, m * d, n * m, 0, 1,
                     // a mask beyond an L2's reach (4 MiB) is kept in place, one part per XCD; below that
                     // the heads' keys gain more from contiguous spans (measured at n = m = 512 .. 2048)
                     n * m >= (int64_t{1} << 21) ? 1u : 0u};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* a = static_cast<const half_t*>(Q);
  const half_t* w = static_cast<const half_t*>(Kmat);
  const int bm = cfg.tile[0], bn = cfg.tile[1], ns = cfg.unroll >= 2 ? cfg.unroll : 2, b = static_cast<int>(heads);
  if (bm == 256 && bn == 256)
    return cfg.block == 256 ? launch_mfma<256, 256, 2, 2, 2>(s, a, w, ep, out, n, m, d, 1, b)
                            : launch_mfma<256, 256, 2, 4, 2, false, false, true>(s, a, w, ep, out, n, m, d, 1, b);
  if (bm == 256 && bn == 128) return launch_mfma<256, 128, 2, 2, 2>(s, a, w, ep, out, n, m, d, 1, b);
  if (bm == 128 && bn == 256) return launch_mfma<128, 256, 2, 2, 2>(s, a, w, ep, out, n, m, d, 1, b);
  if (bm == 128 && bn == 128)
    return ns >= 3 ? launch_mfma<128, 128, 2, 2, 3>(s, a, w, ep, out, n, m, d, 1, b) : launch_mfma<128, 128, 2, 2, 2>(s, a, w, ep, out, n, m, d, 1, b);
  if (bm == 64 && bn == 128) return launch_mfma<64, 128, 2, 2, 2>(s, a, w, ep, out, n, m, d, 1, b);
  if (bm == 128 && bn == 64) return launch_mfma<128, 64, 2, 2, 2>(s, a, w, ep, out, n, m, d, 1, b);
  if (bm == 64 && bn == 64)
    return ns >= 3 ? launch_mfma<64, 64, 2, 2, 3>(s, a, w, ep, out, n, m, d, 1, b) : launch_mfma<64, 64, 2, 2, 2>(s, a, w, ep, out, n, m, d, 1, b);
  return fail("attn_scores: no MFMA kernel for tile %dx%d", bm, bn);
}

extern "C" int dtas_attn_pv_f16(const void* P, const void* V, void* out, int64_t heads, int64_t n, int64_t m, int64_t d,
                                const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (heads < 0 || n < 0 || m < 0 || d < 0)
    return fail("attn_pv: negative extent heads=%lld n=%lld m=%lld d=%lld", (long long)heads, (long long)n, (long long)m, (long long)d);
  if (heads == 0 || n == 0 || d == 0) return 0;
  if (heads > 65535) return fail("attn_pv: at most 65535 heads, got %lld", (long long)heads);
  if ((m > 0 && n > INT64_MAX / 8 / m / heads) || n > INT64_MAX / 8 / d / heads || (m > 0 && d > INT64_MAX / 8 / m / heads))
    return fail("attn_pv: extents overflow");
  if (!out || (m > 0 && (!P || !V))) return fail("attn_pv: NULL buffer");
  if (overlaps(out, heads * n * d * 2, P, heads * n * m * 2) || overlaps(out, heads * n * d * 2, V, heads * m * d * 2))
    return fail("attn_pv: output overlaps an input");
  const bool v_vec = d % 8 == 0 && aligned(V, 16);                  // 16-byte pieces of V's rows
  const bool p_vec = m % 8 == 0 && aligned(P, 16);                  // 16-byte pieces of P's rows
  dtas_config cfg;
  if (user) {
    cfg = *user;
  } else {
    // Fewer workgroups than CUs and many keys: the workgroups of a tile split m.  Fitted to measurements at
    // 13 .. 256 rows against 512 .. 8192 keys: a k tile costs a workgroup ~0.8 us, combining S partial tiles
    // ~3 / 5.5 / 10 us for S = 2 / 4 / 8 (16 loses everywhere).  Returns the split and its estimate in us.
    auto key_split = [](int64_t wgs, int64_t wg_limit, int64_t ktiles, double* us) {
      const double combine[4] = {0.0, 3.0, 5.5, 10.0};
      const double whole = 0.8 * static_cast<double>(ktiles);
      double best = 0.8 * whole;  // (a split has to promise a fifth less: the fit is coarse)
      int chosen = 1;
      for (int i = 1; i < 4; ++i) {
        const int split = 1 << i;
        if (wgs * split > wg_limit || ktiles < 2 * split) break;
        const double t = 0.8 * static_cast<double>(ceil_div(ktiles, split)) + combine[i];
        if (t < best) {
          best = t;
          chosen = split;
        }
      }
      *us = chosen == 1 ? whole : best;
      return chosen;
    };
    const int64_t ktiles = ceil_div(m, kBK);
    const int bn = d <= 64 ? 64 : 128;
    bool rows = false;
    if (n <= 12 && v_vec) {
      // a handful of rows (decoding, short continuations): the row kernel (two rows per workgroup, four when the
      // keys are many: ~4.5 + 0.7 n m / 1000 us and ~6 + 0.4 n m / 1000 us, measured at n = 2 .. 12 against 512 ..
      // 4096 keys) unless the 64-row MFMA tiles with their keys split come out ahead (from ~8 rows against 4096
      // keys, ~12 against 512: 15 us against 25 at n = 8, m = 4096)
      const double nm = 1e-3 * static_cast<double>(n) * static_cast<double>(m);
      const double r2 = 4.5 + 0.7 * nm, r4 = n >= 4 ? 6.0 + 0.4 * nm : 1e30;
      double mfma_us = 1e30;
      const bool mfma_ok = n >= 2 && (p_vec || (aligned(P, 2) && m >= 8));  // (any key count: P is read where it lies)
      if (mfma_ok) {
        key_split(heads, 4 * kNumCU, ktiles, &mfma_us);
        mfma_us = mfma_us + 1.5 < 5.5 ? 5.5 : mfma_us + 1.5;  // (no launch of the tiles takes less: 2 rows against 77 keys 7.5 us, the row kernel 4.6)
      }
      // 2 .. 8 rows, one workgroup per (head, row) while these fit the chip at once: a head's V in one contiguous sweep
      // per row -- or two workgroups, each with half of the pieces of a key, while those fit as well (measured with V
      // from memory, 32 heads of 80, us: 4 rows against 1024 / 2048 / 4096 keys 6.5 / 8.4 / 16.0 in halves, 7.1 / 9.6 /
      // 21.4 whole, where the row kernel takes 8.0 / 14.2 / 33.4 and the key-split tiles 19.3 at 4096; 8 rows, whole:
      // 7.2 / 9.9 / 21.1 against 12.4 / 16.7 for the tiles up to 2048 keys and 19.4 at 4096; 2 rows in halves 6.3 / 8.3 /
      // 16.2, the row kernel 6.7 / 9.1 / 19.1).  One row: the row kernel (7.0 against 8.3 us at 2048 keys: 64 workgroups
      // are too few to pull V in)
      const int64_t pieces = d / 8;
      const int halves = pieces % 2 == 0 && heads * n * 2 <= kNumCU ? 2 : 1;
      // many keys (from ~3000) and room on the chip for several workgroups per (head, row): the workgroups share the keys,
      // a run each, and meet in the split-K workspace (1 row against 4096 / 8192 keys in 8 runs 11.8 / 15.0 us, the row
      // kernel 16.8 / 30.6; 2 rows in 4 runs 12.1 / 16.9 against 16.5 / 28.0; 4 rows in 2 runs 15.1 / 23.8 against 16.3 /
      // 28.0 in halves / on the tiles; up to 2048 keys the hand-over costs more than it saves: 8.2 against 7.1)
      int runs = 1;
      while (heads * n * runs * 2 <= kNumCU && runs < 8) runs *= 2;
      if (m >= 3072 && runs >= 2 && pieces <= 128) {
        rows = true;
        cfg = dtas_config{DTAS_GEMM_SKINNY, 1024, 8, 1, {1, 8, static_cast<int32_t>(d)}, runs, 0};
      } else if (n >= 2 && n <= 8 && heads * n <= kNumCU && pieces <= 128 && (m < (halves == 2 ? 6144 : 3072) || !mfma_ok)) {
        rows = true;
        cfg = dtas_config{DTAS_GEMM_SKINNY, 1024, 8, 1, {1, 8, static_cast<int32_t>(d / halves)}, 1, 0};
      } else if (n >= 2 && n <= 8 && m >= 3072 && heads * n <= kNumCU && mfma_ok) {
        rows = false;  // (4 rows against 4096 / 8192 keys with V from memory: the row kernel 33 / 61 us, one sweep per row 22 / 39, the tiles 19 / 28)
      } else {
        rows = mfma_us >= (r2 < r4 ? r2 : r4);
        if (rows) cfg = dtas_config{DTAS_GEMM_SKINNY, 256, 8, 1, {n <= 1 ? 1 : r4 < r2 ? 4 : 2, 8, 0}, 1, 0};
      }
    }
    if (!rows) {
      // what this op moves is P (2*n*m bytes per head).  Measured over n = m = 128 .. 4096 with 32 heads of 80:
      // 64-row tiles while 128-row tiles would leave most CUs idle; 128-row tiles with three stages up to
      // one per CU; 256-row tiles with three stages beyond (n = m = 1280: 37 us against 44 for 128x128
      // with three stages and 61 with two; 2048: 74 / 79 / 98).  Head dimensions up to 64 keep the
      // 64-column tiles: two workgroups of two stages per CU
      const int64_t t128 = heads * ceil_div(n, 128);
      if (t128 <= kNumCU / 4) cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 2, {64, bn, kBK}, 1, 0};
      else if (t128 <= kNumCU && bn == 128) cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {128, 128, kBK}, 1, 0};
      else if (bn == 128) cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {256, 128, kBK}, 1, 0};
      else cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 2, {128, bn, kBK}, 1, 0};
      // 128-row tiles (one workgroup per CU) gain only while all parts run at once: 512 rows against 4096 keys
      // take 47 us in two parts, 58 whole, 80 in eight.  Partial tiles of 256 rows cost more to combine than a
      // split saves.
      const int64_t wgs = heads * ceil_div(n, cfg.tile[0]);
      const int64_t wg_limit = cfg.tile[0] <= 64 ? 4 * kNumCU : kNumCU;
      double us;
      if (wgs < kNumCU && cfg.tile[0] <= 128) cfg.split_k = key_split(wgs, wg_limit, ktiles, &us);
    }
  }
  if (cfg.vec == 8 && cfg.variant == DTAS_GEMM_SKINNY && !v_vec) cfg.vec = 1;
  if (cfg.vec == 8 && cfg.variant == DTAS_GEMM_MFMA && (!v_vec || m == 0)) cfg.vec = 1;  // m == 0: zeros
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* a = static_cast<const half_t*>(P);
  const half_t* w = static_cast<const half_t*>(V);
  half_t* c = static_cast<half_t*>(out);
  const int b = static_cast<int>(heads);
  GemmEpilogue ep = {nullptr, nullptr, nullptr, DTAS_EPI_BIAS, 0, 1.f, n * m, m * d, n * d, 0};
  // A key count that is not a multiple of 8 (or a P that is not 16-byte aligned): the direct-to-LDS loads fetch the
  // 16-byte pieces of P's rows at the rows' own 2-byte alignment, the MFMA loop covers the whole pieces (m_main keys)
  // and the epilogue adds the last m % 8
  int64_t m_main = m;
  if (cfg.vec == 8 && cfg.variant == DTAS_GEMM_MFMA && !p_vec) {
    m_main = m - m % 8;
    if (!aligned(P, 2) || m_main == 0) cfg.vec = 1;  // (the element-access kernel: correct, slow)
  }
  if (cfg.vec == 1) {
    int64_t grid = ceil_div(n * d, 256);
    grid = grid > 4096 ? 4096 : grid;
    hipLaunchKernelGGL(gemm_scalar_kernel, dim3(static_cast<unsigned>(grid), b), dim3(256), 0, s, a, w, ep, out, n, d, m, true);
    return check_launch("attn_pv");
  }
  if (cfg.vec != 8) return fail("attn_pv: vector width must be 8 (128 bit) or 1, got %d", cfg.vec);
  if (cfg.variant == DTAS_GEMM_SKINNY && (cfg.block == 1024 || cfg.tile[2] > 0)) {  // one row per workgroup, V's head in one sweep
    // tile[2] = columns per workgroup (0: all d), a multiple of 8 that divides d
    const int64_t cols = cfg.tile[2] > 0 ? cfg.tile[2] : d;
    if (cfg.tile[0] != 1 || cfg.tile[1] != 8) return fail("attn_pv: the whole-row kernel takes one row per workgroup and 8-column pieces");
    if (cfg.block != 256 && cfg.block != 512 && cfg.block != 1024) return fail("attn_pv: the whole-row kernel uses 256, 512 or 1024 threads, got %d", cfg.block);
    if (cols > cfg.block) return fail("attn_pv: the whole-row kernel stores a column per thread: %lld columns per workgroup need more than %d threads", (long long)cols, cfg.block);
    if (cols % 8 != 0 || d % cols != 0 || cols / 8 > 128) return fail("attn_pv: the whole-row kernel takes columns per workgroup that divide d, in pieces of 8, at most 1024 (d=%lld, %lld)", (long long)d, (long long)cols);
    const int nsplit = cfg.split_k < 1 ? 1 : cfg.split_k;
    if (nsplit > 64) return fail("attn_pv: the whole-row kernel splits the keys over at most 64 workgroups, got %d", nsplit);
    if (n > 65535 || heads * (d / cols) > 0x7fffffff) return fail("attn_pv: too many workgroups for the row kernel");
    const size_t tiles = static_cast<size_t>(heads * (d / cols) * n);
    float* partials = nullptr;
    unsigned* arrivals = nullptr;
    std::unique_lock<std::recursive_mutex> ws_lock;  // held until the launch is enqueued
    if (nsplit > 1 && split_scratch(s, tiles * nsplit * cols * sizeof(float), tiles, nsplit, &partials, &arrivals, &ws_lock) != 0) return -1;
    hipLaunchKernelGGL(attn_pv_whole_row_kernel, dim3(static_cast<unsigned>(heads * (d / cols)), static_cast<unsigned>(n), static_cast<unsigned>(nsplit)),
                       dim3(cfg.block), 0, s, a, w, c, n, m, d, static_cast<unsigned>(cols), static_cast<unsigned>(nsplit), partials, arrivals);
    return check_launch("attn_pv");
  }
  if (cfg.variant == DTAS_GEMM_SKINNY) {
    const int R = cfg.tile[0];
    if (cfg.block != 256 || cfg.tile[1] != 8) return fail("attn_pv: the row kernel uses 256 threads and 8-column pieces");
    if (R != 1 && R != 2 && R != 4 && R != 8) return fail("attn_pv: the row kernel takes 1, 2, 4 or 8 rows per workgroup, got %d", R);
    if (cfg.split_k > 1) return fail("attn_pv: the row kernel does not split K");
    const int64_t blocks = ceil_div(n, R);
    if (heads * (d / 8) > 0x7fffffff || blocks > 65535) return fail("attn_pv: too many workgroups for the row kernel");
    const dim3 grid(static_cast<unsigned>(heads * (d / 8)), static_cast<unsigned>(blocks));
    switch (R) {
      case 1: hipLaunchKernelGGL(attn_pv_rows_kernel<1>, grid, dim3(256), 0, s, a, w, c, n, m, d); break;
      case 2: hipLaunchKernelGGL(attn_pv_rows_kernel<2>, grid, dim3(256), 0, s, a, w, c, n, m, d); break;
      case 4: hipLaunchKernelGGL(attn_pv_rows_kernel<4>, grid, dim3(256), 0, s, a, w, c, n, m, d); break;
      default: hipLaunchKernelGGL(attn_pv_rows_kernel<8>, grid, dim3(256), 0, s, a, w, c, n, m, d); break;
    }
    return check_launch("attn_pv");
  }
  if (cfg.variant != DTAS_GEMM_MFMA) return fail("attn_pv: unknown variant %d", cfg.variant);
  const int sk = cfg.split_k < 1 ? 1 : cfg.split_k;
  if (cfg.unroll > 3) return fail("attn_pv: the transposing kernels hold two or three LDS stages, got %d", cfg.unroll);
  if (m * d >= (int64_t{1} << 31)) return fail("attn_pv: a head's V exceeds the 4 GiB a buffer descriptor spans");
  int64_t la[7];
  if (describe_gemm(n, d, m, cfg, la) != 0) return -1;
  const int bm = cfg.tile[0], bn = cfg.tile[1];
  const bool three = cfg.unroll == 3;
  ep.lda = m;
  ep.k_tail = static_cast<unsigned>(m - m_main);
  if (bm == 256 && bn == 128 && three) return launch_mfma<256, 128, 2, 2, 3, true>(s, a, w, ep, out, n, d, m_main, sk, b);
  if (bm == 128 && bn == 128 && three) return launch_mfma<128, 128, 2, 2, 3, true>(s, a, w, ep, out, n, d, m_main, sk, b);
  if (three) return fail("attn_pv: three stages come with the 256x128 and 128x128 tiles, got %dx%d", bm, bn);
  if (bm == 128 && bn == 128) return launch_mfma<128, 128, 2, 2, 2, true>(s, a, w, ep, out, n, d, m_main, sk, b);
  if (bm == 64 && bn == 128) return launch_mfma<64, 128, 2, 2, 2, true>(s, a, w, ep, out, n, d, m_main, sk, b);
  if (bm == 128 && bn == 64) return launch_mfma<128, 64, 2, 2, 2, true>(s, a, w, ep, out, n, d, m_main, sk, b);
  if (bm == 64 && bn == 64) return launch_mfma<64, 64, 2, 2, 2, true>(s, a, w, ep, out, n, d, m_main, sk, b);
  return fail("attn_pv: no transposing MFMA kernel for tile %dx%d", bm, bn);
}

extern "C" int dtas_gemm_q8_f16_fused(const void* A, const void* Wq, const void* scale, const void* bias, const void* res1,
                                      const void* res2, void* C, int64_t M, int64_t N, int64_t K, int32_t epilogue,
                                      const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (M < 0 || N < 0 || K < 0) return fail("gemm_q8: negative extent M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (K % 32 != 0) return fail("gemm_q8: K must be a multiple of the scale group, 32 (K=%lld)", (long long)K);
  if (epilogue < DTAS_EPI_BIAS || epilogue > DTAS_EPI_BIAS_GELU) return fail("gemm_q8: unknown epilogue %d", epilogue);
  if (M == 0 || N == 0) return 0;
  if ((K != 0 && (M > INT64_MAX / 8 / K || N > INT64_MAX / 8 / K)) || M > INT64_MAX / 8 / N) return fail("gemm_q8: extents overflow");
  const bool add2 = epilogue == DTAS_EPI_BIAS_ADD2 || epilogue == DTAS_EPI_BIAS_ADD2_CAST_F32;
  if (!A || !Wq || !scale || !C) {
    if (K > 0 || !C) return fail("gemm_q8: NULL buffer");
  }
  if (add2 && (!res1 || !res2)) return fail("gemm_q8: epilogue %d needs both residuals", epilogue);
  if (!add2 && (res1 || res2)) return fail("gemm_q8: epilogue %d takes no residuals", epilogue);
  const int out_bytes = epilogue == DTAS_EPI_BIAS_ADD2_CAST_F32 ? 4 : 2;
  if (overlaps(C, M * N * out_bytes, A, M * K * 2) || overlaps(C, M * N * out_bytes, Wq, N * K) ||
      overlaps(C, M * N * out_bytes, scale, N * (K / 32) * 2) ||
      (add2 && (overlaps(C, M * N * out_bytes, res1, M * N * 2) || overlaps(C, M * N * out_bytes, res2, M * N * 2))))
    return fail("gemm_q8: output overlaps an input");
  // one row with a plain or GELU epilogue is the dequantising GEMV
  if (!user && M == 1 && (epilogue == DTAS_EPI_BIAS || epilogue == DTAS_EPI_BIAS_GELU))
    return dtas_gemv_q8_f16(A, Wq, scale, bias, C, N, K, epilogue, nullptr, stream);
  GemmEpilogue ep = {static_cast<const half_t*>(bias), static_cast<const half_t*>(res1), static_cast<const half_t*>(res2),
                     epilogue, out_bytes == 4 ? 1 : 0, 0.f, 0, 0, 0, 0, 1, 0, static_cast<const half_t*>(scale)};
  // Few rows of A: the launch is one read of the bytes of W.  The W-streaming kernel widens them on their way
  // from the LDS into the MFMA (cfg: DTAS_GEMM_STREAM with tile 16x64x512, 16x64x1024 or 32x64x512).
  {
    const bool stream_ok = K > 0 && K % 256 == 0 && aligned(A, 16) && aligned(Wq, 16) && aligned(scale, 16) && K < (int64_t{1} << 24);
    const half_t* a = static_cast<const half_t*>(A);
    const half_t* w = static_cast<const half_t*>(Wq);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (user && user->variant == DTAS_GEMM_STREAM) {
      const int bm = user->tile[0], bn = user->tile[1], bk = user->tile[2];
      if (!((bm == 16 && bn == 64 && (bk == 512 || bk == 1024)) || ((bm == 32 || bm == 64) && bn == 64 && bk == 512)))
        return fail("gemm_q8: the W-streaming kernel takes tiles 16x64x512, 16x64x1024, 32x64x512 and 64x64x512 for 8-bit weights, got %dx%dx%d", bm, bn, bk);
      if (user->block != 256) return fail("gemm_q8: the 64-column streaming tile uses 256 threads, got %d", user->block);
      if (M > bm) return fail("gemm_q8: a streaming tile of %d rows cannot hold M=%lld", bm, (long long)M);
      if (!stream_ok) return fail("gemm_q8: the W-streaming kernel needs K %% 256 == 0 and 16-byte aligned A, W and scales");
      if (bm == 64) return launch_stream<4, 1, 4, true>(s, a, w, ep, C, M, N, K);
      if (bm == 32) return launch_stream<2, 1, 4, true>(s, a, w, ep, C, M, N, K);
      return bk == 512 ? launch_stream<1, 1, 4, true>(s, a, w, ep, C, M, N, K) : launch_stream<1, 2, 4, true>(s, a, w, ep, C, M, N, K);
    }
    if (!user && stream_ok && M <= 32) {
      // measured at the model's shapes (M = 16: 10.1 against 25.6 us at 7680x2560, 14.9 against 92 at 2560x10240;
      // M = 32: 14.0 against 26.3 and 20.5 against 33.8).  512-element slices (three workgroups per CU) unless K is
      // long: from 16 slices on the hand-over of the partial sums costs more than the second workgroup hides
      if (M > 16) return launch_stream<2, 1, 4, true>(s, a, w, ep, C, M, N, K);
      if (K >= 8192) return launch_stream<1, 2, 4, true>(s, a, w, ep, C, M, N, K);
      return launch_stream<1, 1, 4, true>(s, a, w, ep, C, M, N, K);
    }
    // up to 64 rows (one workgroup per CU) only where the column tiles number at most a quarter of the CUs' slots:
    // 14.0 against 26.3 us at 64 x 2560 x 2560 and 25.1 against 39.5 at 4096 x 4096, but 38 against 27 at N = 10240
    if (!user && stream_ok && M <= 64 && N <= 4096 && K <= 4096) return launch_stream<4, 1, 4, true>(s, a, w, ep, C, M, N, K);
  }
  // Two routes.  Dequantising in the W path of the GEMM (no intermediate) runs on a plain burst pipeline without
  // split K: measured at the model's shapes it wins for M <= 64 with K <= 4096 (18 against 24 us at 7680x2560)
  // and loses beyond (M = 2048: 109 against 84 us; K = 10240: 2x or more).  Otherwise: the dequantiser into a
  // library-owned fp16 buffer, then the fp16 GEMM with everything its table offers.  A cfg selects the first route.
  if (!user && !(M <= 64 && K <= 4096)) {
    void* wbuf = nullptr;
    std::lock_guard<std::recursive_mutex> ws_lock(g_ws_mutex);  // until both launches are enqueued
    if (operand_workspace(static_cast<hipStream_t>(stream), static_cast<size_t>(N) * K * 2, &wbuf) != 0) return -1;
    if (dtas_decode_q8_f16(Wq, scale, wbuf, N, K, nullptr, stream) != 0) return -1;
    return dtas_gemm_f16_fused(A, wbuf, bias, res1, res2, C, M, N, K, epilogue, nullptr, stream);
  }
  dtas_config cfg = user ? *user : dtas_config{DTAS_GEMM_MFMA, 256, 8, 2, {64, 64, kBK}, 1, 0};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* a = static_cast<const half_t*>(A);
  const half_t* w = static_cast<const half_t*>(Wq);  // (bytes; the kernels take the pointer as they take fp16 W)
  const bool vec_ok = aligned(A, 16) && aligned(Wq, 16) && aligned(scale, 2) && N * K < (int64_t{1} << 32) && K > 0;
  if (cfg.vec == 8 && !vec_ok) cfg.vec = 1;
  if (cfg.vec == 1) {
    int64_t grid = ceil_div(M * N, 256);
    grid = grid > 65536 ? 65536 : grid;
    hipLaunchKernelGGL(gemm_scalar_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, s, a, w, ep, C, M, N, K, false);
    return check_launch("gemm_q8");
  }
  if (cfg.vec != 8) return fail("gemm_q8: vector width must be 8 (128 bit) or 1, got %d", cfg.vec);
  if (cfg.variant != DTAS_GEMM_MFMA) return fail("gemm_q8: only the MFMA kernels serve 8-bit weights");
  if (cfg.split_k > 1) return fail("gemm_q8: K is not split for 8-bit weights");
  int64_t la[7];
  if (describe_gemm(M, N, K, cfg, la) != 0) return -1;
  const int bm = cfg.tile[0], bn = cfg.tile[1];
  if (bm == 256 && bn == 128 && cfg.unroll == 3) return launch_mfma<256, 128, 2, 2, 3, false, true>(s, a, w, ep, C, M, N, K, 1);
  if (bm == 128 && bn == 128 && cfg.unroll == 3) return launch_mfma<128, 128, 2, 2, 3, false, true>(s, a, w, ep, C, M, N, K, 1);
  if (bm == 64 && bn == 64 && cfg.unroll == 2) return launch_mfma<64, 64, 2, 2, 2, false, true>(s, a, w, ep, C, M, N, K, 1);
  return fail("gemm_q8: 8-bit weights come with tiles 256x128 and 128x128 (three stages) and 64x64 (two), got %dx%d with %d", bm, bn, cfg.unroll);
}

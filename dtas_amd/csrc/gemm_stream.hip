// The GEMM kernels that stream W once, for few rows of A (C[M,N] = A[M,K] . W[N,K]^T, fp16, fp32 accumulation):
// SKINNY kernel (M <= 80): a workgroup owns 16 columns of C and all of M, its wavefronts split K,
//              v_mfma_f32_16x16x32_f16 operands are loaded straight from global memory, partial tiles are folded
//              through the LDS.
// STREAM kernel (M <= 64; the built-in choice for M <= 16): W rows come in as 1 KiB direct-to-LDS loads, everything
//              a workgroup needs requested at once; K slices meet in the workspace.  With 8-bit weights (M <= 32)
//              the bytes ride the same loads and are widened between the LDS and the MFMA.  For a W with many rows
//              (4096 < N <= 16384, K <= 4096) the looping form: a workgroup keeps its columns over the whole of K,
//              walked through a ring of LDS stages.
// ROWS kernel (M <= 4; the built-in choice for M = 2): W streamed in whole rows on the vector ALU.
// The element-access kernel (any K and alignment; k-major or 8-bit W as well) is here too, and the kernel that keeps
// the reference's fp16 accumulator (DTAS_GEMM_MFMA_ACC16).
// Replaces, for these shapes, the kernels DTAS's WMMA rule generates (python/dtas/schedule/tir_wmma.py:20-222), which
// pad M up to a whole tile.
#include "gemm_common.h"

namespace dtas {
namespace {

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

// The reference's scheduled GEMM arithmetic (DTAS_GEMM_MFMA_ACC16): its WMMA rule keeps the accumulator fragment in fp16
// and updates it with one 16x16x16 tensor-core instruction per k step (python/dtas/schedule/tir_wmma.py:20-222; the
// generated kernel experiment/testIR/GEMM/m_n2560_k10240/wmma/16x16x16/i2j4_x7y2_in8.py:19,37).  Here a k step of 16 is
// one v_mfma_f32_32x32x16_f16 whose sums are rounded to fp16 (and widened again) before the next step reads them, so
// every step's 16 products meet the accumulator at fp32 precision and the result is rounded once per step.
// Workgroup = 64 x 64 of C, a wavefront 32 x 32; lane l supplies row (l & 31), elements 8 * (l >> 5) .. + 8 of the
// step for both operands, straight from global memory (W rows are the first MFMA operand: accumulator register 4 g + e
// of lane l is C row l & 31, column 8 g + 4 (l >> 5) + e).  Nothing is pipelined: a step waits for its rounding.
template <bool VEC>
__global__ void __launch_bounds__(256) gemm_acc16_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W, GemmEpilogue ep,
                                                         void* __restrict__ C, int64_t M, int64_t N, int64_t K, unsigned tiles_n) {
  const unsigned t = threadIdx.x, l = t & 63u, wv = t >> 6;
  const int64_t m0 = static_cast<int64_t>(blockIdx.x / tiles_n) * 64 + (wv >> 1) * 32;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x % tiles_n) * 64 + (wv & 1u) * 32;
  if (m0 >= M || n0 >= N) return;  // (no barrier below: a wavefront without work just leaves)
  const int64_t arow = m0 + (l & 31u) < M ? m0 + (l & 31u) : M - 1;  // clamped rows are computed and never stored
  const int64_t wrow = n0 + (l & 31u) < N ? n0 + (l & 31u) : N - 1;
  const half_t* ap = A + arow * K + 8 * (l >> 5);
  const half_t* wp = W + wrow * K + 8 * (l >> 5);
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  for (int64_t k0 = 0; k0 < K; k0 += 16) {
    const int64_t k = k0 + 8 * (l >> 5);
    f16x8 fa, fw;
    if (VEC) {  // K % 8 == 0: a lane's 8 elements are all inside the row or all past its end
      const f16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
      fa = k < K ? *reinterpret_cast<const f16x8*>(ap + k0) : zero;
      fw = k < K ? *reinterpret_cast<const f16x8*>(wp + k0) : zero;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        fa[e] = k + e < K ? ap[k0 + e] : static_cast<half_t>(0.f);
        fw[e] = k + e < K ? wp[k0 + e] : static_cast<half_t>(0.f);
      }
    }
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw, fa, acc, 0, 0, 0);
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = static_cast<float>(static_cast<half_t>(acc[v]));
  }
  const int64_t row = m0 + (l & 31u);
  if (row >= M) return;
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int64_t col = n0 + 8 * g + 4 * (l >> 5) + e;
      if (col < N) finish(acc[4 * g + e], ep, C, row, col, N);
    }
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

}  // namespace

int launch_gemm_rows(const dtas_config& cfg, const int64_t la[7], hipStream_t s, const half_t* a, const half_t* w,
                     const GemmEpilogue& b, void* c, int64_t M, int64_t N, int64_t K) {
  const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
#define DTAS_ROWS_CASE(MV_, R_) \
  if (cfg.tile[0] == MV_ && cfg.tile[1] == R_) hipLaunchKernelGGL((gemm_rows_kernel<R_, MV_>), grid, block, 0, s, a, w, b, c, M, N, K)
  DTAS_ROWS_CASE(2, 1); DTAS_ROWS_CASE(2, 2); DTAS_ROWS_CASE(2, 4);
  DTAS_ROWS_CASE(4, 1); DTAS_ROWS_CASE(4, 2); DTAS_ROWS_CASE(4, 4);
#undef DTAS_ROWS_CASE
  return check_launch("gemm");
}

int launch_gemm_skinny(const dtas_config& cfg, const int64_t la[7], hipStream_t s, const half_t* a, const half_t* w,
                       const GemmEpilogue& b, void* c, int64_t M, int64_t N, int64_t K) {
  const dim3 grid(static_cast<unsigned>(la[0])), block(static_cast<unsigned>(la[3]));
  switch (cfg.tile[0]) {
    case 16: hipLaunchKernelGGL(gemm_skinny_kernel<1>, grid, block, 0, s, a, w, b, c, M, N, K); break;
    case 32: hipLaunchKernelGGL(gemm_skinny_kernel<2>, grid, block, 0, s, a, w, b, c, M, N, K); break;
    case 48: hipLaunchKernelGGL(gemm_skinny_kernel<3>, grid, block, 0, s, a, w, b, c, M, N, K); break;
    case 64: hipLaunchKernelGGL(gemm_skinny_kernel<4>, grid, block, 0, s, a, w, b, c, M, N, K); break;
    case 80: hipLaunchKernelGGL(gemm_skinny_kernel<5>, grid, block, 0, s, a, w, b, c, M, N, K); break;
    default: return fail("gemm: no skinny kernel for %d rows", cfg.tile[0]);
  }
  return check_launch("gemm");
}

int launch_gemm_stream(const dtas_config& cfg, hipStream_t s, const half_t* a, const half_t* w, const GemmEpilogue& b, void* c,
                       int64_t M, int64_t N, int64_t K) {
  if (cfg.tile[2] == 256) {
    if (cfg.tile[0] == 16 && cfg.tile[1] == 64) return launch_stream_loop<1, 4, 4>(s, a, w, b, c, M, N, K);
    if (cfg.tile[0] == 16 && cfg.tile[1] == 16) return launch_stream_loop<1, 1, 4>(s, a, w, b, c, M, N, K);
    return fail("gemm: no looping W-streaming kernel for tile %dx%d", cfg.tile[0], cfg.tile[1]);
  }
#define DTAS_STREAM_CASE(BM_, BN_, BK_) \
  if (cfg.tile[0] == BM_ && cfg.tile[1] == BN_ && cfg.tile[2] == BK_) return launch_stream<BM_ / 16, BK_ / 512, BN_ / 16>(s, a, w, b, c, M, N, K)
  DTAS_STREAM_CASE(16, 64, 512); DTAS_STREAM_CASE(16, 64, 1024); DTAS_STREAM_CASE(16, 128, 512);
  DTAS_STREAM_CASE(32, 64, 512); DTAS_STREAM_CASE(32, 128, 512);
  DTAS_STREAM_CASE(64, 64, 512);
#undef DTAS_STREAM_CASE
  return fail("gemm: no W-streaming kernel for tile %dx%dx%d", cfg.tile[0], cfg.tile[1], cfg.tile[2]);
}

int launch_gemm_stream_q8(int rows_a, int k_slice, hipStream_t s, const half_t* a, const half_t* wq, const GemmEpilogue& ep, void* C,
                          int64_t M, int64_t N, int64_t K) {
  if (rows_a == 64 && k_slice == 512) return launch_stream<4, 1, 4, true>(s, a, wq, ep, C, M, N, K);
  if (rows_a == 32 && k_slice == 512) return launch_stream<2, 1, 4, true>(s, a, wq, ep, C, M, N, K);
  if (rows_a == 16 && k_slice == 512) return launch_stream<1, 1, 4, true>(s, a, wq, ep, C, M, N, K);
  if (rows_a == 16 && k_slice == 1024) return launch_stream<1, 2, 4, true>(s, a, wq, ep, C, M, N, K);
  return fail("gemm_q8: no W-streaming kernel for %d rows and K slices of %d", rows_a, k_slice);
}

int launch_gemm_acc16(const dtas_config& cfg, hipStream_t s, const half_t* a, const half_t* w, const GemmEpilogue& ep, void* C,
                      int64_t M, int64_t N, int64_t K) {
  const int64_t tm = ceil_div(M, 64), tn = ceil_div(N, 64);
  if (tm * tn > 0x7fffffff || tn > 0x7fffffff) return fail("gemm: too many workgroups");
  const dim3 grid(static_cast<unsigned>(tm * tn)), block(256);
  if (cfg.vec == 8) hipLaunchKernelGGL(gemm_acc16_kernel<true>, grid, block, 0, s, a, w, ep, C, M, N, K, static_cast<unsigned>(tn));
  else hipLaunchKernelGGL(gemm_acc16_kernel<false>, grid, block, 0, s, a, w, ep, C, M, N, K, static_cast<unsigned>(tn));
  return check_launch("gemm");
}

int launch_gemm_scalar(const char* what, unsigned grid_x, unsigned batch, hipStream_t s, const half_t* a, const half_t* w,
                       const GemmEpilogue& ep, void* C, int64_t M, int64_t N, int64_t K, bool w_kmajor) {
  hipLaunchKernelGGL(gemm_scalar_kernel, dim3(grid_x, batch), dim3(256), 0, s, a, w, ep, C, M, N, K, w_kmajor);
  return check_launch(what);
}

}  // namespace dtas

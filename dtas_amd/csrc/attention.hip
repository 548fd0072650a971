// The two batched attention matmuls for gfx950, all heads in one launch:
//   scores : fused_NT_matmul1_divide_maximum_minimum_cast2 (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:116-160),
//            out[h] = fp32(min(max(fp16(Q[h] . K[h]^T * scale), -65504), mask)), n query rows and m keys both dynamic;
//   P.V    : matmul8 / matmul10 (before_dl.py:899-929), out[h] = P[h] . V[h] with V k-major.
// attn_scores_kernel (Q.K^T for head dimensions up to 128, walking tiles; attn_scores_pipe_kernel: its two-deep
// pipeline for head dimensions 80 and 96), attn_scores_rows_kernel (a handful of query rows: a workgroup sweeps a run
// of the head's keys), attn_pv_rows_kernel (P.V for one or two query rows) and attn_pv_whole_row_kernel (P.V for a few
// query rows: a workgroup sweeps the head's V, the keys shared between workgroups when they are many).  Everything
// else runs on the GEMM family's tile kernel: the scores through its row-major instantiations (gemm_tiles.hip) with
// the scores epilogue, P.V through the k-major instantiations made here (template flag WT: V tiles are transposed on
// their way into the LDS).
#include "gemm_tile_kernel.h"

namespace dtas {
namespace {

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

}  // namespace
}  // namespace dtas

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
      // (whole passes can leave a few workgroups more than two per CU, and those few a round of their own -- 40 heads of
      // 128 against 4096 keys: 13 x 40 = 520 workgroups, 16.2 us; 11 x 40: 13.3 -- so the keys are dealt to no more
      // workgroups than fit at once)
      const int64_t per_key_run = heads * ceil_div(n, R);
      if (per_key_run <= 2 * kNumCU && ceil_div(m, keys_per_wg) * per_key_run > 2 * kNumCU)
        keys_per_wg = ceil_div(ceil_div(m, (2 * kNumCU) / per_key_run), per_pass) * per_pass;
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
    if (d < 8 || d / 8 > 128) return fail("attn_scores: the row kernel holds head dimensions from 8 to 1024, got %lld", (long long)d);
    if (user->tile[2] < 0 || user->tile[2] % (1024 / (d / 8)) != 0)
      return fail("attn_scores: keys per workgroup must be a multiple of the %lld keys a pass covers", (long long)(1024 / (d / 8)));
    return launch_rows(R, user->tile[2]);
  }
  // one or two rows always, three or four against many keys (with K from memory, 32 heads of 80, us: 1 row against 2048 /
  // 4096 / 8192 keys 4.7 / 7.0 / 11.6 where the 64x64 tiles take 6.0 / 10.5 / 18.8; 2 rows 5.6 / 8.3 / 14.5 against 6.1 /
  // 10.6 / 18.8; 4 rows 6.7 / 9.3 / 16.4 against 6.1 / 10.6 / 19.2; 8 rows lose: 11.1 against 6.2 at 2048)
  // (head dimensions above 96: one row only -- 32 heads of 128, 4 rows against 4096 keys: 16.2 us where the 64x64 tiles take 11.3,
  // 2 rows against 2048: 7.3 / 6.6; one row 9.9 / 11.2)
  if (!user && d >= 8 && d / 8 <= 128 && (d <= 96 ? (n <= 2 || (n <= 4 && m >= 3072)) : n <= 1)) return launch_rows(n <= 1 ? 1 : n <= 2 ? 2 : 4, 0);
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
  // two stages (two k tiles per head dimension up to 128), three on request for the 128x128 and 64x64 tiles; 4 wavefronts
  const bool deep = (cfg.tile[0] == cfg.tile[1]) && (cfg.tile[0] == 128 || cfg.tile[0] == 64) && cfg.unroll >= 3;
  cfg.unroll = deep ? 3 : 2;
  if (cfg.tile[0] + cfg.tile[1] == 384) cfg.block = 256;
  cfg.split_k = 1;
  return launch_tile_f16(cfg, s, a, w, ep, out, n, m, d, static_cast<int>(heads));
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
      // (n m as it weighs with 32 heads of 80, where these were measured: the row kernels' time goes with the heads and the
      // head dimension -- 8 rows against 2048 keys, 40 heads of 128: 37.5 us on the row kernel, 12.6 on the tiles)
      const double nm = 1e-3 * static_cast<double>(n) * static_cast<double>(m) * (static_cast<double>(heads * d) / (32.0 * 80.0));
      // (one row, the one-row form of the row kernel: 1.6 + 2.9 nm -- 7.3 / 10.9 / 14.9 / 20.0 us against 2048 keys with 32 heads of 80 / 32 / 40 / 64 heads of 128)
      const double r2 = n == 1 ? 1.6 + 2.9 * nm : 4.5 + 0.7 * nm, r4 = n >= 4 ? 6.0 + 0.4 * nm : 1e30;
      double mfma_us = 1e30;
      const bool mfma_ok = p_vec || (aligned(P, 2) && m >= 8);  // (any key count: P is read where it lies)
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
      // (a workgroup's sweep of V, keys x head dimension, is what the whole-row forms pay for: the limits below are the 3072 /
      // 6144 / 4096 keys of 80 they were measured at -- 8 rows against 8192 keys, 16 heads of 128, in 2 runs: 33.2 us, the tiles 18.8)
      const int64_t md = m * d, kMd = 80;
      const double whole_row_runs_us = 7.0 + 5e-5 * static_cast<double>(ceil_div(m, runs) * d) + 0.5 * runs;  // (4 rows of 128 against 4096 keys in 2 runs: 20.7 us, the tiles 16.0; 4 rows of 80 against 8192: 23.4 / 19.2)
      if (m >= 3072 && runs >= 2 && pieces <= 128 && (!mfma_ok || whole_row_runs_us <= mfma_us)) {
        rows = true;
        cfg = dtas_config{DTAS_GEMM_SKINNY, 1024, 8, 1, {1, 8, static_cast<int32_t>(d)}, runs, 0};
      } else if (n >= 2 && n <= 8 && heads * n <= kNumCU && pieces <= 128 && (md < (halves == 2 ? 6144 : 3072) * kMd || !mfma_ok)) {
        rows = true;
        cfg = dtas_config{DTAS_GEMM_SKINNY, 1024, 8, 1, {1, 8, static_cast<int32_t>(d / halves)}, 1, 0};
      } else if (n >= 2 && n <= 8 && md >= 3072 * kMd && heads * n <= kNumCU && mfma_ok) {
        rows = false;  // (4 rows against 4096 / 8192 keys with V from memory: the row kernel 33 / 61 us, one sweep per row 22 / 39, the tiles 19 / 28)
      } else {
        rows = mfma_us >= (r2 < r4 ? r2 : r4);
        if (rows) cfg = dtas_config{DTAS_GEMM_SKINNY, 256, 8, 1, {n <= 1 ? 1 : r4 < r2 ? 4 : 2, 8, 0}, 1, 0};
      }
    }
    if (!rows) {
      // what this op moves is P (2*n*m bytes per head).  Measured over n = m = 128 .. 4096 with 32 heads of 80:
      // 64-row tiles (three stages) while 128-row tiles would leave half of the CUs idle (n = m = 512: 8.9 us against
      // 11.0 for 128x128); 128-row tiles with three stages up to one per CU; 256-row tiles with three stages beyond
      // (n = m = 1280: 30.5 us against 37.9 for 128x128 with three stages and 47.0 with two; 2048: 73 / 75 / 82, every
      // tile within 5 %: there the launch is bound by how P streams in, 128 bytes of a row per request).  Head dimensions up to 64 keep the
      // 64-column tiles: two workgroups of two stages per CU
      const int64_t t128 = heads * ceil_div(n, 128);
      bool fitted = false;
      if (bn == 128 && t128 <= kNumCU) {
        // Up to one 128-row tile per CU (n <= 1024 with 32 heads): 64x128 and 128x128 with three stages or 64x64 with two, the
        // keys in 1 / 2 / 4 / 8 parts, by us = start + (k tiles per part) x (cost of one at that many workgroups) + hand-over,
        // fitted to a sweep of n = 16 .. 768 against 512 .. 8192 keys (32 heads of 80, P and V from memory).  Measured, new /
        // old choice: 256 rows against 1024 / 4096 / 8192 keys 12.1 / 26.7 / 42.9 us (16.7 / 42.4 / 61.5), 384 against 1024 /
        // 2048 / 4096 13.2 / 21.4 / 31.2 (24.6 / 33.3 / 43.7), 128 against 4096 18.9 (24.6), 128 x 128 4.7 (6.3)
        // (the constants refitted over 16 / 32 / 40 / 64 heads of 128 as well: mean ratio to the best of 28 configurations 1.004 /
        // 1.006 / 1.013 / 1.035 -- 1.010 / 1.009 / 1.051 / 1.042 with the first fit -- and 1.001 still on the 32 heads of 80)
        const double hand64[4] = {0.0, 1.6, 4.0, 4.9}, hand[4] = {0.0, 2.1, 3.9, 7.8}, hand128[4] = {0.0, 3.4, 8.0, 16.0};
        const int64_t t64 = heads * ceil_div(n, 64);
        double best = 1e30;
        for (int i = 0; i < 4; ++i) {
          const int parts = 1 << i;
          if (i > 0 && ktiles < 2 * parts) break;
          const double steps = static_cast<double>(ceil_div(ktiles, parts));
          const double w64 = static_cast<double>(t64 * parts), w128 = static_cast<double>(t128 * parts);
          // 64x64, two stages: short sweeps on a chip that is not full
          const double us_a = w64 <= 128 && steps <= 8 ? 4.2 + (0.3 + 0.3 * w64 / 192.0) * steps + hand64[i] : 1e30;
          // 64x128, three stages (two workgroups per CU)
          const double us_b = w64 <= 2 * kNumCU ? 5.7 + 0.51 * (w64 <= kNumCU ? 1.0 : 1.25 * w64 / kNumCU) * steps + hand[i] : 1e30;
          // 128x128, three stages (one per CU)
          const double us_c = w128 <= kNumCU ? 7.4 + (0.45 + 0.335 * (w128 / kNumCU) * (w128 / kNumCU)) * steps + hand128[i] : 1e30;
          if (us_a < best) best = us_a, cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 2, {64, 64, kBK}, parts, 0};
          if (us_b < best) best = us_b, cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {64, 128, kBK}, parts, 0};
          if (us_c < best) best = us_c, cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {128, 128, kBK}, parts, 0};
        }
        fitted = true;
      } else if (t128 <= kNumCU / 2) {
        cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, bn == 128 ? 3 : 2, {64, bn, kBK}, 1, 0};
        if (bn == 64) {
          // head dimensions up to 64: the 64x64 term of the fit above, the keys in parts while the workgroups number at most
          // two per CU (32 heads of 64: 256 rows against 4096 keys 30.3 -> 24.4 us in 4 parts, 512 against 2048 28.2 -> 21.4 in 2)
          const double hand64[4] = {0.0, 1.6, 4.0, 4.9};
          const int64_t t64 = heads * ceil_div(n, 64);
          double best = 1e30;
          for (int i = 0; i < 4; ++i) {
            const int parts = 1 << i;
            if (i > 0 && (ktiles < 2 * parts || t64 * parts > 2 * kNumCU)) break;
            const double us = 4.2 + (0.3 + 0.3 * static_cast<double>(t64 * parts) / 192.0) * static_cast<double>(ceil_div(ktiles, parts)) + hand64[i];
            if (us < best) best = us, cfg.split_k = parts;
          }
          fitted = true;
        }
      }
      else if (t128 <= kNumCU && bn == 128) cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {128, 128, kBK}, 1, 0};
      else if (bn == 128) {
        cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {256, 128, kBK}, 1, 0};
        // Rows of P off the 16-byte grid cost the loads of a workgroup more, and a last round of 256-row tiles that leaves
        // CUs idle then shows: 64-row tiles (two workgroups per CU) instead -- n = m = 1025: 29.9 against 35.0 us (160
        // workgroups of 256 rows), 2049: 84.9 / 94.9, 3001: 159 / 170; with rows on the grid the big tiles stay ahead
        // whatever the fill (1088: 25.0 against 29.0), and so they do off the grid from three quarters of the CUs on
        // (1281: 43.9 / 45.9, 1537: 50.0 / 54.0)
        const int64_t w256 = heads * ceil_div(n, 256), last_round = w256 % kNumCU;
        if (!p_vec && last_round != 0 && last_round * 10 < kNumCU * 7) cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {64, 128, kBK}, 1, 0};
        // Rows on the grid, and the 256-row tiles make one round of the chip and a thin second one: the smaller tiles'
        // rounds end closer together -- 64-row tiles up to 1.3 rounds (40 heads, n = m = 1600: 56.8 us against 63.7;
        // 32 heads, 2560: 97.4 / 109.7; not against more than 4096 keys: 64 heads, 1280 x 8192: 328 / 314), 128-row tiles
        // up to 1.5 (32 heads, 3072: 126 / 135; 64 heads, 1536: 73.9 / 78.2; 64 heads, 1280 x 8192: 291 / 314).  Measured
        // with 16 .. 64 heads of 80 and 128 at n = 1100 .. 4096; from 1.5 rounds on the 256-row tiles are ahead again
        else if (p_vec && w256 > kNumCU && w256 * 10 <= kNumCU * 13 && ktiles <= 64) cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {64, 128, kBK}, 1, 0};
        else if (p_vec && w256 > kNumCU && w256 * 2 <= kNumCU * 3) cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {128, 128, kBK}, 1, 0};
      } else cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 2, {128, bn, kBK}, 1, 0};
      // 128-row tiles (one workgroup per CU) gain only while all parts run at once: 512 rows against 4096 keys
      // take 47 us in two parts, 58 whole, 80 in eight.  Partial tiles of 256 rows cost more to combine than a
      // split saves.
      const int64_t wgs = heads * ceil_div(n, cfg.tile[0]);
      const int64_t wg_limit = cfg.tile[0] <= 64 ? 4 * kNumCU : kNumCU;
      double us;
      if (!fitted && wgs < kNumCU && cfg.tile[0] <= 128) cfg.split_k = key_split(wgs, wg_limit, ktiles, &us);
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
    return launch_gemm_scalar("attn_pv", static_cast<unsigned>(grid), static_cast<unsigned>(b), s, a, w, ep, out, n, d, m, true);
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
  if (m * d >= (int64_t{1} << 31)) return fail("attn_pv: a head's V exceeds the 4 GiB a buffer descriptor spans");
  int64_t la[7];
  if (describe_gemm(n, d, m, cfg, la) != 0) return -1;   // (also: no more LDS stages than the tile allows)
  const int bm = cfg.tile[0], bn = cfg.tile[1];
  const int ns = cfg.unroll >= 2 ? cfg.unroll : 2;
  ep.lda = m;
  ep.k_tail = static_cast<unsigned>(m - m_main);
  // Rows of P a multiple of 4 KiB apart (m = 2048, 4096, ...; a few elements more still count): the same k tile of every
  // row lies in the same few memory channels, and workgroups that walk k in lockstep queue up there.  Each then starts
  // at a k tile of its own.  Measured, lockstep / staggered us, 32 heads of 80: n x m = 1024 x 2048 38.0 / 34.2, 2048 x
  // 2048 73.3 / 57.5, 4096 x 2048 137 / 110, 2048 x 4096 131 / 103, 1024 x 8192 135 / 103, 2048 x 6144 174 / 151, 2048 x
  // 2049 77.6 / 70.3; other row pitches lose 1-7 % (1024 x 1024 18.9 / 19.6, 2048 x 1024 32.8 / 35.4, 2048 x 1984 53.2 / 54.8).
  ep.k_stagger = (m * 2) % 4096 < 32 ? 1u : 0u;
#define DTAS_PV_CASE(BM_, BN_, NS_) \
  if (bm == BM_ && bn == BN_ && ns == NS_) return launch_mfma<BM_, BN_, 2, 2, NS_, true>(s, a, w, ep, out, n, d, m_main, sk, b)
  // (four stages measured level with or behind three on every tile, n = m = 256 .. 4096: not instantiated)
  DTAS_PV_CASE(256, 128, 3);
  DTAS_PV_CASE(128, 128, 2); DTAS_PV_CASE(128, 128, 3);
  DTAS_PV_CASE(64, 128, 2); DTAS_PV_CASE(64, 128, 3);
  DTAS_PV_CASE(128, 64, 2);
  DTAS_PV_CASE(64, 64, 2);
#undef DTAS_PV_CASE
  if (ns != 2) return fail("attn_pv: three LDS stages come with the 256x128, 128x128 and 64x128 tiles, two with every tile but 256x128; got %dx%d with %d", bm, bn, ns);
  return fail("attn_pv: no transposing MFMA kernel for tile %dx%d", bm, bn);
}
// The LDS-tiled MFMA kernel of the GEMM family and its launcher, as templates: each source that includes this
// instantiates the forms it serves (gemm_tiles.hip: row-major fp16 W; attention.hip: the k-major V of P.V;
// gemm_q8.hip: 8-bit W dequantised on its way into the LDS).  Internal to libdtas_gfx950.so.
#pragma once
#include "gemm_common.h"

// Tile rows per group of the tile order (groups of this many tile rows are walked column-wise, and each XCD takes a
// contiguous span of that order: with 32 workgroups resident per XCD a group of 8 makes an XCD's patch 8 x 4 tiles).
#ifndef DTAS_GEMM_TILE_GROUP
#define DTAS_GEMM_TILE_GROUP 8
#endif
// Cache policy bits of the direct-to-LDS operand loads (the builtin's last argument: 1 = sc0, 2 = nt, 16 = sc1).
#ifndef DTAS_GEMM_LOAD_AUX
#define DTAS_GEMM_LOAD_AUX 0
#endif

namespace dtas {
namespace {

// WT: W is given k-major ([K][N], N contiguous -- the V operand of attention's P.V); its tiles sit in the LDS as they lie
// in memory (the same direct-to-LDS loads and pipelines as a row-major W) and the MFMA fragments are read with the
// transposing LDS read ds_read_b64_tr_b16 (4 wavefronts only).
// WQ: W is 8-bit with an fp16 scale per 32 elements of a row (Wq bytes [N][K], ep.wscale [N][K/32]); its
// tiles pass through registers and are dequantised on their way into the LDS.
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
  constexpr bool WREG = WQ;  // W tiles pass through registers (dequantised), not the direct-to-LDS path
  static_assert(!WREG || (NS <= 3 && NW == 4), "the register W path is written for two or three stages and 4 wavefronts");
  static_assert(!(WT && WQ), "k-major 8-bit weights are not served");
  static_assert(!WT || (NW == 4 && BN >= 64), "the k-major W path is written for the 4-wavefront 32x32x16 loops");
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
  constexpr unsigned kGroup = DTAS_GEMM_TILE_GROUP;
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
  // row-major W: the tile's rows; k-major W ([K][N], the V of P.V): the whole matrix, so that k rows past K read as zeros
  const __amdgpu_buffer_rsrc_t rw = WT ? make_rsrc(W, static_cast<unsigned>(K * N * 2))
                                       : make_rsrc(W + n0 * K, static_cast<unsigned>(rows_w) * row_bytes);
  const unsigned r_in = 2u * (l >> 4) + (((l >> 3) & 1u) ^ (wv & 1u));  // row inside the 8-row block
  const unsigned c_in = (l & 7u) ^ r_in;                                // chunk of that row
  const unsigned g_off = (8u * wv + r_in) * row_bytes + c_in * 16u;
  const unsigned g_step = 8u * NW * row_bytes;

  // ---- k-major W (WT).  A W tile is 64 k x BN columns of W[K][N] and sits in the LDS as it lies in memory: k row after
  // k row of BN * 2 bytes, brought in by the same direct-to-LDS block loads (slot p of a 1 KiB block <- lane p; columns past N
  // and k rows past K are out of range and arrive as zeros).  The MFMA wants a lane to hold 8 consecutive k of one column:
  // ds_read_b64_tr_b16 delivers that -- in each group of 16 lanes, lane r names 8 bytes (4 columns of one k row) and lane i
  // receives element i & 3 of the rows that lanes i >> 2, 4 + (i >> 2), 8 + (i >> 2), 12 + (i >> 2) named; with lane r naming
  // k row r >> 2, columns 4 (r & 3) .. + 3, lane i receives 4 consecutive k of column i.  16-byte chunk c of k row k is kept at
  // chunk position c ^ wt_swz(k), which spreads the 32 lanes the LDS serves together (4 k rows x two 16-column groups) over all
  // 64 banks (a k row is a whole number of bank rows, or half of one when BN = 64).
  constexpr int kWtRowB = BN * 2, kWtRpb = 1024 / kWtRowB;  // bytes per k row in the LDS; k rows per 1 KiB block
  static_assert(!WT || (kWtRpb >= 1 && 1024 % kWtRowB == 0 && (NW * kWtRpb) % 4 == 0), "k rows per block");
  auto wt_swz = [](unsigned k) -> unsigned { return BN >= 128 ? 4u * (k & 3u) : 4u * ((k >> 1) & 1u); };
  const unsigned wt_k = wv * kWtRpb + (l * 16u) / kWtRowB;                 // k row (inside a stage) of this lane's slot in block 0
  const unsigned wt_c = (((l * 16u) % kWtRowB) / 16u) ^ wt_swz(wt_k);      // the chunk that belongs at this lane's slot
  const bool wt_col_ok = n0 + 8 * static_cast<int64_t>(wt_c) < N;         // (N % 8 == 0: a chunk is all-in or all-out)
  const unsigned wt_off = static_cast<unsigned>((static_cast<int64_t>(wt_k) * N + n0 + 8 * wt_c) * 2);
  // one block load further: NW * kWtRpb k rows on.  The block's offset is added to the lane's (vector) offset, which the
  // descriptor's range check covers: k rows past K must read as zeros (the k tail is added in the epilogue, and what lies
  // behind a head's V is another head's), and an out-of-range lane (0x80000000 + ...) stays out of range
  const unsigned wt_step = static_cast<unsigned>(NW * kWtRpb * N * 2);
  // fragment reads: lane l = 16 g + r; group g serves columns 16 (g & 1) .. + 15 of a 32-column block and k 8 (g >> 1) .. + 7
  // of a k16 step, in two reads of 4 k each
  unsigned wt_rd[NT];
  {
    const unsigned g = l >> 4, r = l & 15u;
    const unsigned krow = 8u * (g >> 1) + (r >> 2);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const unsigned c = (wn * WTN + j * 32 + 16u * (g & 1u)) / 8u + ((r >> 1) & 1u);
      wt_rd[j] = krow * kWtRowB + ((c ^ wt_swz(krow)) * 16u) + (r & 1u) * 8u;
    }
  }

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
  // k-major W (P.V): a workgroup starts at a k tile of its own and wraps around.  The rows of P lie a power of two apart
  // when the key count is one, so the same k tile of every row maps to the same few memory channels, and workgroups
  // that all start at k tile 0 walk the channels in lockstep (the bare load pattern of 32 x 2048 x 2048 with 256-row
  // tiles: 4.3 TB/s in lockstep, 5.8 staggered, 6.0 with rows 4224 bytes apart).  Which k tile comes when is a function
  // of the tile alone, so a launch still adds in the same order every time.
  const int kt_rot = WT && ep.k_stagger && ktiles > 1 ? static_cast<int>(__builtin_amdgcn_readfirstlane((batch_u * total + pid) % static_cast<unsigned>(ktiles))) : 0;
  auto kt_abs = [&](int kt) -> int {  // k tile of the matrix that is this workgroup's kt-th
    if constexpr (!WT) return kt0 + kt;
    const int v = kt + kt_rot;
    return kt0 + (v >= ktiles ? v - ktiles : v);
  };

  // k-major W: this lane's byte offset in W for k tile kt of this workgroup (k rows past K lie past the descriptor's range)
  auto wt_lane_off = [&](int kt) -> unsigned {
    return wt_col_ok ? wt_off + static_cast<unsigned>(static_cast<int64_t>(kt_abs(kt)) * kBK * N * 2) : kOob;
  };
  // tile kt -> LDS stage kt % NS, asynchronously (completion is counted by vmcnt)
  auto fetch = [&](int kt) {
    // a chunk past K is pointed out of range; K % 8 == 0, so chunks are all-in or all-out
    const unsigned off = (static_cast<int64_t>(kt_abs(kt)) * kBK + c_in * 8 < K)
                             ? g_off + static_cast<unsigned>(kt_abs(kt)) * kRowBytes : kOob;
    char* base = lds + (kt % NS) * kStage + wv * 1024;
    // (the block's row offset rides in the scalar offset operand: no vector add per load)
#pragma unroll
    for (int i = 0; i < LA; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + i * NW * 1024), 16, off, i * g_step, 0, DTAS_GEMM_LOAD_AUX);
    if constexpr (WT) {
      const unsigned woff = wt_lane_off(kt);
#pragma unroll
      for (int i = 0; i < LB; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(base + kABytes + i * NW * 1024), 16, woff + i * wt_step, 0, 0, DTAS_GEMM_LOAD_AUX);
    } else if constexpr (!WREG) {
#pragma unroll
      for (int i = 0; i < LB; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(base + kABytes + i * NW * 1024), 16, off, i * g_step, 0, DTAS_GEMM_LOAD_AUX);
    }
  };

  // ---- 8-bit W through registers: an item is 16 weights of a row (16 bytes -> two 16-byte chunks of fp16) and their
  // scale: a lane loads them into registers (wt_load, issued just before the tile's A blocks) and later (wt_commit, once
  // the tile is next in line) stores the dequantised chunks to where the row-major path would have put them; lane t takes
  // piece t % 4 of row t / 4 (+ 64 rows per further item), so a wavefront reads 64 contiguous bytes of each of 16 rows.
  // The pieces come through buffer loads (out of range -> zeros), so every lane issues the same number of loads per tile
  // whatever its rows: the waits below count them.  Every row of the tile is written every time (rows past N as zeros).
  constexpr int kWtItems = WREG ? 4 * BN / (64 * NW) : 1;
  constexpr int kWtSlots = WREG ? NS - 1 : 1;  // register sets: one per tile in flight
  constexpr int kWtLoads = 2 * kWtItems;  // per lane and tile: a piece and its scale per item
  u32x4 wt_reg[kWtSlots][kWtItems][1];
  unsigned short wq_scale[kWtSlots][kWtItems];
  const __amdgpu_buffer_rsrc_t rv = make_rsrc(W, WQ ? static_cast<unsigned>(K * N) : 0u);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(ep.wscale, WQ ? static_cast<unsigned>((K / 32) * N * 2) : 0u);
  auto wt_load = [&](int kt, auto slot_tag) {
    constexpr int SLOT = decltype(slot_tag)::value;
#pragma unroll
    for (int i = 0; i < kWtItems; ++i) {
      const unsigned item = t + i * 64 * NW, r = item >> 2, c4 = item & 3u;
      const int64_t row = n0 + r, k = static_cast<int64_t>(kt_abs(kt)) * kBK + c4 * 16;
      const bool in = row < N && k < K;  // K % 32 == 0: a piece and its scale group are all-in or all-out
      wt_reg[SLOT][i][0] = __builtin_amdgcn_raw_buffer_load_b128(rv, in ? static_cast<unsigned>(row * K + k) : kOob, 0, 0);
      wq_scale[SLOT][i] = __builtin_amdgcn_raw_buffer_load_b16(rs, in ? static_cast<unsigned>((row * (K >> 5) + (k >> 5)) * 2) : kOob, 0, 0);
    }
  };
  auto wt_commit = [&](int kt, auto slot_tag) {
    constexpr int SLOT = decltype(slot_tag)::value;
    char* base = lds + (kt % NS) * kStage + kABytes;
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
  };

  f16x8 fa[2][MT], fb[2][NT];
  auto read_a = [&](int set, int i, const char* stage, int ks) {
    fa[set][i] = *reinterpret_cast<const f16x8*>(stage + a_base + i * 4096 + lds_rd[ks]);
  };
  // (k-major W) The transposing reads are issued as inline assembly: through the compiler's builtin every one of them
  // is preceded by a wait for all outstanding direct-to-LDS loads (the compiler takes the read to alias them), which
  // serialises the pipeline.  The compiler then knows nothing of these reads' completion either: wait_frag_b() is the
  // wait, placed where the fragments are first used.
  const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_ptr_t)lds));
  auto read_b = [&](int set, int j, const char* stage, int ks) {
    if constexpr (WT) {
      // k 16 ks + 8 (g >> 1) .. + 7 of this lane's column: two transposing reads of 4 k each
      const unsigned at = lds_base + static_cast<unsigned>(stage - lds) + kABytes + ks * 16 * kWtRowB + wt_rd[j];
      f16x4 lo, hi;
      asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(at));
      asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(hi) : "v"(at + 4 * kWtRowB));
      fb[set][j] = f16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    } else {
      fb[set][j] = *reinterpret_cast<const f16x8*>(stage + b_base + j * 4096 + lds_rd[ks]);
    }
  };
  // (k-major W) every LDS read issued so far has returned; the W fragments of `set` pass through an empty statement that
  // follows the wait, so nothing that uses them can be moved ahead of it
  auto wait_frag_b = [&](int set) {
    if constexpr (WT) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int j = 0; j < NT; ++j) asm volatile("" : "+v"(fb[set][j]));
    }
  };
  // The MT*NT MFMAs of register set `set`, with the MT+NT fragment reads of the next step (from
  // `stage`, step `ks`, into the other set) spread evenly between them.  W rows are the first MFMA
  // operand, so a lane ends up with 4 consecutive columns of one C row per accumulator quad.
  auto step = [&](int set, const char* stage, int ks, bool reads) {
    constexpr int kReads = MT + NT, kMfma = MT * NT;
    wait_frag_b(set);
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
      return (static_cast<int64_t>(kt_abs(kt)) * kBK + c16 * 8 < K && kt < ktiles) ? g16 + static_cast<unsigned>(kt_abs(kt)) * kRowBytes : kOob;
    };
    auto fetch16 = [&](int slot, unsigned voff) {
      char* base = lds + slot * kUnit + (wv & 3u) * 1024;
      if (hi) {
#pragma unroll
        for (int q = 0; q < kLoadsW; ++q) __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(base + q * 4096), 16, voff, q * g16_step, 0, DTAS_GEMM_LOAD_AUX);
      } else {
#pragma unroll
        for (int q = 0; q < kLoadsA; ++q) __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + q * 4096), 16, voff, q * g16_step, 0, DTAS_GEMM_LOAD_AUX);
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
      return (static_cast<int64_t>(kt_abs(kt)) * kBK + c_in * 8 < K) ? g_off + static_cast<unsigned>(kt_abs(kt)) * kRowBytes : kOob;
    };
    // block load b of a unit (the descriptor is named here, not passed down through the lambdas)
    auto fetch_one = [&](bool is_w, unsigned voff, int slot, int b) {
      lds_ptr_t dst = (lds_ptr_t)(lds + slot * kUnit + wv * 1024 + b * NW * 1024);
      if (is_w) __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, dst, 16, voff, b * g_step, 0, DTAS_GEMM_LOAD_AUX);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, dst, 16, voff, b * g_step, 0, DTAS_GEMM_LOAD_AUX);
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
      return (static_cast<int64_t>(kt_abs(kt)) * kBK + c_in * 8 < K) ? g_off + static_cast<unsigned>(kt_abs(kt)) * kRowBytes : kOob;
    };
    // block load l (0 .. kL-1: A blocks, then W blocks) of a tile into `stage`
    // (k-major W: the W blocks take the lane's offset in W, `woff`)
    auto fetch_one = [&](int l_, unsigned voff, char* stage, unsigned woff = 0u) {
      if (l_ < LA)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(stage + wv * 1024 + l_ * NW * 1024), 16, voff, l_ * g_step, 0, DTAS_GEMM_LOAD_AUX);
      else if constexpr (WT)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(stage + kABytes + wv * 1024 + (l_ - LA) * NW * 1024), 16,
                                                 woff + (l_ - LA) * wt_step, 0, 0, DTAS_GEMM_LOAD_AUX);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(stage + kABytes + wv * 1024 + (l_ - LA) * NW * 1024), 16, voff,
                                                 (l_ - LA) * g_step, 0, DTAS_GEMM_LOAD_AUX);
    };
    // MFMAs of `set`, the next step's fragment reads, and part `part` of a tile's loads (if `dma`)
    auto step_dma = [&](int set, const char* stage, int ks, bool reads, bool dma, int part, unsigned voff, char* dst, unsigned woff) {
      constexpr int kReads = MT + NT, kMfma = MT * NT;
      wait_frag_b(set);
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
            if (l_ >= lo && l_ < hi && (l_ - lo) * kMfma / (hi - lo) == q) fetch_one(l_, voff, dst, woff);
        }
        DTAS_SCHED_FENCE();
      }
    };
    // every stage is free: tile 0, tiles 1 .. NS-2 whole and part 0 of tile NS-1 are requested together, and only
    // tile 0 is waited for (loads complete in order: whole tiles requested after it may stay outstanding)
    if (ktiles > 0) {
      const unsigned v0 = lane_off(0), w0 = WT ? wt_lane_off(0) : 0u;
#pragma unroll
      for (int l_ = 0; l_ < kL; ++l_) fetch_one(l_, v0, lds, w0);
    }
#pragma unroll
    for (int p = 1; p < NS; ++p) {
      if (p < ktiles) {
        const unsigned vp = lane_off(p), wp = WT ? wt_lane_off(p) : 0u;
#pragma unroll
        for (int l_ = 0; l_ < (p < NS - 1 ? kL : kL / 4); ++l_) fetch_one(l_, vp, lds + p * kStage, wp);
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
      const unsigned w_late = WT ? wt_lane_off(kt + NS - 1) : 0u, w_new = WT ? wt_lane_off(kt + NS) : 0u;
      step_dma(0, cur, 1, true, have_late, 1, v_late, late, w_late);
      step_dma(1, cur, 2, true, have_late, 2, v_late, late, w_late);
      step_dma(0, cur, 3, true, have_late, 3, v_late, late, w_late);
      // tile kt+1 must have landed; later tiles (at most NS-2 of them) may stay in flight.  Loads
      // complete in order, so it is enough to allow that many tiles' worth of loads outstanding.
      if (steady) {
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 2) * kL));
      } else {
        wait_whole_tiles<kL, NS - 2>(ktiles - 2 - kt);  // tiles after kt+1 that have been requested
      }
      __builtin_amdgcn_s_barrier();  // ... and every wavefront has finished reading tile kt
      DTAS_SCHED_FENCE();
      step_dma(1, nxt, 0, steady || kt + 1 < ktiles, have_new, 0, v_new, cur, w_new);
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
    // pair q of a lane's accumulators (in whatever order the main loop keeps them)
    constexpr int kPer = M16 ? MT16 * NT16 * 2 : MT * NT * 8;  // 8-byte units per lane and partial tile
    static_assert(kPer * 64 * NW == kTilePairs, "the wavefronts' partial tiles tile the workgroup's");
    unsigned long long* mine = tile_ws + static_cast<size_t>(z) * kTilePairs + wv * (kPer * 64);
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
            // streamed past the operands in the L2 (1-3 % on wide outputs: 2048 x 10240 x 2560 109.0 -> 106.2 us, 1024 x 5120 x 5120
            // 83.7 -> 82.5; level elsewhere)
            __builtin_nontemporal_store(hv, reinterpret_cast<cvec_a2*>(dst));
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

}  // namespace
}  // namespace dtas

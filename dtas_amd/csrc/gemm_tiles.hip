// Dynamic-M GEMM for gfx950: C[M,N] = A[M,K] . W[N,K]^T (+ bias[N]); fp16 in/out, fp32
// accumulation on the MFMA matrix cores: the entry points, the launch descriptions and the
// instantiations of the tile kernel for a row-major fp16 W.  The fused-epilogue GEMMs and the
// two batched attention matmuls run on the same kernel.
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
// The kernels for few rows of A (SKINNY, STREAM, ROWS) are in gemm_stream.hip, the attention kernels in attention.hip,
// the 8-bit-weight entry point in gemm_q8.hip, the split-K workspace in workspace.hip; the tile kernel itself is the
// template in gemm_tile_kernel.h.
#include "gemm_tile_kernel.h"

namespace dtas {
namespace {

// threads per workgroup of the MFMA kernel for a tile: 8 wavefronts for 256x256, else 4
inline int mfma_threads(int bm, int bn) { return bm == 256 && bn == 256 ? 512 : 256; }
// LDS stages a launch uses unless told otherwise: 2 for 256x256, 3 for 256x128, 4 below that
inline int mfma_max_stages(int bm, int bn) { return bm + bn >= 512 ? 2 : bm + bn >= 384 ? 3 : 4; }

}  // namespace

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
  if (cfg.variant == DTAS_GEMM_MFMA_ACC16) {  // the reference's fp16 accumulator, rounded once per k step of 16
    if (cfg.tile[0] != 64 || cfg.tile[1] != 64 || cfg.tile[2] != 16) return fail("gemm: the fp16-accumulator kernel takes tile 64x64x16, got %dx%dx%d", cfg.tile[0], cfg.tile[1], cfg.tile[2]);
    if (cfg.block != 256) return fail("gemm: the fp16-accumulator kernel uses 256 threads, got %d", cfg.block);
    if (cfg.vec != 8 && cfg.vec != 1) return fail("gemm: vector width must be 8 (128 bit) or 1, got %d", cfg.vec);
    if (cfg.split_k > 1) return fail("gemm: the fp16 accumulator is rounded step by step along K: K cannot be split (split_k = %d)", cfg.split_k);
    const int64_t tm = ceil_div(M, 64), tn = ceil_div(N, 64);
    if (tm * tn > 0x7fffffff) return fail("gemm: too many tiles");
    la[0] = tm * tn;
    la[3] = 256;
    la[5] = tm;
    la[6] = tn;
    return 0;
  }
  if (cfg.vec == 1) {  // element-access fallback
    int64_t grid = ceil_div(M * N, 256);
    la[0] = grid > 65536 ? 65536 : (grid < 1 ? 1 : grid);
    la[3] = 256;
    return 0;
  }
  if (cfg.vec != 8) return fail("gemm: vector width must be 8 (128 bit) or 1, got %d", cfg.vec);
  if (cfg.variant == DTAS_GEMM_MFMA) {
    const int bm = cfg.tile[0], bn = cfg.tile[1];
    // tiles of 192 rows (8 wavefronts only): between the others in size, for tile counts that fill the chip better
    const bool with_192 = bm == 192 && (bn == 256 || bn == 128);  // (192 columns: the epilogue's lane map wants wavefront tiles of 64 columns)
    const bool known = (bm == 256 && bn == 256) || (bm == 256 && bn == 128) || (bm == 128 && bn == 256) ||
                       (bm == 128 && bn == 128) || (bm == 64 && bn == 128) || (bm == 128 && bn == 64) ||
                       (bm == 64 && bn == 64) || with_192;
    if (!known || cfg.tile[2] != kBK) return fail("gemm: no MFMA kernel for tile %dx%dx%d", bm, bn, cfg.tile[2]);
    // 256x256 comes as 8 wavefronts (two per SIMD, 128x64 each) or 4 (one per SIMD, 128x128 each); 256x128 and
    // 128x256 as 4 wavefronts on whole-tile stages or 8 (64x64 each) on the 16x16x32 ring loop (128x128 on that
    // loop, 64x32 per wavefront, measured slower than on 4 wavefronts at every M: not instantiated)
    const bool four_waves = bm == 256 && bn == 256 && cfg.block == 256;
    const bool eight_waves = (bm + bn == 384 || with_192) && cfg.block == 512;
    if (with_192 && !eight_waves) return fail("gemm: the %dx%d MFMA kernel uses 512 threads, got %d", bm, bn, cfg.block);
    if (cfg.block != mfma_threads(bm, bn) && !four_waves && !eight_waves)
      return fail("gemm: the %dx%d MFMA kernel uses %d threads, got %d", bm, bn, mfma_threads(bm, bn), cfg.block);
    if (K * 2 * (bm > bn ? bm : bn) >= (int64_t{1} << 31)) return fail("gemm: K=%lld too large for 32-bit tile offsets", (long long)K);
    const int64_t tm = ceil_div(M, bm), tn = ceil_div(N, bn);
    if (tm * tn > 0x7fffffff) return fail("gemm: too many tiles");
    // cfg.unroll = LDS stages (the depth of the load pipeline); 0 or 1 = as many as fit
    const int max_stages = with_192 ? 2 : mfma_max_stages(bm, bn);
    if (cfg.unroll < 0 || cfg.unroll > max_stages)
      return fail("gemm: the %dx%d tile holds at most %d LDS stages, got %d", bm, bn, max_stages, cfg.unroll);
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

// Every instantiation of the tile kernel for a row-major fp16 W, chosen by cfg (validated by describe_gemm): tile,
// 4 or 8 wavefronts, LDS stages, K split.  `batch` problems in one launch (strides in ep): the attention scores.
int launch_tile_f16(const dtas_config& cfg, hipStream_t s, const half_t* a, const half_t* w, const GemmEpilogue& b, void* c,
                    int64_t M, int64_t N, int64_t K, int batch) {
  const int bm = cfg.tile[0], bn = cfg.tile[1];
  const int ns = cfg.unroll >= 2 ? cfg.unroll : 0;
  const int sk = cfg.split_k < 1 ? 1 : cfg.split_k;
  if (bm == 256 && bn == 256)
  {
    if (cfg.block == 256) return launch_mfma<256, 256, 2, 2, 2>(s, a, w, b, c, M, N, K, sk, batch);
    int split = sk;
    unsigned unsplit = 0;
    if (cfg.split_k == 0 && batch == 1) tail_split_256(M, N, K, &split, &unsplit);  // (split_k >= 1: that split for every tile)
    return launch_mfma<256, 256, 2, 4, 2, false, false, true>(s, a, w, b, c, M, N, K, split, batch, unsplit);
  }
  if (cfg.block == 512) {  // 8 wavefronts on the 16x16x32 ring loop
    if (bm == 256 && bn == 128) return launch_mfma<256, 128, 4, 2, 2, false, false, true>(s, a, w, b, c, M, N, K, sk, batch);
    if (bm == 128 && bn == 256) return launch_mfma<128, 256, 2, 4, 2, false, false, true>(s, a, w, b, c, M, N, K, sk, batch);
    if (bm == 192 && bn == 256) return launch_mfma<192, 256, 2, 4, 2, false, false, true>(s, a, w, b, c, M, N, K, sk, batch);
    if (bm == 192 && bn == 128) return launch_mfma<192, 128, 4, 2, 2, false, false, true>(s, a, w, b, c, M, N, K, sk, batch);
  }
  if (bm == 256 && bn == 128) return ns == 2 ? launch_mfma<256, 128, 2, 2, 2>(s, a, w, b, c, M, N, K, sk, batch)
                                             : launch_mfma<256, 128, 2, 2, 3>(s, a, w, b, c, M, N, K, sk, batch);
  if (bm == 128 && bn == 256) return ns == 2 ? launch_mfma<128, 256, 2, 2, 2>(s, a, w, b, c, M, N, K, sk, batch)
                                             : launch_mfma<128, 256, 2, 2, 3>(s, a, w, b, c, M, N, K, sk, batch);
  if (bm == 128 && bn == 128) return ns == 2   ? launch_mfma<128, 128, 2, 2, 2>(s, a, w, b, c, M, N, K, sk, batch)
                                     : ns == 3 ? launch_mfma<128, 128, 2, 2, 3>(s, a, w, b, c, M, N, K, sk, batch)
                                               : launch_mfma<128, 128, 2, 2, 4>(s, a, w, b, c, M, N, K, sk, batch);
  if (bm == 64 && bn == 128) return ns == 2   ? launch_mfma<64, 128, 2, 2, 2>(s, a, w, b, c, M, N, K, sk, batch)
                                    : ns == 3 ? launch_mfma<64, 128, 2, 2, 3>(s, a, w, b, c, M, N, K, sk, batch)
                                              : launch_mfma<64, 128, 2, 2, 4>(s, a, w, b, c, M, N, K, sk, batch);
  if (bm == 128 && bn == 64) return ns == 2   ? launch_mfma<128, 64, 2, 2, 2>(s, a, w, b, c, M, N, K, sk, batch)
                                    : ns == 3 ? launch_mfma<128, 64, 2, 2, 3>(s, a, w, b, c, M, N, K, sk, batch)
                                              : launch_mfma<128, 64, 2, 2, 4>(s, a, w, b, c, M, N, K, sk, batch);
  if (bm == 64 && bn == 64) return ns == 2    ? launch_mfma<64, 64, 2, 2, 2>(s, a, w, b, c, M, N, K, sk, batch)
                                   : ns == 3  ? launch_mfma<64, 64, 2, 2, 3>(s, a, w, b, c, M, N, K, sk, batch)
                                              : launch_mfma<64, 64, 2, 2, 4>(s, a, w, b, c, M, N, K, sk, batch);
  return fail("gemm: no MFMA kernel for tile %dx%d", bm, bn);
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
  if (!user && M == 2 && vec_ok) cfg = dtas_config{DTAS_GEMM_ROWS, 64, 8, 1, {2, N <= 2560 ? 1 : 2, 8}, 1, 0};
  // three or four rows against a W of few rows: a row of W per wavefront fills the chip where 64-column tiles do not
  // (4 x 2560 x 2560: 5.3 us against 7.6, 2560 x 10240: 14.1 / 18.5; level at 4096 x 4096, behind at 7680 x 2560: 11.5 / 10.1)
  if (!user && (M == 3 || M == 4) && vec_ok && (N <= 2560 || (N <= 4096 && K <= 4096))) cfg = dtas_config{DTAS_GEMM_ROWS, 64, 8, 1, {4, 1, 8}, 1, 0};
  if (cfg.vec == 8 && !vec_ok) cfg.vec = 1;  // K % 8 != 0 or odd pointers: element accesses
  int64_t la[7];
  if (describe_gemm(M, N, K, cfg, la) != 0) return -1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* a = static_cast<const half_t*>(A);
  const half_t* w = static_cast<const half_t*>(W);
  const GemmEpilogue& b = ep;
  void* c = C;
  if (cfg.variant == DTAS_GEMM_MFMA_ACC16) return launch_gemm_acc16(cfg, s, a, w, b, c, M, N, K);
  if (cfg.vec == 1) return launch_gemm_scalar("gemm", static_cast<unsigned>(la[0]), 1, s, a, w, b, c, M, N, K, false);
  if (cfg.variant == DTAS_GEMM_ROWS) return launch_gemm_rows(cfg, la, s, a, w, b, c, M, N, K);
  if (cfg.variant == DTAS_GEMM_SKINNY) return launch_gemm_skinny(cfg, la, s, a, w, b, c, M, N, K);
  if (cfg.variant == DTAS_GEMM_STREAM) return launch_gemm_stream(cfg, s, a, w, b, c, M, N, K);
  return launch_tile_f16(cfg, s, a, w, b, c, M, N, K, 1);
}

// Shape-bucket dispatcher: the MI355X counterpart of the call_table / index_table that DTAS
// splices into its generated host code (python/dtas/engine/tuner.py:156-299 builds the tables,
// python/dtas/codegen/code_gen.py:242-405 emits them; emitted form
// experiment/dtas_tuned/elementwise/add/float16/top1_256/host.cc:105-125).
//
// The dynamic extent n is cut into buckets [1, div], [div+1, 2*div], ... up to kUpperBound
// (python/dtas/common/config.py:64-78); a call picks
//     index = min((n - 1) / kRangeDiv, last)
// and uses the config of that bucket.  (The reference's emitted statement is n / div, which
// sends n = k*div to the bucket above the one whose label contains it; that is harmless there
// because every bucket kernel is predicated on n, but here a bucket's config is sized for its
// upper end, so the built-in tables use the labelled ranges exactly.  Tables produced by the
// Python Engine keep the reference's statement.)  The reference fills each bucket by timing top-k
// candidates on the GPU and keeps one kernel per merged bucket range; here each bucket's
// config is a closed-form function of the bucket's upper end and the static extents, written
// for gfx950 (256 CUs, wave64, 160 KiB LDS), evaluated at call time.  dtas_select_bucket
// reports the merged range [lo, hi] of equal configs around n, named as the reference names
// bucket kernels.
#include "dtas_host.h"

namespace dtas {

namespace {
thread_local char g_error[512] = {0};

constexpr int64_t kRangeDiv = 16;      // bucket width of the built-in tables
constexpr int64_t kUpperBound = 8192;  // dynamic extents above it share the last bucket
constexpr int64_t kLastIndex = (kUpperBound + kRangeDiv - 1) / kRangeDiv - 1;

dtas_config make(int variant, int block, int vec, int unroll, int t0 = 0, int t1 = 0, int t2 = 0, int split_k = 1,
                 int64_t cap = 0) {
  dtas_config c;
  c.variant = variant;
  c.block = block;
  c.vec = vec;
  c.unroll = unroll;
  c.tile[0] = t0;
  c.tile[1] = t1;
  c.tile[2] = t2;
  c.split_k = split_k;
  c.grid_cap = cap;
  return c;
}

bool same(const dtas_config& a, const dtas_config& b) {
  return a.variant == b.variant && a.block == b.block && a.vec == b.vec && a.unroll == b.unroll &&
         a.tile[0] == b.tile[0] && a.tile[1] == b.tile[1] && a.tile[2] == b.tile[2] && a.split_k == b.split_k &&
         a.grid_cap == b.grid_cap;
}

// bytes per element of the wider of an op's input / output types
int wide_bytes(int op) {
  switch (op) {
    case DTAS_OP_ADD_F16: case DTAS_OP_COPY_F16: return 2;
    case DTAS_OP_ADD_I8: case DTAS_OP_COPY_I8: return 1;
    default: return 4;  // fp32 add / copy and both casts
  }
}

// ---- per-family policies: config for a bucket whose upper end is n_hi -----------------
// The constants below were read off sweeps of every variant on an MI355X (GB/s per launch,
// buffers rotating through more than the Infinity Cache).

// Elementwise: accesses of 128 bit on the wider side (a cast then moves 64 bit on the narrow
// side: 128-bit narrow accesses would make the wide ones 256 bit per lane, which measured ~40 %
// slower).  As many accesses in flight per thread (up to 8) as still leaves >= 4 workgroups per CU.
dtas_config elementwise_policy(int op, int64_t n_hi, int64_t H) {
  const int vec = 16 / wide_bytes(op);
  const int64_t nvec = n_hi * (H > 0 ? H : 1) / vec;
  int unroll = 8;
  while (unroll > 1 && nvec / (256 * unroll) < 4 * kNumCU) unroll /= 2;
  // Eight accesses per thread win while all workgroups are resident at once: 8 per CU, 6 for the two-input ops
  // (16 vectors per thread).  Beyond one round the tail of long workgroups shows, and many short ones are ahead
  // ([8192, 4096]: add 37.3 -> 32.6 us, cast to fp32 37.2 -> 33.3, cast to fp16 36.0 -> 33.0 with two per thread).
  const bool two_inputs = op == DTAS_OP_ADD_F16 || op == DTAS_OP_ADD_F32 || op == DTAS_OP_ADD_I8;
  if (unroll == 8 && nvec / (256 * 8) > (two_inputs ? 6 : 8) * kNumCU) unroll = op == DTAS_OP_CAST_F32_F16 ? 2 : 1;
  return make(DTAS_ELT_VECTOR, 256, vec, unroll);
}

// One workgroup per `rows_per_trip` rows, sized for about two 128-bit vectors per thread and row
// (a multiple of 64 threads, so that 640 vectors take 320 threads x 2 and no lane idles).
dtas_config block_row(int vec, int64_t nvec, int rows_per_trip) {
  int64_t block = ((nvec + 1) / 2 + 63) / 64 * 64;
  if (block > 1024) block = 1024;
  const int64_t iters = (nvec + block - 1) / block;
  if (iters > 8) return make(DTAS_RED_STREAM_ROW, 1024, 1, 1);
  while (rows_per_trip > 1 && iters * rows_per_trip > 8) rows_per_trip /= 2;
  return make(DTAS_RED_BLOCK_ROW, static_cast<int>(block), vec, rows_per_trip);
}

// the vectors-per-thread counts the register kernels are instantiated for
int64_t row_iters(int64_t nvec, int64_t block) {
  const int64_t v = (nvec + block - 1) / block;
  for (int64_t i : {1, 2, 3, 4, 5, 6, 8, 10, 12, 16})
    if (i >= v) return i;
  return 17;
}

int64_t round64(int64_t v) { return v < 64 ? 64 : v > 1024 ? 1024 : (v + 63) / 64 * 64; }

// A workgroup of `block` threads per `rpt` rows where the kernels have that form (2 rows up to 8 vectors per
// thread, 4 up to 4, more than 8 vectors per thread in all only up to 512 threads); else block_row's choice.
dtas_config row_cfg(int vec, int64_t nvec, int64_t block, int rpt) {
  const int64_t it = row_iters(nvec, block);
  const bool ok = it <= 16 && (rpt == 1 || (rpt == 2 && it <= 8) || (rpt == 4 && it <= 4)) && (it * rpt <= 8 || block <= 512);
  return ok ? make(DTAS_RED_BLOCK_ROW, static_cast<int>(block), vec, rpt) : block_row(vec, nvec, rpt);
}

// Norms: n rows of static length H, a workgroup per row or per few rows.  Rows of 320 .. 1024 vectors (RMSNorm:
// H = 2560 .. 8192) and 512 .. 2048 (LayerNorm, the same H) follow sweeps of every block size x rows per trip
// at H = 2560, 4096, 5120, 8192 and n = 256 .. 16384, which show three regimes:
//  * up to 4 rows per CU: one row per workgroup and ~2 vectors per thread (latency: the most threads per row);
//  * 4 .. 16-24 rows per CU: the configs that keep every row resident in one round win, and among them those
//    that take several rows per trip (the per-column parameters are fetched once per trip: LayerNorm's two
//    fp32 vectors are otherwise twice the traffic of the row itself) in workgroups of 128 .. 256 threads
//    (LayerNorm H = 5120, n = 1536: 9.6 us against 13.2 with one row of 640 threads, whose 1536 workgroups
//    need two rounds; RMSNorm H = 8192, n = 4096: 22.5 against 26.6);
//  * beyond: RMSNorm one row per trip at ~3 vectors per thread (H = 8192, n = 16384: 85.4 against 94.0 with
//    4 rows per trip), LayerNorm two rows at ~2.
// Mean / worst ratio to the best swept config over that grid: 1.02 / 1.15 (1.08 / 1.37 with the single rule
// "~2 vectors per thread, 4 or 2 rows per trip from 8 rows per CU").  Other row lengths keep that single rule.
dtas_config norm_policy(int op, int64_t n_hi, int64_t H) {
  const bool rms = op == DTAS_OP_RMS_NORM_F16;
  const int vec = rms ? 8 : 4;
  const int64_t nvec = (H + vec - 1) / vec;
  const int64_t pref = round64((nvec + 1) / 2), narrow = round64((nvec + 4) / 5);
  const int64_t n4 = 4 * kNumCU, n8 = 8 * kNumCU, n12 = 12 * kNumCU, n16 = 16 * kNumCU, n24 = 24 * kNumCU;
  if (rms && nvec >= 256 && nvec <= 1024) {
    if (n_hi <= n4) return block_row(vec, nvec, 1);
    if (n_hi < n8 || (n_hi == n8 && nvec < 1024)) return row_cfg(vec, nvec, pref < 256 ? pref : 256, 2);
    if (n_hi <= n24 && nvec < 512) return row_cfg(vec, nvec, pref, n_hi <= n12 ? 2 : 4);
    if (n_hi <= n16) return row_cfg(vec, nvec, nvec >= 512 ? 256 : pref, 4);
    return row_cfg(vec, nvec, round64((nvec + 2) / 3), 1);
  }
  if (!rms && nvec >= 512 && nvec <= 2048) {
    if (n_hi < n4) return block_row(vec, nvec, 1);
    if (n_hi < n8) {
      if (nvec <= 640) return row_cfg(vec, nvec, pref, n_hi <= n4 ? 1 : 2);
      return row_cfg(vec, nvec, nvec <= 1024 ? 320 : 256, 2);
    }
    if (n_hi <= n16) {
      if (nvec <= 640) return row_cfg(vec, nvec, narrow, 2);
      if (nvec <= 1024) return n_hi <= n12 ? row_cfg(vec, nvec, 128, 2) : row_cfg(vec, nvec, 256, 4);
      if (n_hi <= n8) return nvec < 2048 ? row_cfg(vec, nvec, 256, 2) : row_cfg(vec, nvec, 512, 4);
      return row_cfg(vec, nvec, 768, 2);
    }
    return block_row(vec, nvec, 2);
  }
  if (rms) return block_row(vec, nvec, n_hi >= n8 ? 4 : 1);
  // LayerNorm, 8 to 16 rows per CU: narrow workgroups (about five vectors per thread) are all
  // co-resident and measured ~15 % faster than wide ones, which need a second, partial round.
  if (n_hi >= n8 && n_hi <= n16 && (nvec + narrow - 1) / narrow <= 5 && narrow <= 512)
    return row_cfg(vec, nvec, narrow, 2);
  return block_row(vec, nvec, n_hi >= n8 ? 2 : 1);
}

// Softmax: 32*n rows of dynamic length n (the reduction axis is the dynamic one).  One wavefront
// per row (reductions on the DPP path only) up to 8 vectors per lane; short rows launch one
// row per workgroup so that the many small workgroups spread evenly.  Longer rows, or few
// rows, take a workgroup per row: up to 2048 vectors 4 wavefronts while there are at most 32 rows per CU
// (several such workgroups share a CU and overlap one row's reduction with another's loads: 4096 rows of
// 8192 fp32 33.2 us against 38.9 with 1024 threads) and 4 .. 8 wavefronts at ~3 vectors per thread for
// more rows; wider workgroups for longer rows.
dtas_config softmax_policy(int op, int64_t cols_hi, int64_t rows) {
  const int vec = op == DTAS_OP_SOFTMAX_F16 ? 8 : 4;
  const int64_t nvec = (cols_hi + vec - 1) / vec;
  // (exactly 8 vectors per lane: the wavefront form up to 32 rows per CU only -- 4096 rows of 4096 fp16 11.5 us
  // against 13.8 -- beyond, four wavefronts per row are as fast or 2 % faster)
  if ((nvec < 64 * 8 || (nvec == 64 * 8 && rows > 0 && rows <= 32 * kNumCU)) && (rows <= 0 || rows > 2 * kNumCU))
    return make(DTAS_RED_WAVE_ROW, nvec <= 64 ? 64 : 256, vec, 1);
  if (nvec >= 64 * 8 && nvec <= 256 * 8) {
    // (beyond 32 rows per CU ~3 vectors per thread in 256 .. 512 threads: 262144 rows of 8192 fp16 1387 us against 1491)
    int64_t block = 256;
    if (rows <= 0 || rows > 32 * kNumCU) block = round64((nvec + 2) / 3) < 256 ? 256 : round64((nvec + 2) / 3) > 512 ? 512 : round64((nvec + 2) / 3);
    return make(DTAS_RED_BLOCK_ROW, static_cast<int>(block), vec, 1);
  }
  return block_row(vec, nvec, 1);
}

// GEMV: one row of W per workgroup of 4 wavefronts keeps the most independent streams in
// flight; long rows (K >= 8192) do better with 8 wavefronts on two rows, and so do, on 4 wavefronts, rows that
// leave the last pass of the workgroup's 2048 elements partly empty (K = 2560: 4096 / 10240 / 32000 / 50280 rows
// 5.5 / 9.7 / 24.6 / 37.3 us with two rows against 6.1 / 10.5 / 27.3 / 40.9 with one).
dtas_config gemv_policy(int64_t N, int64_t K) {
  if (K >= 8192) return make(DTAS_GEMV_SPLITK, 512, 8, 2, 2);
  // short rows: a row of up to 1024 elements is one pass of 2 wavefronts, of up to 2048 one pass of 4 -- several rows per
  // workgroup then (28672 rows of 1024 / 2048: 10.9 / 18.3 us against 13.0 / 22.8 with 4 wavefronts on two rows / one row)
  if (K <= 512 && N >= 12288) return make(DTAS_GEMV_SPLITK, 64, 8, 2, 4);   // (one wavefront on 4 rows: 50280 x 512 11.3 -> 9.9 us)
  if (K <= 1024) return make(DTAS_GEMV_SPLITK, 128, 8, 2, N >= 12288 ? 4 : 2);
  if (K <= 2048) return make(DTAS_GEMV_SPLITK, 256, 8, 2, 2);
  if (K % 2048 != 0) return make(DTAS_GEMV_SPLITK, 256, 8, 2, 2);
  return make(DTAS_GEMV_SPLITK, 256, 8, 2, 1);
}

// GEMM: a cost model fitted to sweeps of every tile x stage count x K split over M on an MI355X.
// A candidate's time is (rounds of workgroups over the chip) x (time of one k tile) x (k tiles):
//  * time of one k tile with every CU busy: 256x256 1.50 us, 256x128 (8 wavefronts) 1.00 us, 128x128
//    0.665 us with 4 stages (one workgroup per CU) or 1.14 us per round of two per CU with 2 stages;
//  * a partly filled last round is faster than a full one: x (0.55 + 0.45 * fill); 128x128 with 4
//    stages in a single round gains less: x (0.8 + 0.2 * fill);
//  * 64x64: 0.33 us per k tile up to 256 workgroups, x 0.82 * (workgroups on the fullest CU) beyond;
//  * 128x64 (4 stages, one workgroup per CU at most): 0.47 us per k tile whatever the fill;
//  * few tiles: K split over up to 4 workgroups per tile, each partial tile costing the last
//    workgroup ~4 us (128x128), ~2.5 us (128x64), ~1 us (64x64; 2.5 us with more than one per CU)
//    to add up; 256x128 splits while its workgroups fit one round and each keeps 32 k tiles or
//    more (~4.5 us per partial tile: 512 x 5120 x 13824 in 3 parts 86.8 us against 98.2 for 256x256, 640 x 4096 x 8192 in 2 parts 63.8 against 67.3);
//  * a floor: W (2NK bytes) streams at 3.1 .. 4.3 TB/s depending on the tile (few rows against a very wide W);
//  * M <= 32: the W-streaming SKINNY kernel, whose time grows with N*K (about 3.5 TB/s of W).
struct GemmChoice {
  double us;
  int bm, bn, block, stages, split;
};

double gemm_rounds(double wgs, double slots) {
  const double full = static_cast<double>(static_cast<int64_t>(wgs / slots));
  const double rem = wgs - full * slots;
  return full + (rem > 0 ? 0.55 + 0.45 * rem / slots : 0.0);
}

dtas_config gemm_policy(int64_t M_hi, int64_t N, int64_t K) {
  const int64_t n = N > 0 ? N : 1, k = K > 0 ? K : 1;
  const int64_t ktiles = ceil_div(k, 64);
  GemmChoice best = {1e30, 64, 64, 256, 4, 1};
  auto consider = [&](double us, int bm, int bn, int block, int stages, int split) {
    if (us < best.us) best = {us, bm, bn, block, stages, split};
  };
  auto tiles_of = [&](int bm, int bn) { return static_cast<double>(ceil_div(M_hi, bm) * ceil_div(n, bn)); };
  const double kt = static_cast<double>(ktiles);
  // no candidate is faster than it streams W: TB/s measured at M = 64 against a 50280 x 2560 W
  const double w_mb = 2.0 * static_cast<double>(n) * static_cast<double>(k) * 1e-6;
  // (candidates that all sit on the floor are told apart by their own estimates: 256 x 32000 x 4096, 125 tiles of 256x256
  // 89.0 us, 250 of 256x128 74.4)
  auto floored = [&](double us, double tbs) { return (us > w_mb / tbs ? us : w_mb / tbs) + 1e-3 * us; };
  auto relief = [](double fill) { return fill <= 0.5 ? 0.63 : 0.63 + 0.74 * (fill - 0.5); };
  {
    // 256x256 on 8 wavefronts (16x16x32 MFMA): a round of the chip costs ~8 us plus 1.50 us per k tile with every CU
    // busy; with half of the CUs or fewer busy the card clocks higher and a k tile takes 0.63 of that, linearly in
    // between.  split_k = 0: the tiles of a partly filled last round are shared by 2..4 workgroups each
    // (tail_split_256), which costs ~15 / 18 / 21 us to combine the partial tiles.
    const int64_t tiles = static_cast<int64_t>(tiles_of(256, 256));
    const int64_t full = tiles / kNumCU, rem = tiles % kNumCU;
    double us = static_cast<double>(full) * (8.0 + 1.50 * kt);
    if (rem > 0) {
      int split = 1;
      unsigned unsplit = 0;
      tail_split_256(M_hi, n, k, &split, &unsplit);
      if (split >= 2)
        us += 8.0 + 1.50 * static_cast<double>(ceil_div(ktiles, split)) * relief(static_cast<double>(rem * split) / kNumCU) + 12.0 + 3.0 * (split - 1);
      else
        us += 8.0 + 1.50 * kt * relief(static_cast<double>(rem) / kNumCU);
    }
    consider(floored(us, 3.5), 256, 256, 512, 2, 0);
  }
  {
    // 192x256 on 8 wavefronts (96x64 each, the same loop): 1.18 us per k tile with every CU busy -- as many flops per us
    // as 256x256 -- and the same relief in a partly filled round; there for the tile counts it fills the chip better
    // with (M = 4096 against N = 2560: 220 tiles where 256x256 makes 160, 196 against 219 us at K = 10240; 3072 x 4096:
    // 256 tiles against 192; 2048 x 10240: 440 against 320)
    const int64_t tiles = static_cast<int64_t>(tiles_of(192, 256));
    const int64_t full = tiles / kNumCU, rem = tiles % kNumCU;
    double us = static_cast<double>(full) * (8.0 + 1.18 * kt);
    if (rem > 0) us += 8.0 + 1.18 * kt * relief(static_cast<double>(rem) / kNumCU);
    consider(floored(us, 3.5), 192, 256, 512, 2, 1);
  }
  // 256x128 on 8 wavefronts (64x64 each, the 16x16x32 ring loop): 1.00 us per k tile against 1.045 us on 4 wavefronts
  consider(floored(gemm_rounds(tiles_of(256, 128), kNumCU) * 1.0 * kt, 3.5), 256, 128, 512, 2, 1);
  // 192x128 on 8 wavefronts (48x64 each), where its tiles fill three quarters of the chip or more in one round: ~6 us plus
  // 0.66 us per k tile (2048 x 2560 x 2560: 220 tiles, 29.8 us against 32.6 for the 160 tiles of 256x128; 1536 x 4096 x 4096:
  // 48.2 against 49.7).  With fewer tiles the split tiles are ahead of what this model says of them (1024 x 2560 x 4096:
  // 37.0 against 31.3), a second round costs it more than its share (1536 x 11008 x 4096: 164 against 145), and past 64 k
  // tiles each one takes it 0.8 us (1536 x 4096 x 11008: 144 against 138 for 256x256)
  if (tiles_of(192, 128) <= kNumCU && tiles_of(192, 128) * 4 >= 3 * kNumCU && kt <= 64)
    consider(floored(6.0 + gemm_rounds(tiles_of(192, 128), kNumCU) * 0.66 * kt, 3.5), 192, 128, 512, 2, 1);
  consider(floored(gemm_rounds(tiles_of(128, 128), 2 * kNumCU) * 1.14 * kt, 3.1), 128, 128, 256, 2, 1);
  for (int split = 1; split <= 4; ++split) {
    // (K <= 1024: a launch is mostly its start, and a hand-over costs what the shorter loop saves: 512 x 1024 x 1024 7.8 us whole, 8.6 in two parts)
    if (split > 1 && (ktiles / split < 8 || ktiles <= 16)) continue;
    const double steps = static_cast<double>(ceil_div(ktiles, split));
    const double t128 = tiles_of(128, 128) * split, t64 = tiles_of(64, 64) * split;
    if (split == 1 || t128 <= kNumCU)
      consider(floored((t128 <= kNumCU ? 0.8 + 0.2 * t128 / kNumCU : gemm_rounds(t128, kNumCU)) * 0.665 * steps + (split > 1 ? 4.0 * split : 0.0), split > 1 ? 3.5 : 4.1), 128, 128, 256, 4, split);   // (in K parts W streams slower: 128 x 14336 x 4096 in two parts 39.1 us, 3.0 TB/s)
    consider(floored((t64 <= kNumCU ? 1.0 : 0.82 * static_cast<double>(ceil_div(static_cast<int64_t>(t64), kNumCU))) * 0.33 * steps + (split > 1 ? (t64 <= kNumCU ? 1.0 : 2.5) * split : 0.0), 4.3), 64, 64, 256, 4, split);
    const double t256128 = tiles_of(256, 128) * split;
    if (split > 1 && steps >= 32 && t256128 <= kNumCU)
      consider(floored(gemm_rounds(t256128, kNumCU) * 1.0 * steps + 4.5 * split, 3.5), 256, 128, 512, 2, split);
    const double t12864 = tiles_of(128, 64) * split;
    if (t12864 <= kNumCU)
      consider(floored(0.47 * steps + (split > 1 ? 2.5 * split : 0.0), 3.8), 128, 64, 256, 4, split);   // (128 x 8192 x 8192 in two parts: 38.4 us, 3.5 TB/s of W)
  }
  // M <= 16 and at most one workgroup per CU of the W-streaming kernel (64 columns x 1024 of K each): 10.9 against
  // 12.8 us at 4096 x 4096, 7.2 against 10.2 at 2560 x 2560; with more workgroups than CUs a workgroup's loads,
  // MFMAs and the hand-over of its partial sums are no longer hidden behind another's, and the tiles win again
  if (M_hi <= 16 && ceil_div(n, 64) * ceil_div(k, 1024) <= kNumCU) return make(DTAS_GEMM_STREAM, 256, 8, 1, 16, 64, 1024);
  // 17 .. 32 rows: the same with 32 rows of A and 512 of K per workgroup, where that gives a quarter of a round or more
  // and at most one (8.4 against 9.8 us at 2560 x 2560, 9.5 / 10.7 at 2048 x 4096, 11.4 / 13.9 at 1024 x 8192, 8.9 / 10.2 at
  // 3072 x 2560; behind at 1024 x 1024, whose 32 workgroups leave the chip idle)
  // (from K = 2048 on: at 4096 x 1024 the 64x64 tiles take 7.4 us, this form 8.2)
  if (M_hi > 16 && M_hi <= 32 && k >= 2048 && ceil_div(n, 64) * ceil_div(k, 512) <= kNumCU && ceil_div(n, 64) * ceil_div(k, 512) >= kNumCU / 4)
    return make(DTAS_GEMM_STREAM, 256, 8, 1, 32, 64, 512);
  // M <= 16 against more rows of W: the looping form (the whole of K per workgroup, nothing handed over) while its
  // workgroups run in one round -- 16 columns each (one wavefront, two workgroups per CU) for 4096 < N <= 8192, 64
  // columns (one per CU) for 8192 <= N <= 16384 -- and K is short enough for a round to be worth its start:
  // 15.9 against 20.2 us at 8192 x 4096, 10.6 / 13.5 at 7680 x 2560, 20.4 / 24.5 at 11008 x 4096, 13.0 / 16.4 at
  // 10240 x 2560; level at K = 8192 and from two rounds on (32000 x 4096), behind at N <= 4096
  if (M_hi <= 16 && k <= 4096) {
    if (ceil_div(n, 16) > kNumCU && ceil_div(n, 16) <= 2 * kNumCU) return make(DTAS_GEMM_STREAM, 64, 8, 1, 16, 16, 256);
    if (ceil_div(n, 64) >= kNumCU / 2 && ceil_div(n, 64) <= kNumCU) return make(DTAS_GEMM_STREAM, 256, 8, 1, 16, 64, 256);
  }
  if (M_hi <= 32) {
    // (one workgroup per 16 rows of W: fewer than one per CU leave CUs idle)
    const double skinny_wgs = static_cast<double>(ceil_div(n, 16));
    const double skinny_us = static_cast<double>(n) * static_cast<double>(k) * 2.0 / 3.5e6 * (M_hi <= 8 ? 0.9 : M_hi <= 16 ? 0.95 : 1.35) *
                             (skinny_wgs < kNumCU ? kNumCU / skinny_wgs : 1.0);
    if (skinny_us <= best.us) return make(DTAS_GEMM_SKINNY, 512, 8, 4, static_cast<int>((M_hi + 15) / 16 * 16), 16, 32);
  }
  return make(DTAS_GEMM_MFMA, best.block, 8, best.stages, best.bm, best.bn, 64, best.split);
}

dtas_config policy(int op, int64_t n_hi, int64_t d0, int64_t d1) {
  switch (op) {
    case DTAS_OP_LAYER_NORM_F32_F16:
    case DTAS_OP_RMS_NORM_F16: return norm_policy(op, n_hi, d0);
    case DTAS_OP_SOFTMAX_F32_F16:
    case DTAS_OP_SOFTMAX_F16: return softmax_policy(op, n_hi, d0);
    case DTAS_OP_GEMV_F16: return gemv_policy(d0, d1);
    case DTAS_OP_GEMM_F16: return gemm_policy(n_hi, d0, d1);
    default: return elementwise_policy(op, n_hi, d0);
  }
}

int64_t bucket_index(int64_t n) {
  const int64_t i = n <= 0 ? 0 : (n - 1) / kRangeDiv;
  return i > kLastIndex ? kLastIndex : i;
}
// upper end of the reference-style range [index*div + 1, (index + 1)*div]
int64_t bucket_hi(int64_t index) { return (index + 1) * kRangeDiv; }

const char* op_func_name(int op) {
  switch (op) {
    case DTAS_OP_ADD_F16: case DTAS_OP_ADD_F32: case DTAS_OP_ADD_I8: return "add";
    case DTAS_OP_COPY_F16: case DTAS_OP_COPY_F32: case DTAS_OP_COPY_I8: return "copy";
    case DTAS_OP_CAST_F16_F32: case DTAS_OP_CAST_F32_F16: return "cast";
    case DTAS_OP_LAYER_NORM_F32_F16: return "fused_layer_norm_cast1";
    case DTAS_OP_RMS_NORM_F16: return "rms_norm";
    case DTAS_OP_SOFTMAX_F32_F16: case DTAS_OP_SOFTMAX_F16: return "fused_softmax_cast";
    case DTAS_OP_GEMV_F16: return "fused_NT_matmul10_add5";
    case DTAS_OP_GEMM_F16: return "fused_NT_matmul4_add1";
  }
  return "unknown";
}

int describe(int op, int64_t n, int64_t d0, int64_t d1, const dtas_config& cfg, int64_t la[7]) {
  switch (op) {
    case DTAS_OP_LAYER_NORM_F32_F16:
    case DTAS_OP_RMS_NORM_F16: return describe_reduction(op, n, d0, cfg, la);
    case DTAS_OP_SOFTMAX_F32_F16:
    case DTAS_OP_SOFTMAX_F16: return describe_reduction(op, d0, d1, cfg, la);
    case DTAS_OP_GEMV_F16: return describe_gemv(d0, d1, cfg, la);
    case DTAS_OP_GEMM_F16: return describe_gemm(n, d0, d1, cfg, la);
    default: return describe_eltwise(op, n * d0, cfg, la);
  }
}
}  // namespace

char* error_buffer() { return g_error; }
void clear_error() { g_error[0] = 0; }
int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return -1;
}

void bucket_kernel_name(char* dst, size_t cap, const char* func, const char* var, int64_t lo, int64_t hi) {
  snprintf(dst, cap, "%s_%s_%lld_to_%lld__kernel", func, var, (long long)lo, (long long)hi);
}

Bucketed builtin_config(int op, int64_t n, int64_t d0, int64_t d1) {
  Bucketed b;
  b.index = static_cast<int32_t>(bucket_index(n < 0 ? 0 : n));
  b.row = b.index;
  b.lo = b.index * kRangeDiv + 1;
  b.hi = bucket_hi(b.index);
  // the last bucket also takes every n above the upper bound: size it for the n at hand
  const int64_t n_hi = (b.index == kLastIndex && n > b.hi) ? n : b.hi;
  b.cfg = policy(op, n_hi, d0, d1);
  return b;
}

}  // namespace dtas

extern "C" {

int dtas_abi_version(void) { return DTAS_ABI_VERSION; }

const char* dtas_last_error(void) { return dtas::error_buffer(); }

int dtas_init(void) {
  using namespace dtas;
  clear_error();
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail("dtas_init: no HIP device: %s", hipGetErrorString(e));
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return fail("dtas_init: hipGetDeviceProperties: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail("dtas_init: device %d is %s; this library holds gfx950 code only", dev, prop.gcnArchName);
  // loads the code object on this device and looks up the static scratch array of dtas_gemm_f16_static
  return resolve_static_scratch(nullptr);
}

int dtas_select_bucket(int op, int64_t n, int64_t d0, int64_t d1, dtas_launch_info* out) {
  using namespace dtas;
  clear_error();
  if (!out) return fail("dtas_select_bucket: out is NULL");
  if (op < 0 || op >= DTAS_OP_COUNT) return fail("dtas_select_bucket: unknown op %d", op);
  if (n < 0) return fail("dtas_select_bucket: negative dynamic extent %lld", (long long)n);
  memset(out, 0, sizeof(*out));
  const bool softmax = op == DTAS_OP_SOFTMAX_F16 || op == DTAS_OP_SOFTMAX_F32_F16;
  // softmax: the dynamic extent is the row length; callers pass (n, rows, cols)
  const Bucketed b = builtin_config(op, n, d0, d1);
  // merge neighbouring buckets that resolve to the same config (tuner.py:211-299)
  int64_t lo_idx = b.index, hi_idx = b.index;
  while (lo_idx > 0 && same(policy(op, bucket_hi(lo_idx - 1), d0, d1), b.cfg)) --lo_idx;
  while (hi_idx < kLastIndex && same(policy(op, bucket_hi(hi_idx + 1), d0, d1), b.cfg)) ++hi_idx;
  // table_row = number of config changes below this bucket = row of the merged call table
  int32_t row = 0;
  for (int64_t i = 1; i <= lo_idx; ++i)
    if (!same(policy(op, bucket_hi(i), d0, d1), policy(op, bucket_hi(i - 1), d0, d1))) ++row;
  out->index = b.index;
  out->table_row = row;
  out->bucket_lo = lo_idx * kRangeDiv + 1;
  out->bucket_hi = bucket_hi(hi_idx);
  out->config = b.cfg;
  const char* var = (op == DTAS_OP_GEMM_F16) ? "n" : (softmax ? "m" : "n");
  bucket_kernel_name(out->name, sizeof(out->name), op_func_name(op), var, out->bucket_lo, out->bucket_hi);
  const int64_t nn = n > 0 ? n : 1;
  return describe(op, nn, d0, softmax ? nn : d1, b.cfg, out->launch_args);
}

int dtas_describe_launch(int op, int64_t n, int64_t d0, int64_t d1, const dtas_config* cfg, dtas_launch_info* out) {
  using namespace dtas;
  clear_error();
  if (!out || !cfg) return fail("dtas_describe_launch: NULL argument");
  if (op < 0 || op >= DTAS_OP_COUNT) return fail("dtas_describe_launch: unknown op %d", op);
  memset(out, 0, sizeof(*out));
  out->config = *cfg;
  out->index = -1;
  out->table_row = -1;
  snprintf(out->name, sizeof(out->name), "%s_kernel", op_func_name(op));
  return describe(op, n, d0, d1, *cfg, out->launch_args);
}
}

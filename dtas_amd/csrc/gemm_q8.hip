// The dynamic-n GEMMs on 8-bit weights (q8f16_1: four bytes to a word, an fp16 scale per 32 elements of a row):
// fused_fused_decode2_fused_NT_matmul6_add4 and its fused-epilogue relatives
// (experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py:371-502), C = epilogue(A . dequant(Wq)^T).
// Few rows: the W-streaming kernel on the bytes (gemm_stream.hip).  Otherwise the tile kernel with the dequantiser in
// its W path (template flag WQ, instantiated here), or the dequantiser into a library-owned fp16 buffer followed by
// the fp16 GEMM.
#include "gemm_tile_kernel.h"

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
      return launch_gemm_stream_q8(bm, bk, s, a, w, ep, C, M, N, K);
    }
    if (!user && stream_ok && M <= 32) {
      // measured at the model's shapes (M = 16: 10.1 against 25.6 us at 7680x2560, 14.9 against 92 at 2560x10240;
      // M = 32: 14.0 against 26.3 and 20.5 against 33.8).  512-element slices (three workgroups per CU) unless K is
      // long: from 16 slices on the hand-over of the partial sums costs more than the second workgroup hides
      if (M > 16) return launch_gemm_stream_q8(32, 512, s, a, w, ep, C, M, N, K);
      return launch_gemm_stream_q8(16, K >= 8192 ? 1024 : 512, s, a, w, ep, C, M, N, K);
    }
    // up to 64 rows only while its workgroups (64 columns x 512 of K each) run in one round: 48 rows against 2560 x 2560 /
    // 2048 x 4096 / 4096 x 2048 11.3 / 12.1 / 10.6 us where the tiles take 11.8 / 12.8 / 11.5, but 16.4 / 16.5 / 21.2 against
    // 13.0 / 12.5 / 15.5 at 3072 x 3072 / 4096 x 2560 / 4096 x 4096
    if (!user && stream_ok && M <= 64 && ceil_div(N, 64) * ceil_div(K, 512) <= kNumCU) return launch_gemm_stream_q8(64, 512, s, a, w, ep, C, M, N, K);
  }
  // Two routes.  (1) Dequantising in the W path of the tile kernel: no intermediate, W read once per row of tiles as
  // bytes; a plain burst pipeline on 4 wavefronts, with K split over workgroups while the tiles leave CUs idle.
  // (2) The dequantiser into a library-owned fp16 buffer, then the fp16 GEMM with everything its table offers: 3 more
  // bytes per weight through memory (9-14 us at the model's shapes), worth it once the GEMM itself is long.
  // Measured at the model's shapes with rotating weights, us, route 1 (tile, K parts) / route 2 / the fp16 GEMM on
  // fp16 weights: 7680x2560, M = 64 / 128 / 256 / 512 / 1024: 16.4 (64x64, 4) / 28.0 / 14.3, 21.9 (64x64, 3) / 29.6 /
  // 17.7, 26.8 (128x128, 2) / 33.6 / 25.3, 38.6 (128x128, 1) / 41.4 / 33.4, 58.8 / 52.6 / 43.3; 10240x2560, M = 64 / 128 /
  // 256 / 512: 19.5 / 29.9 / 18.7, 24.2 (128x128, 3) / 34.7 / 26.0, 35.1 / 40.5 / 33.3, 56.4 / 48.8 / 39.6; 2560x10240,
  // M = 64 / 256 / 512 / 1024: 25.7 (64x64, 8) / 34.0 / 22.6, 37.4 (128x128, 6) / 44.1 / 38.5, 52.9 / 57.3 / 50.0, 87.9 /
  // 76.0 / 66.8.  So route 1 up to 512 rows while 128x128 tiles fit the chip in one round; 64x64 tiles (two stages, ~2
  // workgroups per CU wanted) up to 128 rows unless they already number more than the CUs, 128x128 (three stages, one
  // per CU) beyond; K parts to fill the chip, each at least 4 k tiles.  A cfg selects route 1 with its own tile and split.
  const int64_t t128 = ceil_div(M, 128) * ceil_div(N, 128), t64 = ceil_div(M, 64) * ceil_div(N, 64), ktiles = ceil_div(K, kBK);
  const bool fused_route = M <= 512 && t128 <= kNumCU;
  if (!user && !fused_route) {
    void* wbuf = nullptr;
    std::lock_guard<std::recursive_mutex> ws_lock(g_ws_mutex);  // until both launches are enqueued
    if (operand_workspace(static_cast<hipStream_t>(stream), static_cast<size_t>(N) * K * 2, &wbuf) != 0) return -1;
    if (dtas_decode_q8_f16(Wq, scale, wbuf, N, K, nullptr, stream) != 0) return -1;
    return dtas_gemm_f16_fused(A, wbuf, bias, res1, res2, C, M, N, K, epilogue, nullptr, stream);
  }
  dtas_config cfg;
  if (user) {
    cfg = *user;
  } else {
    // three tiles of three stages -- 64x64 (three workgroups per CU), 128x64 (two), 128x128 (one) -- with K in 1 .. 8 parts of
    // 4 k tiles or more: us = start + (k tiles per part) x (cost of one, growing with the workgroups on the chip) + a
    // hand-over per part, fitted to a sweep of the model's shapes at M = 96 .. 512 with the weights streamed from memory
    // (2560 x 2560, M = 256: 64x64 in 3 parts 15.4 us, 22 before; 10240 x 2560, M = 192: 64x64 28.3, 34 before; within 10 % of
    // the best of 36 configurations on the sweep's 24 shapes, 3 % on average)
    const int64_t t12864 = ceil_div(M, 128) * ceil_div(N, 64);
    // (rows 5, 6, 10, ... KiB of fp16 apart: a loaded chip takes a k tile of the 128x64 tile 20-25 % longer -- 2560 x 10240,
    // M = 512 in 3 parts: 58.6 us where the fit without it says 47.6, 128x128 53.6)
    const bool odd_pitch = K % 1024 == 0 && ((K / 1024) & (K / 1024 - 1)) != 0;
    double best = 1e30;
    cfg = dtas_config{DTAS_GEMM_MFMA, 256, 8, 3, {128, 128, kBK}, 1, 0};
    for (int parts = 1; parts <= 8; ++parts) {
      if (parts > 1 && ktiles / parts < 4) break;
      const double steps = static_cast<double>(ceil_div(ktiles, parts));
      const double w64 = static_cast<double>(t64 * parts), w12864 = static_cast<double>(t12864 * parts), w128 = static_cast<double>(t128 * parts);
      const double us64 = w64 <= 512 ? 4.4 + (0.30 + 0.26 * w64 / 480.0) * steps + 1.33 * (parts - 1) : 1e30;
      const double b12864 = 0.18 + 0.69 * (odd_pitch ? 1.35 : 1.0) * w12864 / 480.0;
      const double us12864 = w12864 <= 512 ? 8.4 + (b12864 < 0.44 ? 0.44 : b12864) * steps + 1.5 * (parts - 1) : 1e30;
      const double us128 = w128 <= kNumCU ? 9.2 + (0.373 + 0.45 * w128 / 480.0) * steps + 1.87 * (parts - 1) : 1e30;
      if (us64 < best) best = us64, cfg.tile[0] = 64, cfg.tile[1] = 64, cfg.split_k = parts;
      if (us12864 < best) best = us12864, cfg.tile[0] = 128, cfg.tile[1] = 64, cfg.split_k = parts;
      if (us128 < best) best = us128, cfg.tile[0] = 128, cfg.tile[1] = 128, cfg.split_k = parts;
    }
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* a = static_cast<const half_t*>(A);
  const half_t* w = static_cast<const half_t*>(Wq);  // (bytes; the kernels take the pointer as they take fp16 W)
  const bool vec_ok = aligned(A, 16) && aligned(Wq, 16) && aligned(scale, 2) && N * K < (int64_t{1} << 32) && K > 0;
  if (cfg.vec == 8 && !vec_ok) cfg.vec = 1;
  if (cfg.vec == 1) {
    int64_t grid = ceil_div(M * N, 256);
    grid = grid > 65536 ? 65536 : grid;
    return launch_gemm_scalar("gemm_q8", static_cast<unsigned>(grid), 1, s, a, w, ep, C, M, N, K, false);
  }
  if (cfg.vec != 8) return fail("gemm_q8: vector width must be 8 (128 bit) or 1, got %d", cfg.vec);
  if (cfg.variant != DTAS_GEMM_MFMA) return fail("gemm_q8: only the MFMA kernels serve 8-bit weights");
  const int sk = cfg.split_k < 1 ? 1 : cfg.split_k;
  int64_t la[7];
  if (describe_gemm(M, N, K, cfg, la) != 0) return -1;
  const int bm = cfg.tile[0], bn = cfg.tile[1];
  if (bm == 256 && bn == 128 && cfg.unroll == 3) return launch_mfma<256, 128, 2, 2, 3, false, true>(s, a, w, ep, C, M, N, K, sk);
  if (bm == 128 && bn == 128 && cfg.unroll == 3) return launch_mfma<128, 128, 2, 2, 3, false, true>(s, a, w, ep, C, M, N, K, sk);
  if (bm == 64 && bn == 64 && cfg.unroll == 2) return launch_mfma<64, 64, 2, 2, 2, false, true>(s, a, w, ep, C, M, N, K, sk);
  if (bm == 128 && bn == 64 && cfg.unroll == 3) return launch_mfma<128, 64, 2, 2, 3, false, true>(s, a, w, ep, C, M, N, K, sk);
  if (bm == 64 && bn == 64 && cfg.unroll == 3) return launch_mfma<64, 64, 2, 2, 3, false, true>(s, a, w, ep, C, M, N, K, sk);
  if (bm == 64 && bn == 128 && cfg.unroll == 3) return launch_mfma<64, 128, 2, 2, 3, false, true>(s, a, w, ep, C, M, N, K, sk);
  return fail("gemm_q8: 8-bit weights come with tiles 256x128, 128x128, 128x64, 64x128 (three stages) and 64x64 (two or three), got %dx%d with %d", bm, bn, cfg.unroll);
}
// Dynamic-M GEMM for gfx950: C[M,N] = A[M,K] . W[N,K]^T (+ bias[N]); fp16 in/out, fp32
// accumulation on the MFMA matrix cores.
//
// Replaces the kernels DTAS's WMMA rule generates (python/dtas/schedule/tir_wmma.py:20-222:
// pad M to a tile multiple, block tile (i*micro_x*16) x (j*micro_y*16), k tile micro_k*16,
// A/B staged in shared.dyn by cooperative_fetch (python/dtas/schedule/tir_base.py:37-97),
// two-stage software pipeline, accumulators through shared memory to a guarded vector
// store; example output experiment/testIR/GEMM/m_n2560_k10240/wmma/16x16x16/i2j4_x7y2_in8.py).
//
// MI355X shape
//   MFMA   : 256 threads = 4 wavefronts in a 2x2 grid; a wavefront owns (BM/2)x(BN/2) of the
//            BMxBN tile as 32x32 blocks of v_mfma_f32_32x32x16_f16, accumulators in registers
//            (256 per lane for the 256x256 tile).  K advances 64 at a time; both operands are
//            K-contiguous, so a tile row is one 128-byte line = 8 chunks of 16 bytes.
//            Global -> registers with 128-bit buffer loads (rows past M / N read as zero by the
//            buffer's range check), registers -> LDS, LDS -> MFMA operands with 128-bit reads.
//            LDS is double buffered (2 x (BM+BN) x 128 B, 128 KiB of the 160 KiB for 256x256):
//            the loads of tile k+1 are in flight while tile k is multiplied, one barrier per
//            k tile.  The LDS placement of chunk c of row r is swizzled so that both the
//            row-major writes and the column-of-rows MFMA reads spread over all banks.
//            Workgroup ids are remapped so that each XCD (own L2) works on a compact patch of
//            the tile grid.
//   SKINNY : M <= 64 (kernels exist up to 80 rows).  The work is streaming W once; a workgroup owns 16 columns of C and all
//            of M, its wavefronts split K, v_mfma_f32_16x16x32_f16 operands are loaded
//            straight from global memory, partial tiles are folded through LDS.
#include "dtas_device.h"
#include "dtas_host.h"

namespace dtas {
namespace {

typedef float f32x4v __attribute__((ext_vector_type(4)));

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

__device__ __forceinline__ half_t finish(float acc, const half_t* bias, int64_t j) {
  half_t r = static_cast<half_t>(acc);
  if (bias) r = static_cast<half_t>(static_cast<float>(r) + static_cast<float>(bias[j]));
  return r;
}

// Position of workgroup `wg` in a tile order in which each XCD gets a contiguous span:
// the hardware deals consecutive workgroup ids round-robin over the 8 XCDs.
__device__ __forceinline__ unsigned xcd_contiguous_id(unsigned wg, unsigned total) {
  const unsigned xcd = wg % kNumXCD, local = wg / kNumXCD;
  const unsigned base = total / kNumXCD, rem = total % kNumXCD;
  return xcd * base + (xcd < rem ? xcd : rem) + local;
}

template <int BM, int BN>
__global__ void __launch_bounds__(256) gemm_mfma_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W,
                                                        const half_t* __restrict__ bias, half_t* __restrict__ C,
                                                        int64_t M, int64_t N, int64_t K, unsigned tiles_m,
                                                        unsigned tiles_n) {
  constexpr int WTM = BM / 2, WTN = BN / 2;  // wavefront tile
  constexpr int MT = WTM / 32, NT = WTN / 32;
  constexpr int LA = BM / 32, LB = BN / 32;  // 128-bit loads per thread per k tile
  constexpr int kABytes = BM * kRowBytes, kStage = (BM + BN) * kRowBytes;
  __shared__ __attribute__((aligned(1024))) char lds[2 * kStage];

  const unsigned t = threadIdx.x, l = t & 63u, wv = t >> 6, wm = wv >> 1, wn = wv & 1u;

  // ---- which tile: XCD-contiguous order, then groups of 8 tile rows walked column-wise
  const unsigned total = tiles_m * tiles_n;
  const unsigned pid = xcd_contiguous_id(blockIdx.x, total);
  constexpr unsigned kGroup = 8;
  const unsigned width = kGroup * tiles_n;
  const unsigned first_m = (pid / width) * kGroup;
  const unsigned gsize = tiles_m - first_m < kGroup ? tiles_m - first_m : kGroup;
  const unsigned tm = first_m + (pid % width) % gsize, tn = (pid % width) / gsize;
  const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;

  // ---- global side: chunk ld_c of rows ld_r + 32*i; rows past the operand's end are out of
  // the buffer's range and read as zero
  const int64_t rows_a = M - m0 < BM ? M - m0 : BM, rows_w = N - n0 < BN ? N - n0 : BN;
  const unsigned row_bytes = static_cast<unsigned>(K) * 2u;
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(A + m0 * K, static_cast<unsigned>(rows_a) * row_bytes);
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(W + n0 * K, static_cast<unsigned>(rows_w) * row_bytes);
  const unsigned ld_r = t >> 3, ld_c = t & 7u;
  const unsigned g_off = ld_r * row_bytes + ld_c * 16u;
  const unsigned g_step = 32u * row_bytes;
  const unsigned lds_wr = lds_chunk_offset(ld_r, ld_c);  // + i * 4096 for row ld_r + 32*i

  // ---- LDS -> MFMA operands: lane l supplies row (l & 31), chunk 2*ks + (l >> 5)
  unsigned lds_rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) lds_rd[ks] = lds_chunk_offset(l & 31u, 2u * ks + (l >> 5));
  const unsigned a_base = wm * (WTM / 2) * 256u, b_base = kABytes + wn * (WTN / 2) * 256u;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int ktiles = static_cast<int>((K + kBK - 1) / kBK);
  u32x4 sa[LA], sb[LB];

  auto fetch = [&](int kt) {
    const unsigned kb = static_cast<unsigned>(kt) * kRowBytes;
    // a chunk past K is pointed out of range; K % 8 == 0, so chunks are all-in or all-out
    const unsigned off = (static_cast<int64_t>(kt) * kBK + ld_c * 8 < K) ? g_off + kb : kOob;
#pragma unroll
    for (int i = 0; i < LA; ++i) sa[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, off + i * g_step, 0, 0);
#pragma unroll
    for (int i = 0; i < LB; ++i) sb[i] = __builtin_amdgcn_raw_buffer_load_b128(rw, off + i * g_step, 0, 0);
  };
  auto stash = [&](int buf) {
    char* base = lds + buf * kStage + lds_wr;
#pragma unroll
    for (int i = 0; i < LA; ++i) *reinterpret_cast<u32x4*>(base + i * 4096) = sa[i];
#pragma unroll
    for (int i = 0; i < LB; ++i) *reinterpret_cast<u32x4*>(base + kABytes + i * 4096) = sb[i];
  };

  if (ktiles > 0) {
    fetch(0);
    stash(0);
  }
  __syncthreads();

  for (int kt = 0; kt < ktiles; ++kt) {
    const bool more = kt + 1 < ktiles;
    if (more) fetch(kt + 1);
    const char* buf = lds + (kt & 1) * kStage;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      f16x8 fa[MT], fb[NT];
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[i] = *reinterpret_cast<const f16x8*>(buf + a_base + i * 4096 + lds_rd[ks]);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb[j] = *reinterpret_cast<const f16x8*>(buf + b_base + j * 4096 + lds_rd[ks]);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (more) stash((kt + 1) & 1);
    __syncthreads();
  }

  // ---- accumulators -> C: register v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32
  // of its 32x32 block
  const int64_t col_l = l & 31u, row_l = 4 * (l >> 5);
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int64_t col = n0 + wn * WTN + j * 32 + col_l;
      if (col < N) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int64_t row = m0 + wm * WTM + i * 32 + 8 * (v / 4) + row_l + (v % 4);
          if (row < M) C[row * N + col] = finish(acc[i][j][v], bias, col);
        }
      }
    }
  }
}

// M <= 16 * MT.  Workgroup = 16 columns of C; wavefront w takes k steps w, w + nwaves, ...
// of 32 elements.  Lane l supplies row (l & 15), elements 8*(l >> 4) .. +8 of the step, for both
// operands, loaded straight from global memory.  Result register v of lane l is row
// 4*(l >> 4) + v, column l & 15 of the 16x16 block.
template <int MT>
__global__ void __launch_bounds__(512) gemm_skinny_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W,
                                                          const half_t* __restrict__ bias, half_t* __restrict__ C,
                                                          int64_t M, int64_t N, int64_t K) {
  __shared__ f32x4v part[8][MT][64];
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
#pragma unroll 4
  for (int64_t s = wv; s < steps; s += nwaves) {
    const f16x8 fw = __builtin_bit_cast(f16x8, load_stream(reinterpret_cast<const u32x4*>(wp + s * 32)));
    f16x8 fa[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) fa[i] = *reinterpret_cast<const f16x8*>(ap[i] + s * 32);
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[i], fw, acc[i], 0, 0, 0);
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
        if (row < M) C[row * N + col] = finish(s[v], bias, col);
      }
    }
  }
}

// Any K and alignment: one thread per element of C.
__global__ void __launch_bounds__(256) gemm_scalar_kernel(const half_t* __restrict__ A, const half_t* __restrict__ W,
                                                          const half_t* __restrict__ bias, half_t* __restrict__ C,
                                                          int64_t M, int64_t N, int64_t K) {
  const int64_t total = M * N;
  for (int64_t ij = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; ij < total;
       ij += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const half_t* a = A + (ij / N) * K;
    const half_t* w = W + (ij % N) * K;
    float acc = 0.f;
    for (int64_t k = 0; k < K; ++k) acc += static_cast<float>(a[k]) * static_cast<float>(w[k]);
    C[ij] = finish(acc, bias, ij % N);
  }
}

template <int BM, int BN>
int launch_mfma(const int64_t la[7], hipStream_t s, const half_t* A, const half_t* W, const half_t* bias, half_t* C,
                int64_t M, int64_t N, int64_t K) {
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(M, BM)), tiles_n = static_cast<unsigned>(ceil_div(N, BN));
  hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN>), dim3(static_cast<unsigned>(la[0])), dim3(256), 0, s, A, W, bias, C, M, N,
                     K, tiles_m, tiles_n);
  return check_launch("gemm");
}

}  // namespace

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
    if (cfg.block != 256) return fail("gemm: MFMA kernels use 256 threads, got %d", cfg.block);
    if (K * 2 * (bm > bn ? bm : bn) >= (int64_t{1} << 31)) return fail("gemm: K=%lld too large for 32-bit tile offsets", (long long)K);
    const int64_t tm = ceil_div(M, bm), tn = ceil_div(N, bn);
    if (tm * tn > 0x7fffffff) return fail("gemm: too many tiles");
    la[0] = tm * tn;
    la[3] = 256;
    la[4] = 2 * (bm + bn) * kRowBytes;
    la[5] = tm;
    la[6] = tn;
    return 0;
  }
  if (cfg.variant == DTAS_GEMM_SKINNY) {
    const int mt = cfg.tile[0] / 16;
    if (cfg.tile[0] % 16 != 0 || mt < 1 || mt > 5 || cfg.tile[1] != 16)
      return fail("gemm: skinny tile must be {16,32,48,64,80}x16, got %dx%d", cfg.tile[0], cfg.tile[1]);
    if (M > cfg.tile[0]) return fail("gemm: skinny tile of %d rows cannot hold M=%lld", cfg.tile[0], (long long)M);
    if (cfg.block < 64 || cfg.block > 512 || cfg.block % 64 != 0)
      return fail("gemm: block must be a multiple of 64 in [64, 512], got %d", cfg.block);
    la[0] = ceil_div(N, 16);
    la[3] = cfg.block;
    la[4] = 8 * mt * 64 * 16;
    la[5] = 1;
    la[6] = la[0];
    return 0;
  }
  return fail("gemm: unknown variant %d", cfg.variant);
}

}  // namespace dtas

extern "C" int dtas_gemm_f16(const void* A, const void* W, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                             const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (M < 0 || N < 0 || K < 0) return fail("gemm: negative extent M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (M == 0 || N == 0) return 0;
  if ((K != 0 && (M > INT64_MAX / 4 / K || N > INT64_MAX / 4 / K)) || M > INT64_MAX / 4 / N) return fail("gemm: extents overflow");
  if (!C || (K > 0 && (!A || !W))) return fail("gemm: NULL buffer");
  if (overlaps(C, M * N * 2, A, M * K * 2) || overlaps(C, M * N * 2, W, N * K * 2)) return fail("gemm: output overlaps an input");
  // one row of A is the decode GEMV: same PrimFunc shape, dedicated kernel
  if (!user && M == 1) return dtas_gemv_f16(A, W, bias, C, N, K, nullptr, stream);
  dtas_config cfg = user ? *user : builtin_config(DTAS_OP_GEMM_F16, M, N, K).cfg;
  const bool vec_ok = K % 8 == 0 && aligned(A, 16) && aligned(W, 16);
  if (cfg.vec == 8 && !vec_ok) {
    if (user) return fail("gemm: 128-bit accesses need K %% 8 == 0 and 16-byte aligned A, W");
    cfg.vec = 1;
  }
  int64_t la[7];
  if (describe_gemm(M, N, K, cfg, la) != 0) return -1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const half_t* a = static_cast<const half_t*>(A);
  const half_t* w = static_cast<const half_t*>(W);
  const half_t* b = static_cast<const half_t*>(bias);
  half_t* c = static_cast<half_t*>(C);
  if (cfg.vec == 1) {
    hipLaunchKernelGGL(gemm_scalar_kernel, dim3(static_cast<unsigned>(la[0])), dim3(256), 0, s, a, w, b, c, M, N, K);
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
  const int bm = cfg.tile[0], bn = cfg.tile[1];
  if (bm == 256 && bn == 256) return launch_mfma<256, 256>(la, s, a, w, b, c, M, N, K);
  if (bm == 256 && bn == 128) return launch_mfma<256, 128>(la, s, a, w, b, c, M, N, K);
  if (bm == 128 && bn == 256) return launch_mfma<128, 256>(la, s, a, w, b, c, M, N, K);
  if (bm == 128 && bn == 128) return launch_mfma<128, 128>(la, s, a, w, b, c, M, N, K);
  if (bm == 64 && bn == 128) return launch_mfma<64, 128>(la, s, a, w, b, c, M, N, K);
  if (bm == 128 && bn == 64) return launch_mfma<128, 64>(la, s, a, w, b, c, M, N, K);
  if (bm == 64 && bn == 64) return launch_mfma<64, 64>(la, s, a, w, b, c, M, N, K);
  return fail("gemm: no MFMA kernel for tile %dx%d", bm, bn);
}

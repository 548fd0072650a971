/*
 * dtas_abi.h -- C ABI of libdtas_gfx950.so: hand-written gfx950 (MI355X) kernels for
 * the PrimFuncs that DTAS's schedule rules cover, behind one shape-bucket dispatcher.
 *
 * What this replaces in the reference (paths relative to the reference checkout):
 * DTAS emits, per PrimFunc, one TVM PackedFunc host function
 *     int32_t <func>(void* args, int32_t* arg_type_ids, int32_t num_args, ...)
 * (experiment/dtas_tuned/elementwise/add/float16/top1_256/host.cc:38-145) that unpacks
 * DLTensor handles, reads the dynamic extent n from shape[1], looks up
 * call_table[index_table[min(n/div, last)]] and launches the bucket's kernel with
 * launch_args = {grid, block[, dyn smem]} through TVM's CUDA module.  Each entry
 * point below is that host function with the DLTensor unpacking already done: plain
 * device pointers and extents in, 0 / -1 out.  The kernel behind it is the replacement
 * for the bucket kernels *_n_<lo>_to_<hi>__kernel in tvm_device_kernels.cu.
 *
 * Conventions (all entry points):
 *  - destination passing: the caller owns every buffer, outputs included
 *    (experiment/dtas_tuned/elementwise/cast/profile_cast.py:15-18);
 *  - buffers are compact row-major, as the reference requires (strides == NULL,
 *    host.cc:64-69); the leading batch-1 dim of (1, n, H) is not passed;
 *  - `stream` is a hipStream_t (NULL = the default stream); nothing synchronises, the kernel is
 *    enqueued on `stream` on the current device.  Nothing is allocated, with one exception:
 *    dtas_gemm_f16 with K split over workgroups (split_k > 1, 0 on the 256x256 tile, or the
 *    W-streaming kernel, also behind dtas_gemm_q8_f16_fused for few rows; the built-in table chooses
 *    these when M x N leaves CUs idle) keeps fp32 partial tiles in a workspace that the
 *    library allocates on first use and grows on demand (32 MiB at first, at most 1 GiB; growing
 *    waits for the device).  There is one workspace per (device, stream): launches on one stream are
 *    ordered by it, launches on different streams use different workspaces and may overlap; the
 *    library holds its lock from looking a workspace up to enqueueing the launch, so host threads may
 *    share a stream.  At most 16 streams per device hold one (the one used longest ago is released
 *    first, which waits for the device).  A recorded HIP graph holds the workspace's address: the
 *    first split launch on a stream, and any launch that makes its workspace grow, belong before the
 *    recording.  A cfg with split_k = 1 uses none; dtas_gemm_f16_static
 *    never allocates.  dtas_gemm_q8_f16_fused keeps a second buffer of that kind
 *    (an fp16 copy of the weights it was given) under the same rules;
 *  - `cfg` selects the kernel variant and launch shape explicitly (what one row of the
 *    reference's call_table holds); NULL = use the library's built-in bucket table; either way a
 *    128-bit variant steps down to its element-access kernel for extents or pointers that do not
 *    allow 128-bit accesses (a bucket's row must serve every n and buffer that falls in it).  The
 *    dynamic row lengths are exempt: softmax rows and attention's key count m may be any number and
 *    keep the vector kernels (accesses at the rows' own alignment);
 *  - returns 0 on success, -1 on error (the reference's host functions do the same,
 *    host.cc:75-83,133-143); dtas_last_error() gives the thread-local message;
 *  - n == 0 (an empty dynamic extent) is a no-op that returns 0; negative extents, NULL
 *    buffers with n > 0 and overlapping in/out buffers ("tir.noalias") are errors.
 */
#ifndef DTAS_ABI_H_
#define DTAS_ABI_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DTAS_ABI_VERSION 1

/* ---- op families = the reference's FuncKind (python/dtas/common/analisys.py:49-55) */
enum dtas_kind {
  DTAS_KIND_ELEMENTWISE = 0,
  DTAS_KIND_REDUCTION = 1,
  DTAS_KIND_GEMV = 2,
  DTAS_KIND_GEMM = 3
};

/* ---- ops (one per PrimFunc / dtype combination with its own kernel set) */
enum dtas_op {
  DTAS_OP_ADD_F16 = 0,
  DTAS_OP_ADD_F32,
  DTAS_OP_ADD_I8,
  DTAS_OP_COPY_F16,
  DTAS_OP_COPY_F32,
  DTAS_OP_COPY_I8,
  DTAS_OP_CAST_F16_F32,
  DTAS_OP_CAST_F32_F16,
  DTAS_OP_LAYER_NORM_F32_F16,
  DTAS_OP_RMS_NORM_F16,
  DTAS_OP_SOFTMAX_F32_F16,
  DTAS_OP_SOFTMAX_F16,
  DTAS_OP_GEMV_F16,
  DTAS_OP_GEMM_F16,
  DTAS_OP_COUNT
};

/* ---- kernel variants (the `variant` field of dtas_config) */
enum dtas_variant {
  /* elementwise (python/dtas/schedule/tir_elementwise.py:23-47) */
  DTAS_ELT_VECTOR = 0,    /* `vec`-wide accesses, `unroll` in flight per thread, grid-stride */
  DTAS_ELT_SCALAR = 1,    /* one element per access: any alignment */
  /* row reductions (python/dtas/schedule/tir_reduction.py:36-105) */
  DTAS_RED_WAVE_ROW = 0,  /* one wavefront per row, row held in registers, DPP reduction */
  DTAS_RED_BLOCK_ROW = 1, /* one workgroup per row, row in registers, DPP + LDS staging */
  DTAS_RED_STREAM_ROW = 2,/* one workgroup per row, row re-read per pass: any length / alignment */
  /* GEMV (python/dtas/schedule/tir_gemv.py:33-249) */
  DTAS_GEMV_SPLITK = 0,   /* K split over the lanes and wavefronts of a workgroup; fp32 sums */
  DTAS_GEMV_RF16 = 1,     /* every sum in fp16, in the order of the reference's scheduled kernel
                             (experiment/testIR/GEMV/m1n2560k10240/IR/5wt.py:11-92): for results bit-identical to
                             that kernel's arithmetic; block 256 (8 rows per workgroup), vec 8 or 1 */
  /* GEMM (python/dtas/schedule/tir_wmma.py:20-222) */
  DTAS_GEMM_MFMA = 0,     /* LDS-tiled MFMA, tile = tile[0] x tile[1] x 64 with tile[0], tile[1] in {64, 128, 256}
                             (64x256 and 256x64 excepted); block 256 (4 wavefronts), or 512 (8 wavefronts, 16x16x32
                             MFMA, a ring of five operand units instead of `unroll` stages) for 256x256, 256x128
                             and 128x256; 256x256 takes either.  192x256 and 192x128 exist with block 512 and
                             unroll 2 only */
  DTAS_GEMM_SKINNY = 1,   /* small M: weight-streaming MFMA 16x16x32, split over N and K */
  DTAS_GEMM_ROWS = 2,     /* M <= 4: W streamed once in whole rows (tile[1] per wavefront) against tile[0] >= M
                             rows of A on the vector ALU; tile = {2|4, 1|2|4, 8}, block 64 / 128 / 256 */
  DTAS_GEMM_STREAM = 3,   /* M <= tile[0] in {16, 32, 64}: W streamed once, 1 KiB of a row per access, through the LDS to
                             MFMA 16x16x32; a workgroup of tile[1] / 16 wavefronts owns tile[1] in {64, 128} columns and
                             tile[2] in {512, 1024} elements of K, the K slices are added up in the workspace;
                             (tile[0] + tile[1]) * tile[2] * 2 bytes of LDS, block = 4 * tile[1].
                             tile[2] = 256 is the looping form for a W with many rows: tile = {16, 16 | 64, 256}, a
                             workgroup owns its columns over the whole of K and walks it in segments of 256 through a
                             ring of four LDS stages; no workspace */
  DTAS_GEMM_MFMA_ACC16 = 4 /* the reference's scheduled arithmetic: an fp16 accumulator updated once per k step of 16 by one
                             matrix-core instruction, as its wmma 16x16x16 kernels with a float16 "wmma.accumulator" do
                             (experiment/testIR/GEMM/m_n2560_k10240/wmma/16x16x16/i2j4_x7y2_in8.py:19,37): the 16 products
                             of a step are added to the accumulator at fp32 precision and the sum is rounded to fp16 before
                             the next step.  tile = {64, 64, 16}, block 256, vec 8 or 1, split_k 1 (the rounding order
                             admits no K split); any M; never the built-in choice.  A mode for comparing against the
                             reference's own numbers, not for speed: every step waits for its rounding */
};

/* One row of a call table: the launch-relevant part of the reference's *Config classes
 * (python/dtas/common/config.py:193-429: ElementwiseConfig{len_tx, vector_size, grid_size},
 * ReductionConfig{len_tx, vector_size, temp_storage}, GEMVConfig{TS, TR, TILE_R, VEC_C},
 * WMMAConfig{i, j, micro_shape}). */
typedef struct dtas_config {
  int32_t variant;  /* enum dtas_variant of the op's family */
  int32_t block;    /* threads per workgroup = launch_args[3] */
  int32_t vec;      /* elements per vector access */
  int32_t unroll;   /* elementwise/GEMV: independent vector accesses in flight per thread; row
                       reductions: rows a lane group takes per trip (1, 2, 4); GEMM: LDS stages (0 = max) */
  int32_t tile[3];  /* GEMM: workgroup tile M, N, K; GEMV: rows per workgroup, -, - */
  int32_t split_k;  /* GEMM (MFMA): workgroups that share a tile and split its K extent, 1..16 (1 = none).
                     * 0 on the 256x256 tile with 512 threads: whole rounds of the chip are not split, the tiles of a
                     * last, partly filled round are shared by 2..4 workgroups each (elsewhere 0 means 1) */
  int64_t grid_cap; /* upper limit on workgroups (then the kernel loops); 0 = no limit */
} dtas_config;

/* What the dispatcher decided for one call: the analogue of
 * `kernel_entry_info info = call_table[index_table[index]]` (host.cc:105-125,
 * python/dtas/codegen/runtime_packer.py:32-40). */
typedef struct dtas_launch_info {
  int64_t launch_args[7]; /* grid.x, grid.y, grid.z, block.x, dynamic LDS bytes, then two figures of the family:
                           * row reductions: register iterations per row, rows per workgroup trip; GEMV: rows per
                           * workgroup, 0; GEMM (MFMA): tiles along M, tiles along N; other GEMM kernels: 1, grid.x;
                           * elementwise: 0, 0 */
  int64_t bucket_lo;      /* the merged bucket [lo, hi] of the dynamic extent that n fell in */
  int64_t bucket_hi;
  int32_t index;          /* min((n - 1) / range_div, last): position in the index table */
  int32_t table_row;      /* index_table[index] */
  dtas_config config;
  char name[96];          /* "<func>_<var>_<lo>_to_<hi>__kernel" (python/dtas/common/config.py:28-31) */
} dtas_launch_info;

/* ---- library ------------------------------------------------------------ */
int dtas_abi_version(void);
/* Thread-local text of the last error on this thread ("" if none). */
const char* dtas_last_error(void);
/* Checks that the current device is a gfx950 part, loads the library's code object on it and looks up the
 * static scratch array of dtas_gemm_f16_static there.  Optional: every entry point works without it. */
int dtas_init(void);

/* The built-in bucket table: which config a call with these extents uses.
 * n = the dynamic extent (rows n; softmax: cols when dynamic; GEMM: M), d0/d1 = static extents
 * (elementwise/norm: H, 0; softmax: rows, cols; GEMV: N, K; GEMM: N, K). */
int dtas_select_bucket(int op, int64_t n, int64_t d0, int64_t d1, dtas_launch_info* out);
/* Resolve launch_args for an explicit config (used by tuners to inspect candidates). */
int dtas_describe_launch(int op, int64_t n, int64_t d0, int64_t d1, const dtas_config* cfg,
                         dtas_launch_info* out);

/* ---- elementwise: tuning_test/tune_ele_add.py:10-22, tune_ele_copy.py:10-21,
 *      tune_cast.py:10-21; dtype variants under experiment/dtas_tuned/elementwise/ ------- */
/* T_add[n,H] = A[n,H] + B[n,H] */
int dtas_add_f16(const void* A, const void* B, void* T_add, int64_t n, int64_t H,
                 const dtas_config* cfg, void* stream);
int dtas_add_f32(const void* A, const void* B, void* T_add, int64_t n, int64_t H,
                 const dtas_config* cfg, void* stream);
int dtas_add_i8(const void* A, const void* B, void* T_add, int64_t n, int64_t H,
                const dtas_config* cfg, void* stream);
/* B[n,H] = A[n,H], bit for bit */
int dtas_copy_f16(const void* A, void* B, int64_t n, int64_t H, const dtas_config* cfg, void* stream);
int dtas_copy_f32(const void* A, void* B, int64_t n, int64_t H, const dtas_config* cfg, void* stream);
int dtas_copy_i8(const void* A, void* B, int64_t n, int64_t H, const dtas_config* cfg, void* stream);
/* compute[n,H] = Cast(A[n,H]): fp16 -> fp32 is the reference's direction, fp32 -> fp16 the
 * narrowing one (round to nearest even, overflow to +-inf) */
int dtas_cast_f16_f32(const void* A, void* compute, int64_t n, int64_t H, const dtas_config* cfg,
                      void* stream);
int dtas_cast_f32_f16(const void* A, void* compute, int64_t n, int64_t H, const dtas_config* cfg,
                      void* stream);

/* ---- row reductions ------------------------------------------------------ */
/* fused_layer_norm_cast1 (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:607-636):
 * x fp32 [n,H], gamma/beta fp32 [H] -> out fp16 [n,H]; eps is 1e-5 in the PrimFunc. */
int dtas_layer_norm_f32_f16(const void* x, const void* gamma, const void* beta, void* out,
                            int64_t n, int64_t H, float eps, const dtas_config* cfg, void* stream);
/* layer_norm / layer_norm1 (before_dl.py:846-896): the same normalisation with an fp32 output (the graph's last
 * layer norm, in front of the vocabulary projection). */
int dtas_layer_norm_f32(const void* x, const void* gamma, const void* beta, void* out, int64_t n, int64_t H,
                        float eps, void* stream);
/* RMSNorm (no PrimFunc in the reference; the benchmark's norm): x fp16 [n,H], w fp16 [H]
 * -> out fp16 [n,H] = x * rsqrt(mean(x^2) + eps) * w, fp32 arithmetic. */
int dtas_rms_norm_f16(const void* x, const void* w, void* out, int64_t n, int64_t H, float eps,
                      const dtas_config* cfg, void* stream);
/* fused_softmax_cast (experiment/dtas_tuned/general_reduction/softmax/profile_dlight.py:8-52,
 * before_dl.py:756-800): softmax over the last axis of A[rows, cols], fp32 math, fp16 out.
 * The (1,32,n,m) form is rows = 32*n, cols = m. */
int dtas_softmax_f32_f16(const void* A, void* out, int64_t rows, int64_t cols,
                         const dtas_config* cfg, void* stream);
int dtas_softmax_f16(const void* A, void* out, int64_t rows, int64_t cols, const dtas_config* cfg,
                     void* stream);
/* divide2 (before_dl.py:57-65): out[count] = A[count] / *B, fp32, B one value in device memory (the PrimFunc's
 * 0-d buffer); the correctly rounded division.  softmax2 (:1062-1096): fp32 softmax over each row, fp32 out. */
int dtas_divide_f32(const void* A, const void* B, void* out, int64_t count, void* stream);
int dtas_softmax_f32(const void* A, void* out, int64_t rows, int64_t cols, void* stream);
/* softmax_with_temperature (before_dl.py:4154-4161): divide2 (:57-65) then softmax2 (:1062-1096).
 * out[rows, cols] fp32 = softmax over each row of logits[rows, cols] / *temperature; `temperature` points at
 * one fp32 in device memory (the PrimFunc's 0-d buffer B). */
int dtas_softmax_temperature_f32(const void* logits, const void* temperature, void* out, int64_t rows,
                                 int64_t cols, void* stream);

/* take (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:1151-1163; one row: take1, :1166-1174), the
 * embedding lookup: out[n, H] = A[ids[i], :] for a table A[V, H] fp16 and ids[n] int32 (n dynamic).  Ids
 * outside [0, V) are clipped to the nearest row.  cfg, when given: {DTAS_ELT_VECTOR, block 256, vec 8 | 1}. */
int dtas_take_f16(const void* A, const void* ids, void* out, int64_t n, int64_t V, int64_t H,
                  const dtas_config* cfg, void* stream);

/* rotary_embedding (before_dl.py:1023-1035; one row: rotary_embedding1, :1038-1047), applied to the queries
 * and keys before the scores: A and out are [n, heads, d] fp16 (n dynamic), cos and sin [max_pos, rot] fp16;
 * the first rot elements of every row are rotated with the tables' row m + s - n for position s (m = the
 * length of the whole sequence, m >= n), each step an fp16 value:
 *   out[j] = cos[j] * A[j] + sin[j] * (j < rot/2 ? A[j + rot/2] * -1 : A[j - rot/2])   (j < rot);  A[j] else.
 * cfg, when given: {DTAS_ELT_VECTOR, block 256, vec 8, unroll 0 | 1 | 2}; unroll names the kernel (0: whole rows per
 * wavefront, for rot = 20 and d <= 512; 1: a 16-byte piece per thread with its partners and table entries in the widest
 * loads the width allows -- rot = 20, rot % 16 == 0, rot % 4 == 0; 2: element by element, any even rot) -- the results
 * are the same bits; 0 and 1 step down to the next form where theirs does not apply. */
int dtas_rotary_f16(const void* A, const void* cos_t, const void* sin_t, void* out, int64_t n, int64_t m,
                    int64_t heads, int64_t d, int64_t rot, int64_t max_pos, const dtas_config* cfg, void* stream);

/* The attention mask: fused_min_max_triu_te_broadcast_to (before_dl.py:642-658) followed by extend_te (:68-80),
 * and full (:83-93) when n = 1.  out[n, m] fp16 (n query positions, m >= n key positions, both dynamic):
 *   out[i, j] = j - (m - n) > i ? -65504 : 65504. */
int dtas_attn_mask_f16(void* out, int64_t n, int64_t m, void* stream);
/* transpose6 / transpose7 (before_dl.py:1177-1203): A[a, b, d] -> out[b, a, d] fp16, rows of d elements
 * (d % 8 == 0) moved whole: [n, heads, d] <-> [heads, n, d] around the attention kernels. */
int dtas_swap_axes_f16(const void* A, void* out, int64_t a, int64_t b, int64_t d, void* stream);
/* split (before_dl.py:1099-1125) and fused_reshape7_split1 (:661-688): the fused projection A[rows, 3 d] fp16
 * (rows = positions x heads) cut into out0 / out1 / out2 [rows, d], section s = columns [s d, (s + 1) d). */
int dtas_split3_f16(const void* A, void* out0, void* out1, void* out2, int64_t rows, int64_t d, void* stream);

/* ---- GEMV: fused_NT_matmul10_add5 (before_dl.py:96-113) ------------------
 * y[N] = W[N,K] . x[K] (+ bias[N] when bias != NULL); fp16 in/out, fp32 accumulate. */
int dtas_gemv_f16(const void* x, const void* W, const void* bias, void* y, int64_t N, int64_t K,
                  const dtas_config* cfg, void* stream);
/* The decode GEMVs with the epilogues of dtas_gemm_f16_fused (a DTAS_EPI_* value, defined below; the
 * same fp16 steps): fused_NT_matmul8_add5_add7_add7 (before_dl.py:408-439; DTAS_EPI_BIAS_ADD2, res1
 * and res2 are [N] fp16), .._cast5 (:442-480; DTAS_EPI_BIAS_ADD2_CAST_F32, y is fp32),
 * fused_NT_matmul9_add6_gelu1 (:483-549; DTAS_EPI_BIAS_GELU).  res1 = res2 = NULL for the kinds without
 * residuals.  dtas_gemm_f16_fused with M == 1 and cfg == NULL lands here. */
int dtas_gemv_f16_fused(const void* x, const void* W, const void* bias, const void* res1, const void* res2,
                        void* y, int64_t N, int64_t K, int32_t epilogue, const dtas_config* cfg, void* stream);

/* ---- GEMM: fused_NT_matmul4_add1 (before_dl.py:320-341) -------------------
 * C[M,N] = A[M,K] . W[N,K]^T (+ bias[N] when bias != NULL); M is the dynamic extent;
 * fp16 in/out, fp32 accumulate on MFMA.
 * Memory orderings a launch with K split over workgroups relies on (the partial tiles and arrival counters in the
 * workspace are the only data of the library that one workgroup writes and another reads within a launch):
 *  (1) a partial tile is written with device-scope (agent) relaxed atomic stores, which write through the XCD's L2;
 *      the writing wavefront then waits until none of its stores is outstanding, and a write-through store is
 *      acknowledged only once it is visible to every XCD;
 *  (2) a workgroup barrier follows, and only then one thread adds 1 to the tile's counter with a device-scope
 *      relaxed atomic read-modify-write, which is performed at the memory side, once, for all XCDs;
 *  (3) the workgroup that reads nsplit - 1 there therefore knows that steps (1)-(2) of every other part are complete;
 *      it reads the other parts' tiles with device-scope relaxed atomic loads, which do not hit in its own L2, adds
 *      them in part order (the sum does not depend on who arrives last), and sets the counter back to 0.
 *  No release/acquire fence is used (a device-scope fence writes back and invalidates a whole L2); the order rests on
 *  (1)'s wait and on (2) following the barrier.  Launches that share a workspace must not overlap: the library keeps
 *  one workspace per (device, stream). */
int dtas_gemm_f16(const void* A, const void* W, const void* bias, void* C, int64_t M, int64_t N,
                  int64_t K, const dtas_config* cfg, void* stream);

/* ---- GEMM that allocates nothing ------------------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory where they call: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  dtas_gemm_f16 in every respect (same
 * kernels, same results bit for bit), except that a launch which splits K keeps its fp32 partial tiles and arrival
 * counters in a static device array of the library -- DTAS_STATIC_SCRATCH_PARTIAL_BYTES of partial tiles and
 * DTAS_STATIC_SCRATCH_COUNTERS counters (tiles that are split), held by every GPU the library runs on from the
 * first use of the library on it until the process ends -- instead of the workspace dtas_gemm_f16 allocates.  It
 * calls no hipMalloc, no hipFree and no other allocating routine; a launch that needs more scratch than the array
 * holds returns -1 and says how much (pass a cfg with split_k = 1, or a smaller split).  All calls on one GPU share
 * the array, whatever their streams: calls that overlap in time on one GPU race -- order them (one stream, or
 * events).  dtas_init() resolves the array's address on the current device; otherwise the first call on a
 * device does, which asks the runtime for a symbol address: a call under stream capture therefore requires that
 * dtas_init() (or an uncaptured call) has run on that device before.  The counters are never cleared by a call:
 * the array is zero when the library's code is loaded and every launch leaves its counters at zero. */
#define DTAS_STATIC_SCRATCH_PARTIAL_BYTES (32u << 20)
#define DTAS_STATIC_SCRATCH_COUNTERS 4096u
int dtas_gemm_f16_static(const void* A, const void* W, const void* bias, void* C, int64_t M, int64_t N,
                         int64_t K, const dtas_config* cfg, void* stream);

/* ---- GEMM with the model's fused epilogues ------------------------------------
 * The PrimFuncs keep every intermediate as an fp16 tensor, so each step rounds to fp16:
 *  DTAS_EPI_BIAS               C = mm (+ bias)                        fused_NT_matmul4_add1, before_dl.py:320-341
 *  DTAS_EPI_BIAS_ADD2          C = (res1 + (mm + bias)) + res2        fused_NT_matmul2_add1_add3_add3, :163-200
 *  DTAS_EPI_BIAS_ADD2_CAST_F32 the same, widened into an fp32 C       fused_NT_matmul2_add1_add3_add3_cast, :202-246
 *  DTAS_EPI_BIAS_GELU          t = mm + bias; C = t * (0.5 + 0.5 * erf(t * fp16(0.7071...)))
 *                                                                      fused_NT_matmul3_add2_gelu, :248-318
 * mm = A[M,K] . W[N,K]^T accumulated in fp32 and rounded to fp16 once.  res1, res2: [M,N] fp16,
 * required by the ADD2 kinds and NULL otherwise; bias may be NULL for any kind. */
enum dtas_epilogue {
  DTAS_EPI_BIAS = 0,
  DTAS_EPI_BIAS_ADD2 = 1,
  DTAS_EPI_BIAS_ADD2_CAST_F32 = 2,
  DTAS_EPI_BIAS_GELU = 3
};
int dtas_gemm_f16_fused(const void* A, const void* W, const void* bias, const void* res1,
                        const void* res2, void* C, int64_t M, int64_t N, int64_t K,
                        int32_t epilogue, const dtas_config* cfg, void* stream);

/* ---- attention scores: fused_NT_matmul1_divide_maximum_minimum_cast2 (before_dl.py:116-160) ----
 * out[h,i,j] = fp32(min(max(fp16(fp16(Q[h,i,:] . K[h,j,:]) * fp16(scale)), -65504), mask[i,j]))
 * Q[heads,n,d], K[heads,m,d], mask[n,m] fp16 (shared by the heads), out[heads,n,m] fp32; n and m are the
 * dynamic extents, d (80 in the model) a multiple of 8.  One batched launch over the heads on the MFMA
 * kernels; cfg, when given, is a DTAS_GEMM_MFMA row for the per-head (n, m, d) problem, or a DTAS_GEMM_SKINNY row
 * {block 1024, vec 8, tile {1|2|4|8, 8, k}} for the kernel that serves a handful of query rows (decoding): that many
 * rows per workgroup, k keys per workgroup (a multiple of 1024 / (d / 8); 0: chosen), d <= 1024. */
int dtas_attn_scores_f16_f32(const void* Q, const void* K, const void* mask, void* out, int64_t heads,
                             int64_t n, int64_t m, int64_t d, float scale, const dtas_config* cfg,
                             void* stream);

/* ---- attention output: matmul8 (before_dl.py:915-929; n dynamic) and matmul10 (:899-912; n = 1) ----
 * out[h,i,:] = sum_k P[h,i,k] * V[h,k,:]
 * P[heads,n,m] (the softmaxed scores), V[heads,m,d], out[heads,n,d], all fp16; n and m are the dynamic
 * extents.  V is k-major (its rows run along d): its tiles lie in the LDS as in memory and the matrix-core operands
 * are read from there transposed.
 * fp32 accumulation, one rounding to fp16.  cfg, when given: a DTAS_GEMM_MFMA row for the per-head
 * (n, d, m) problem with tile {64|128, 64|128, 64} and two stages, or {64|128|256, 128, 64} and three (split_k > 1:
 * the workgroups of a (head, tile) split m and meet in the split-K workspace), or a DTAS_GEMM_SKINNY row
 * {block 256, tile {1|2|4|8, 8, 0}} for the kernel that serves a handful of rows (decoding), or {block 1024, tile {1, 8, 0}}
 * for one workgroup per (head, row) that reads the head's V in one contiguous sweep (d <= 1024) -- tile[2] = c > 0
 * (a multiple of 8 that divides d, at most `block`; block 256, 512 or 1024): d / c workgroups per (head, row), c columns
 * each; split_k = s > 1 (at most 64): s workgroups share the keys, a run each, and meet in the split-K workspace.  With m % 8 != 0
 * or a P off a 16-byte boundary the MFMA kernels read the rows of P where they lie (16-byte pieces at 2-byte
 * alignment; the last m % 8 keys are added in the epilogue, in fp32, before the one rounding);
 * d % 8 != 0 or a V off 16 bytes fall back to the element-access kernel; m == 0 writes zeros. */
int dtas_attn_pv_f16(const void* P, const void* V, void* out, int64_t heads, int64_t n, int64_t m,
                     int64_t d, const dtas_config* cfg, void* stream);

/* ---- fp32 GEMV: NT_matmul5 (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:8-19), the 50280 x 2560
 * vocabulary projection of the decode graph: y[N] = x[K] . W[N,K]^T, all fp32, no bias.  cfg, when given, is a
 * DTAS_GEMV_SPLITK row with vec 4 (128-bit accesses) or 1. */
int dtas_gemv_f32(const void* x, const void* W, void* y, int64_t N, int64_t K, const dtas_config* cfg,
                  void* stream);

/* ---- 8-bit weights with fp16 group scales (the q8f16_1 layout of
 * experiment/ModelIR/dolly-v2-3b-q8f16_1/before_dl.py) ----
 * Wq[N, K/4] uint32: element j of a row is byte j % 4 of word j / 4; scale[N, K/32] fp16; K % 32 == 0.
 *   W[i,j] = (fp16(byte) - fp16(127)) * scale[i, j/32]       (fp16 arithmetic: the product is rounded once)
 *
 * dtas_decode_q8_f16: fused_decode3 (:335-343), the dequantiser on its own: W[N,K] fp16 out.  cfg, when given:
 *   {DTAS_ELT_VECTOR, block 256, vec 8 (8 weights per access: 128-bit stores) or 1}.
 * dtas_gemv_q8_f16: y[N] = x[K] . W^T (+ bias[N]) with W dequantised in registers, never written:
 *   fused_fused_decode2_fused_NT_matmul_add (:401-426; epilogue DTAS_EPI_BIAS) and
 *   fused_fused_decode4_fused_NT_matmul3_add2_gelu (:428-502; DTAS_EPI_BIAS_GELU); fp32 accumulation, then
 *   the fp16 steps of dtas_gemm_f16_fused.  cfg, when given, is a DTAS_GEMV_SPLITK row as for dtas_gemv_f16
 *   (vec 8 = 128-bit accesses); NULL = 256 threads and 2 (N >= 16384: 4) rows per workgroup.
 */
/* dtas_take_q8_f16: fused_fused_decode1_take1 (:357-369; one row: fused_fused_decode1_take, :346-355), the
 *   embedding rows dequantised: out[n, K] fp16 = decode(Wq, scale)[ids[i], :], Wq[V, K/4], scale[V, K/32] fp16,
 *   ids[n] int32.  Ids outside [0, V) are clipped to the nearest row.  cfg as dtas_decode_q8_f16.
 * dtas_gemv_q8_f32: fused_fused_decode6_NT_matmul5 (:640-657), the vocabulary projection of the 8-bit model:
 *   x[K], y[N] and scale[N, K/32] are fp32; W = float32(fp16(byte) - fp16(127)) * scale (one fp32 rounding);
 *   y = x . W^T in fp32.  cfg as dtas_gemv_q8_f16. */
int dtas_take_q8_f16(const void* Wq, const void* scale, const void* ids, void* out, int64_t n, int64_t V, int64_t K,
                     const dtas_config* cfg, void* stream);
int dtas_gemv_q8_f32(const void* x, const void* Wq, const void* scale, void* y, int64_t N, int64_t K,
                     const dtas_config* cfg, void* stream);
/* dtas_gemm_q8_f16_fused: C[M,N] = epilogue(A[M,K] . W^T) with W dequantised on its way into the LDS, never
 * written: the dynamic-n forms fused_fused_decode2_fused_NT_matmul6_add4 (:371-399), ..decode4.._matmul9_add6_gelu1
 * (:504-581), ..decode5.._matmul4_add1; epilogues as dtas_gemm_f16_fused.  cfg, when given: a DTAS_GEMM_MFMA row
 * with tile {256,128,64}, {128,128,64}, {128,64,64} or {64,128,64} and unroll 3, or {64,64,64} and unroll 2 or 3; or a DTAS_GEMM_STREAM row
 * (block 256, tile {16,64,512}, {16,64,1024}, {32,64,512} or {64,64,512}; M <= tile[0]; K % 256 == 0; 16-byte
 * aligned A, Wq and scale): the W-streaming kernel on the bytes of W, widened between the LDS and the MFMA; its K
 * slices meet in the split-K workspace.  A DTAS_GEMM_MFMA row may carry split_k in [1, 16]: that many workgroups share
 * a tile and meet in the split-K workspace as in dtas_gemm_f16.  One row with a bias or GELU epilogue goes to
 * dtas_gemv_q8_f16.  With cfg == NULL: M <= 32 (M <= 64 while N / 64 x K / 512 workgroups fit one round of the chip) takes the W-streaming kernel where it
 * applies; up to 512 rows, while 128x128 tiles fit the chip in one round, the tile kernel dequantises in its W path
 * (64x64, 128x64 or 128x128 tiles of three stages with K in 1 .. 8 parts, by a fitted cost model); beyond that the two-pass route:
 * dtas_decode_q8_f16 into a per-device fp16 buffer of its own (allocated on first use, grown on demand, at most
 * 1 GiB; same sharing rule as the split-K workspace), then dtas_gemm_f16_fused. */
int dtas_gemm_q8_f16_fused(const void* A, const void* Wq, const void* scale, const void* bias,
                           const void* res1, const void* res2, void* C, int64_t M, int64_t N, int64_t K,
                           int32_t epilogue, const dtas_config* cfg, void* stream);
int dtas_decode_q8_f16(const void* Wq, const void* scale, void* W, int64_t N, int64_t K,
                       const dtas_config* cfg, void* stream);
int dtas_gemv_q8_f16(const void* x, const void* Wq, const void* scale, const void* bias, void* y,
                     int64_t N, int64_t K, int32_t epilogue, const dtas_config* cfg, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DTAS_ABI_H_ */

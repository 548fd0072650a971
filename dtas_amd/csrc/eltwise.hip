// Elementwise add / copy / cast for gfx950.
//
// Replaces the kernels that DTAS's elementwise rule generates
// (python/dtas/schedule/tir_elementwise.py:23-47: fuse all loops, split into
// [grid, loop, 256 threads, vector], bind, vectorize; generated form
// experiment/dtas_tuned/elementwise/add/float16/top1_256/tvm_device_kernels.cu:90-107).
//
// MI355X shape of the same idea: the fused (1, n, H) space is one flat array; a thread
// moves `vec` contiguous elements per access (up to 128 bit on the narrower side), a
// wavefront's 64 accesses are one contiguous span, each thread keeps `unroll` accesses in
// flight, a workgroup is 256 threads (4 wavefronts) and walks tiles of 256*unroll vectors
// grid-stride.  Accesses are marked non-temporal: every byte is touched once.
#include "dtas_device.h"
#include "dtas_host.h"

namespace dtas {
namespace {

constexpr int kBlock = 256;
// Workgroups per launch of the index-only kernels: a thread per 16-byte piece for as long as a launch may hold them
// (fewer than 2^32 threads) and a grid-stride loop beyond.  A grid capped at a few dozen workgroups per CU that loops
// writes slower: the [16384, 16384] mask, 537 MB, takes 107 us with 64 workgroups per CU looping 8 times and 77 us (7.0 TB/s)
// with a workgroup per 4 KiB; 134 MB 23.7 / 22.0.
constexpr int64_t kMaxGrid = int64_t{1} << 23;

// ---- raw fixed-size accesses ------------------------------------------------------
template <int BYTES>
struct Raw;
template <>
struct Raw<1> {
  uint8_t d;
  static __device__ __forceinline__ Raw load(const void* p, int64_t i) { return {load_stream(static_cast<const uint8_t*>(p) + i)}; }
  __device__ __forceinline__ void store(void* p, int64_t i) const { store_stream(d, static_cast<uint8_t*>(p) + i); }
};
template <>
struct Raw<2> {
  uint16_t d;
  static __device__ __forceinline__ Raw load(const void* p, int64_t i) { return {load_stream(static_cast<const uint16_t*>(p) + i)}; }
  __device__ __forceinline__ void store(void* p, int64_t i) const { store_stream(d, static_cast<uint16_t*>(p) + i); }
};
template <>
struct Raw<4> {
  uint32_t d;
  static __device__ __forceinline__ Raw load(const void* p, int64_t i) { return {load_stream(static_cast<const uint32_t*>(p) + i)}; }
  __device__ __forceinline__ void store(void* p, int64_t i) const { store_stream(d, static_cast<uint32_t*>(p) + i); }
};
template <>
struct Raw<8> {
  u32x2 d;
  static __device__ __forceinline__ Raw load(const void* p, int64_t i) { return {load_stream(static_cast<const u32x2*>(p) + i)}; }
  __device__ __forceinline__ void store(void* p, int64_t i) const { store_stream(d, static_cast<u32x2*>(p) + i); }
};
template <>
struct Raw<16> {
  u32x4 d;
  static __device__ __forceinline__ Raw load(const void* p, int64_t i) { return {load_stream(static_cast<const u32x4*>(p) + i)}; }
  __device__ __forceinline__ void store(void* p, int64_t i) const { store_stream(d, static_cast<u32x4*>(p) + i); }
};
template <>
struct Raw<32> {
  u32x4 d[2];
  static __device__ __forceinline__ Raw load(const void* p, int64_t i) {
    const u32x4* q = static_cast<const u32x4*>(p) + 2 * i;
    return {{load_stream(q), load_stream(q + 1)}};
  }
  __device__ __forceinline__ void store(void* p, int64_t i) const {
    u32x4* q = static_cast<u32x4*>(p) + 2 * i;
    store_stream(d[0], q);
    store_stream(d[1], q + 1);
  }
};

template <typename T, int VEC>
struct Elems {
  T v[VEC];
};

// ---- the three element functions ----------------------------------------------------
// fp16 add is one IEEE rounding per lane (v_add_f16 / v_pk_add_f16), as the generated CUDA
// does with per-lane `half` adds; int8 wraps modulo 256.
template <typename T>
struct AddOp {
  typedef T In;
  typedef T Out;
  static constexpr int kInputs = 2;
  static constexpr bool kBytewise = false;
  static __device__ __forceinline__ T apply(T a, T b) { return a + b; }
  static __device__ __forceinline__ uint32_t apply_word(uint32_t a, uint32_t) { return a; }  // (unused)
};
template <>
struct AddOp<int8_t> {
  typedef int8_t In;
  typedef int8_t Out;
  static constexpr int kInputs = 2;
  static constexpr bool kBytewise = true;
  static __device__ __forceinline__ int8_t apply(int8_t a, int8_t b) {
    return static_cast<int8_t>(static_cast<uint8_t>(static_cast<uint8_t>(a) + static_cast<uint8_t>(b)));
  }
  // four bytes at once, each modulo 256: the low 7 bits of every byte add without reaching the next byte, and the top
  // bit of a byte's sum is the xor of the two top bits and the carry into it
  static __device__ __forceinline__ uint32_t apply_word(uint32_t a, uint32_t b) {
    return ((a & 0x7f7f7f7fu) + (b & 0x7f7f7f7fu)) ^ ((a ^ b) & 0x80808080u);
  }
};
// Copy moves bit patterns through integer registers, so NaN payloads survive.
template <typename Bits>
struct CopyOp {
  typedef Bits In;
  typedef Bits Out;
  static constexpr int kInputs = 1;
  static constexpr bool kBytewise = sizeof(Bits) == 1;
  static __device__ __forceinline__ Bits apply(Bits a, Bits) { return a; }
  static __device__ __forceinline__ uint32_t apply_word(uint32_t a, uint32_t) { return a; }
};
// Cast: fp16 -> fp32 is exact; fp32 -> fp16 rounds to nearest even and overflows to +-inf
// (v_cvt_f16_f32), fp16 subnormal results are kept.
template <typename TI, typename TO>
struct CastOp {
  typedef TI In;
  typedef TO Out;
  static constexpr int kInputs = 1;
  static constexpr bool kBytewise = false;
  static __device__ __forceinline__ TO apply(TI a, TI) { return static_cast<TO>(a); }
  static __device__ __forceinline__ uint32_t apply_word(uint32_t a, uint32_t) { return a; }  // (unused)
};

// ---- kernels ------------------------------------------------------------------------
template <typename Op, int VEC, int U>
__global__ void __launch_bounds__(kBlock) elt_vector_kernel(const void* __restrict__ a, const void* __restrict__ b,
                                                            void* __restrict__ out, int64_t nvec, int64_t count) {
  typedef typename Op::In TI;
  typedef typename Op::Out TO;
  typedef Raw<VEC * sizeof(TI)> RI;
  typedef Raw<VEC * sizeof(TO)> RO;
  constexpr int64_t kTile = static_cast<int64_t>(kBlock) * U;
  const int64_t step = static_cast<int64_t>(gridDim.x) * kTile;
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTile; base < nvec; base += step) {
    RI ra[U], rb[U];
    const int64_t first = base + threadIdx.x;
    const bool full = base + kTile <= nvec;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = first + u * kBlock;
      if (full || i < nvec) {
        ra[u] = RI::load(a, i);
        if (Op::kInputs == 2) rb[u] = RI::load(b, i);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = first + u * kBlock;
      if (full || i < nvec) {
        RO ro;
        if constexpr (Op::kBytewise && VEC % 4 == 0) {
          // whole 32-bit words at once (byte by byte the compiler unpacks and repacks every element, and the launch is
          // bound by that arithmetic: the int8 add over [8192, 4096] took 39.5 us at 8 vectors per thread, 18.0 at one)
          uint32_t wa[VEC / 4], wb[VEC / 4], wo[VEC / 4];
          __builtin_memcpy(wa, &ra[u], sizeof(wa));
          if (Op::kInputs == 2) __builtin_memcpy(wb, &rb[u], sizeof(wb));
#pragma unroll
          for (int e = 0; e < VEC / 4; ++e) wo[e] = Op::apply_word(wa[e], Op::kInputs == 2 ? wb[e] : wa[e]);
          __builtin_memcpy(&ro, wo, sizeof(ro));
        } else {
          Elems<TI, VEC> ea, eb;
          Elems<TO, VEC> eo;
          __builtin_memcpy(&ea, &ra[u], sizeof(ea));
          if (Op::kInputs == 2) __builtin_memcpy(&eb, &rb[u], sizeof(eb)); else eb = ea;
#pragma unroll
          for (int e = 0; e < VEC; ++e) eo.v[e] = Op::apply(ea.v[e], eb.v[e]);
          __builtin_memcpy(&ro, &eo, sizeof(ro));
        }
        ro.store(out, i);
      }
    }
  }
  // the last count % VEC elements, one per thread of workgroup 0
  if (blockIdx.x == 0) {
    const int64_t i = nvec * VEC + threadIdx.x;
    if (i < count) {
      const TI x = static_cast<const TI*>(a)[i];
      const TI y = Op::kInputs == 2 ? static_cast<const TI*>(b)[i] : x;
      static_cast<TO*>(out)[i] = Op::apply(x, y);
    }
  }
}

template <typename Op, int VEC, int U>
int launch_vector(const void* a, const void* b, void* out, int64_t count, int64_t grid, hipStream_t s) {
  const int64_t nvec = count / VEC;
  hipLaunchKernelGGL((elt_vector_kernel<Op, VEC, U>), dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, s, a, b, out,
                     nvec, count);
  return check_launch("elementwise");
}

template <typename Op, int VEC>
int launch_unroll(int unroll, const void* a, const void* b, void* out, int64_t count, int64_t grid, hipStream_t s) {
  switch (unroll) {
    case 1: return launch_vector<Op, VEC, 1>(a, b, out, count, grid, s);
    case 2: return launch_vector<Op, VEC, 2>(a, b, out, count, grid, s);
    case 4: return launch_vector<Op, VEC, 4>(a, b, out, count, grid, s);
    case 8: return launch_vector<Op, VEC, 8>(a, b, out, count, grid, s);
  }
  return fail("elementwise: unroll %d is not one of 1, 2, 4, 8", unroll);
}

// Widest access is 16 bytes on the narrower of the two element types (and so at most 32 on
// the wider one); the three widths are the reference's candidates 128 / 64 / 32 bit
// (python/dtas/policy/elementwise_config_emiter.py:9-34).
template <typename Op>
int launch_op(const dtas_config& cfg, const void* a, const void* b, void* out, int64_t count, int64_t grid,
              hipStream_t s) {
  constexpr int kNarrow = sizeof(typename Op::In) < sizeof(typename Op::Out) ? sizeof(typename Op::In)
                                                                             : sizeof(typename Op::Out);
  constexpr int kMaxVec = 16 / kNarrow;
  if (cfg.variant == DTAS_ELT_SCALAR) return launch_unroll<Op, 1>(cfg.unroll, a, b, out, count, grid, s);
  if (cfg.vec == kMaxVec) return launch_unroll<Op, kMaxVec>(cfg.unroll, a, b, out, count, grid, s);
  if (cfg.vec == kMaxVec / 2) return launch_unroll<Op, kMaxVec / 2>(cfg.unroll, a, b, out, count, grid, s);
  if (cfg.vec == kMaxVec / 4) return launch_unroll<Op, kMaxVec / 4>(cfg.unroll, a, b, out, count, grid, s);
  return fail("elementwise: vector width %d not in {%d, %d, %d}", cfg.vec, kMaxVec, kMaxVec / 2, kMaxVec / 4);
}

struct EltInfo {
  int in_bytes, out_bytes, inputs;
  const char* name;
};

bool elt_info(int op, EltInfo* e) {
  switch (op) {
    case DTAS_OP_ADD_F16: *e = {2, 2, 2, "add"}; return true;
    case DTAS_OP_ADD_F32: *e = {4, 4, 2, "add"}; return true;
    case DTAS_OP_ADD_I8: *e = {1, 1, 2, "add"}; return true;
    case DTAS_OP_COPY_F16: *e = {2, 2, 1, "copy"}; return true;
    case DTAS_OP_COPY_F32: *e = {4, 4, 1, "copy"}; return true;
    case DTAS_OP_COPY_I8: *e = {1, 1, 1, "copy"}; return true;
    case DTAS_OP_CAST_F16_F32: *e = {2, 4, 1, "cast"}; return true;
    case DTAS_OP_CAST_F32_F16: *e = {4, 2, 1, "cast"}; return true;
  }
  return false;
}

int run_eltwise(int op, const void* a, const void* b, void* out, int64_t n, int64_t H, const dtas_config* user,
                void* stream) {
  clear_error();
  EltInfo e;
  if (!elt_info(op, &e)) return fail("elementwise: unknown op %d", op);
  if (n < 0 || H < 0) return fail("%s: negative extent n=%lld H=%lld", e.name, (long long)n, (long long)H);
  if (H != 0 && n > INT64_MAX / 8 / H) return fail("%s: n*H overflows", e.name);
  const int64_t count = n * H;
  if (count == 0) return 0;
  if (!a || !out || (e.inputs == 2 && !b)) return fail("%s: NULL buffer with n=%lld", e.name, (long long)n);
  if (overlaps(a, count * e.in_bytes, out, count * e.out_bytes) ||
      (e.inputs == 2 && overlaps(b, count * e.in_bytes, out, count * e.out_bytes)))
    return fail("%s: output overlaps an input (PrimFunc is tir.noalias)", e.name);

  dtas_config cfg = user ? *user : builtin_config(op, n, H, 0).cfg;
  // A vector access needs its natural alignment on every buffer; for odd pointers the call
  // steps down to element accesses (a bucket's config must serve every n and buffer in it).
  if (cfg.variant == DTAS_ELT_VECTOR) {
    const size_t ia = static_cast<size_t>(cfg.vec) * e.in_bytes, oa = static_cast<size_t>(cfg.vec) * e.out_bytes;
    const size_t ia16 = ia > 16 ? 16 : ia, oa16 = oa > 16 ? 16 : oa;
    const bool ok = cfg.vec > 0 && (ia & (ia - 1)) == 0 && aligned(a, ia16) && aligned(out, oa16) &&
                    (e.inputs == 1 || aligned(b, ia16));
    if (!ok) {
      cfg.variant = DTAS_ELT_SCALAR;
      cfg.vec = 1;
    }
  }
  int64_t la[7];
  if (describe_eltwise(op, count, cfg, la) != 0) return -1;
  const int64_t grid = la[0];
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (op) {
    case DTAS_OP_ADD_F16: return launch_op<AddOp<half_t>>(cfg, a, b, out, count, grid, s);
    case DTAS_OP_ADD_F32: return launch_op<AddOp<float>>(cfg, a, b, out, count, grid, s);
    case DTAS_OP_ADD_I8: return launch_op<AddOp<int8_t>>(cfg, a, b, out, count, grid, s);
    case DTAS_OP_COPY_F16: return launch_op<CopyOp<uint16_t>>(cfg, a, b, out, count, grid, s);
    case DTAS_OP_COPY_F32: return launch_op<CopyOp<uint32_t>>(cfg, a, b, out, count, grid, s);
    case DTAS_OP_COPY_I8: return launch_op<CopyOp<uint8_t>>(cfg, a, b, out, count, grid, s);
    case DTAS_OP_CAST_F16_F32: return launch_op<CastOp<half_t, float>>(cfg, a, b, out, count, grid, s);
    case DTAS_OP_CAST_F32_F16: return launch_op<CastOp<float, half_t>>(cfg, a, b, out, count, grid, s);
  }
  return fail("elementwise: unknown op %d", op);
}

// The embedding rows (take, experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:1151-1163; one row: take1,
// :1166-1174): out[i, :] = A[ids[i], :].  16-byte pieces, piece t of the output is piece t % per_row of row
// ids[t / per_row]; ids outside [0, V) are clipped to the nearest row (the PrimFunc reads whatever address
// they make).  `scalar`: one element per thread, any alignment.
__global__ void __launch_bounds__(kBlock) take_f16_kernel(const u32x4* __restrict__ A, const int* __restrict__ ids,
                                                          u32x4* __restrict__ out, int64_t pieces, int64_t per_row, int64_t V) {
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < pieces;
       t += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    int64_t row = ids[t / per_row];
    row = row < 0 ? 0 : row >= V ? V - 1 : row;
    store_stream(A[row * per_row + t % per_row], out + t);
  }
}
__global__ void __launch_bounds__(kBlock) take_f16_scalar_kernel(const half_t* __restrict__ A, const int* __restrict__ ids,
                                                                 half_t* __restrict__ out, int64_t total, int64_t H, int64_t V) {
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < total;
       t += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    int64_t row = ids[t / H];
    row = row < 0 ? 0 : row >= V ? V - 1 : row;
    out[t] = A[row * H + t % H];
  }
}

// rotary_embedding (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:1023-1035; one row: rotary_embedding1,
// :1038-1047): the first `rot` of the d elements of every (position, head) row are rotated, every step an fp16
// value as the PrimFunc spells it,
//   out[j] = j < rot ? cos[pos, j] * A[j] + sin[pos, j] * (j < rot/2 ? A[j + rot/2] * -1 : A[j - rot/2]) : A[j]
// with pos = m + s - n.  A thread takes 8 consecutive elements; those past `rot` are a 16-byte copy.
__global__ void __launch_bounds__(kBlock) rotary_f16_kernel(const half_t* __restrict__ A, const half_t* __restrict__ cs,
                                                            const half_t* __restrict__ sn, half_t* __restrict__ out,
                                                            int64_t pieces, int64_t heads, int64_t d, int64_t rot, int64_t pos0) {
  // (the two products and the sum are three fp16 tensor ops in the PrimFunc: no fused multiply-add, which the
  // compiler would otherwise form once it has narrowed them to fp16 instructions)
#pragma clang fp contract(off)
  const int64_t per_row = d >> 3, half_rot = rot >> 1;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < pieces;
       t += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t row = t / per_row, j0 = (t % per_row) << 3;
    const half_t* a = A + row * d;
    u32x4 raw = *reinterpret_cast<const u32x4*>(a + j0);
    if (j0 < rot) {
      const int64_t pos = pos0 + row / heads;
      f16x8 v = __builtin_bit_cast(f16x8, raw);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int64_t j = j0 + e;
        if (j < rot) {
          const half_t partner = j < half_rot ? static_cast<half_t>(static_cast<float>(a[j + half_rot]) * -1.f) : a[j - half_rot];
          const half_t t1 = static_cast<half_t>(static_cast<float>(cs[pos * rot + j]) * static_cast<float>(v[e]));
          const half_t t2 = static_cast<half_t>(static_cast<float>(sn[pos * rot + j]) * static_cast<float>(partner));
          v[e] = static_cast<half_t>(static_cast<float>(t1) + static_cast<float>(t2));
        }
      }
      raw = __builtin_bit_cast(u32x4, v);
    }
    *reinterpret_cast<u32x4*>(out + row * d + j0) = raw;
  }
}

// The same for the model's shape (20 of the d elements rotated): every thread takes one 16-byte piece, and a
// piece of the rotated part finds its partners with one or two more 16-byte loads at the elements' alignment
// (piece 0: elements 10..17 negated; piece 1: 18, 19 negated, then 0..5; piece 2: 6..9) and its part of the
// tables' row with 8-byte loads (a table row is 40 bytes).
// I = the index type: 32-bit while the piece count fits (shorter index arithmetic; the time is the same at n = 4096).
template <typename I>
__global__ void __launch_bounds__(kBlock) rotary20_kernel(const half_t* __restrict__ A, const half_t* __restrict__ cs,
                                                          const half_t* __restrict__ sn, half_t* __restrict__ out,
                                                          I pieces, I heads, I d, int64_t pos0) {
#pragma clang fp contract(off)
  typedef u32x4 __attribute__((aligned(2))) u32x4_a2;
  const I per_row = d >> 3;
  const I step = static_cast<I>(gridDim.x) * kBlock;
  for (I t = static_cast<I>(blockIdx.x) * kBlock + threadIdx.x; t < pieces; t += step) {
    const I row = t / per_row, v = t - row * per_row;
    const half_t* a = A + static_cast<int64_t>(row) * d;
    u32x4 raw = *reinterpret_cast<const u32x4*>(a + 8 * v);
    if (v < 3) {
      const f16x8 x = __builtin_bit_cast(f16x8, raw);
      // partners: p[e] for element j = 8 v + e
      const f16x8 far = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4_a2*>(a + (v == 0 ? 10 : v == 1 ? 18 : 6)));
      const f16x8 low = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(a));   // elements 0..7 (piece 1 needs 0..5)
      const int64_t pos = pos0 + row / heads;
      const half_t* cr = cs + pos * 20 + 8 * v;
      const half_t* sr = sn + pos * 20 + 8 * v;
      f16x4 c0 = __builtin_bit_cast(f16x4, *reinterpret_cast<const u32x2*>(cr)), s0 = __builtin_bit_cast(f16x4, *reinterpret_cast<const u32x2*>(sr));
      f16x4 c1 = {}, s1 = {};
      if (v < 2) {  // (piece 2 holds the tables' elements 16..19 only)
        c1 = __builtin_bit_cast(f16x4, *reinterpret_cast<const u32x2*>(cr + 4));
        s1 = __builtin_bit_cast(f16x4, *reinterpret_cast<const u32x2*>(sr + 4));
      }
      f16x8 r = x;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (v == 2 && e >= 4) continue;  // elements 20..23 are not rotated
        half_t partner;
        if (v == 0) partner = static_cast<half_t>(static_cast<float>(far[e]) * -1.f);
        else if (v == 1) partner = e < 2 ? static_cast<half_t>(static_cast<float>(far[e]) * -1.f) : low[e >= 2 ? e - 2 : 0];
        else partner = far[e];
        const half_t cj = e < 4 ? c0[e] : c1[e - 4 < 0 ? 0 : e - 4], sj = e < 4 ? s0[e] : s1[e - 4 < 0 ? 0 : e - 4];
        const half_t t1 = static_cast<half_t>(static_cast<float>(cj) * static_cast<float>(x[e]));
        const half_t t2 = static_cast<half_t>(static_cast<float>(sj) * static_cast<float>(partner));
        r[e] = static_cast<half_t>(static_cast<float>(t1) + static_cast<float>(t2));
      }
      raw = __builtin_bit_cast(u32x4, r);
    }
    store_stream(raw, reinterpret_cast<u32x4*>(out + static_cast<int64_t>(row) * d + 8 * v));
    if (pieces - t <= step) break;   // (t + step might wrap in 32 bits)
  }
}

// Rotated widths that are a multiple of 16 (the whole head dimension of 64 or 128, or a half or a quarter of it): a
// piece's partners are one whole 16-byte piece of the same row, rot / 2 elements on or back, and its part of the tables'
// rows two aligned 16-byte loads.  A thread per piece, as above (32 heads of 128, all rotated, n = 4096: 50.9 us with
// the kernel for any width, which loads partners and table entries element by element).
template <typename I>
__global__ void __launch_bounds__(kBlock) rotary16_kernel(const half_t* __restrict__ A, const half_t* __restrict__ cs,
                                                          const half_t* __restrict__ sn, half_t* __restrict__ out,
                                                          I pieces, I heads, I per_row, I rot_pieces, int64_t pos0) {
#pragma clang fp contract(off)
  const I step = static_cast<I>(gridDim.x) * kBlock, half_pieces = rot_pieces >> 1;
  for (I t = static_cast<I>(blockIdx.x) * kBlock + threadIdx.x; t < pieces; t += step) {
    const I row = t / per_row, v = t - row * per_row;
    const half_t* a = A + static_cast<int64_t>(row) * per_row * 8;
    u32x4 raw = *reinterpret_cast<const u32x4*>(a + 8 * v);
    if (v < rot_pieces) {
      const bool low = v < half_pieces;
      const f16x8 x = __builtin_bit_cast(f16x8, raw);
      const f16x8 p = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(a + 8 * (low ? v + half_pieces : v - half_pieces)));
      const int64_t tab = (pos0 + row / heads) * (static_cast<int64_t>(rot_pieces) * 8) + 8 * v;
      const f16x8 c = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(cs + tab));
      const f16x8 sj = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(sn + tab));
      f16x8 r;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const half_t partner = low ? static_cast<half_t>(static_cast<float>(p[e]) * -1.f) : p[e];
        const half_t t1 = static_cast<half_t>(static_cast<float>(c[e]) * static_cast<float>(x[e]));
        const half_t t2 = static_cast<half_t>(static_cast<float>(sj[e]) * static_cast<float>(partner));
        r[e] = static_cast<half_t>(static_cast<float>(t1) + static_cast<float>(t2));
      }
      raw = __builtin_bit_cast(u32x4, r);
    }
    store_stream(raw, reinterpret_cast<u32x4*>(out + static_cast<int64_t>(row) * per_row * 8 + 8 * v));
    if (pieces - t <= step) break;   // (t + step might wrap in 32 bits)
  }
}

// Rotated widths that are a multiple of 4 but not of 16 (24 of 96): two neighbouring elements have neighbouring
// partners and table entries, so a rotated piece takes four 4-byte loads of each instead of eight 2-byte ones (all
// inside the rotated part of the row, at 4-byte alignment).
template <typename I>
__global__ void __launch_bounds__(kBlock) rotary4_kernel(const half_t* __restrict__ A, const half_t* __restrict__ cs,
                                                         const half_t* __restrict__ sn, half_t* __restrict__ out,
                                                         I pieces, I heads, I per_row, I rot, int64_t pos0) {
#pragma clang fp contract(off)
  const I step = static_cast<I>(gridDim.x) * kBlock, half_rot = rot >> 1;
  for (I t = static_cast<I>(blockIdx.x) * kBlock + threadIdx.x; t < pieces; t += step) {
    const I row = t / per_row, v = t - row * per_row, j0 = 8 * v;
    const half_t* a = A + static_cast<int64_t>(row) * per_row * 8;
    u32x4 raw = *reinterpret_cast<const u32x4*>(a + j0);
    if (j0 < rot) {
      const half_t* cr = cs + (pos0 + row / heads) * static_cast<int64_t>(rot);
      const half_t* sr = sn + (pos0 + row / heads) * static_cast<int64_t>(rot);
      f16x8 x = __builtin_bit_cast(f16x8, raw);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const I j = j0 + 2 * q;
        if (j < rot) {   // (rot % 4 == 0: a pair is rotated or not as a whole, and lies on one side of rot / 2)
          const bool low = j < half_rot;
          const f16x2 p = __builtin_bit_cast(f16x2, *reinterpret_cast<const uint32_t*>(a + (low ? j + half_rot : j - half_rot)));
          const f16x2 c = __builtin_bit_cast(f16x2, *reinterpret_cast<const uint32_t*>(cr + j));
          const f16x2 sj = __builtin_bit_cast(f16x2, *reinterpret_cast<const uint32_t*>(sr + j));
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            const half_t partner = low ? static_cast<half_t>(static_cast<float>(p[e]) * -1.f) : p[e];
            const half_t t1 = static_cast<half_t>(static_cast<float>(c[e]) * static_cast<float>(x[2 * q + e]));
            const half_t t2 = static_cast<half_t>(static_cast<float>(sj[e]) * static_cast<float>(partner));
            x[2 * q + e] = static_cast<half_t>(static_cast<float>(t1) + static_cast<float>(t2));
          }
        }
      }
      raw = __builtin_bit_cast(u32x4, x);
    }
    store_stream(raw, reinterpret_cast<u32x4*>(out + static_cast<int64_t>(row) * per_row * 8 + j0));
    if (pieces - t <= step) break;   // (t + step might wrap in 32 bits)
  }
}

// The same for rows of 3 .. 64 pieces (the model's have 10) without the partner loads: a wavefront takes whole rows,
// floor(64 / pieces per row) of them, one piece per lane (60 of the model's 64 lanes work), and the three lanes of a
// row that hold the rotated pieces get their partners' words from one another through ds_bpermute -- piece 0 wants
// elements 10..17 (words 1..3 of the next lane, word 0 of the one after), piece 1 elements 18, 19 (word 1 of the next
// lane) and 0..5 (words 0..2 of the lane before), piece 2 elements 6..9 (word 3 two lanes back, word 0 one back).
// The tables' 8 elements come as one 16-byte load (piece 2: elements 12..19, of which it uses the upper four), asked
// for together with the piece.  At n = 4096 (32 heads, d = 80): 9.2 us against 11.5 for the kernel above, which was
// 12.2 before its stores became streaming ones; two or more chunks of rows per pass of a wavefront are slower.
__global__ void __launch_bounds__(kBlock) rotary20_rows_kernel(const half_t* __restrict__ A, const half_t* __restrict__ cs,
                                                               const half_t* __restrict__ sn, half_t* __restrict__ out,
                                                               uint32_t rows, uint32_t heads, uint32_t per_row, int64_t pos0) {
#pragma clang fp contract(off)
  typedef u32x4 __attribute__((aligned(8))) u32x4_a8;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t rows_per_chunk = 64u / per_row;
  const uint32_t rr = lane / per_row, v = lane - rr * per_row;
  const bool lane_used = rr < rows_per_chunk;
  const uint32_t chunks = (rows + rows_per_chunk - 1) / rows_per_chunk;
  const uint32_t waves = gridDim.x * (kBlock / 64);
  // the lanes the partner words come from, as byte addresses for ds_bpermute
  const int from0 = static_cast<int>(((v == 0 ? lane + 2 : lane - 1) & 63u) << 2);
  const int from_next = static_cast<int>(((lane + 1) & 63u) << 2), from_prev = static_cast<int>(((lane - 1) & 63u) << 2);
  const int from2 = v == 0 ? from_next : from_prev;
  const int from3 = v == 0 ? from_next : static_cast<int>(((lane - 2) & 63u) << 2);
  const uint32_t table_at = v < 2 ? 8 * v : 12;
  for (uint32_t c = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); c < chunks; c += waves) {   // (uniform over the wavefront)
    const uint32_t row = c * rows_per_chunk + rr;
    const bool on = lane_used && row < rows;
    const int64_t at = (static_cast<int64_t>(row) * per_row + v) * 8;
    u32x4 raw = {0, 0, 0, 0}, cw = {0, 0, 0, 0}, sw = {0, 0, 0, 0};
    if (on) raw = load_stream(reinterpret_cast<const u32x4*>(A + at));
    if (on && v < 3) {
      const int64_t toff = (pos0 + row / heads) * 20 + table_at;
      cw = *reinterpret_cast<const u32x4_a8*>(cs + toff);
      sw = *reinterpret_cast<const u32x4_a8*>(sn + toff);
    }
    const uint32_t w0 = __builtin_amdgcn_ds_bpermute(from0, static_cast<int>(raw[0]));
    const uint32_t w1n = __builtin_amdgcn_ds_bpermute(from_next, static_cast<int>(raw[1]));
    const uint32_t w1p = __builtin_amdgcn_ds_bpermute(from_prev, static_cast<int>(raw[1]));
    const uint32_t w2 = __builtin_amdgcn_ds_bpermute(from2, static_cast<int>(raw[2]));
    const uint32_t w3 = __builtin_amdgcn_ds_bpermute(from3, static_cast<int>(raw[3]));
    if (on && v < 3) {
      const f16x8 x = __builtin_bit_cast(f16x8, raw);
      // the partners of the piece's 8 elements, and how many of the leading ones are negated
      const u32x4 pw = v == 0 ? u32x4{w1n, w2, w3, w0} : v == 1 ? u32x4{w1n, w0, w1p, w2} : u32x4{w3, w0, 0u, 0u};
      const f16x8 far = __builtin_bit_cast(f16x8, pw);
      const int negated = v == 0 ? 8 : v == 1 ? 2 : 0;
      const f16x8 c8 = __builtin_bit_cast(f16x8, cw), s8 = __builtin_bit_cast(f16x8, sw);
      f16x8 r = x;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (e >= 4 && v == 2) continue;   // elements 20..23 are not rotated
        const half_t partner = e < negated ? static_cast<half_t>(static_cast<float>(far[e]) * -1.f) : far[e];
        const half_t cj = v == 2 ? c8[(e + 4) & 7] : c8[e], sj = v == 2 ? s8[(e + 4) & 7] : s8[e];
        const half_t t1 = static_cast<half_t>(static_cast<float>(cj) * static_cast<float>(x[e]));
        const half_t t2 = static_cast<half_t>(static_cast<float>(sj) * static_cast<float>(partner));
        r[e] = static_cast<half_t>(static_cast<float>(t1) + static_cast<float>(t2));
      }
      raw = __builtin_bit_cast(u32x4, r);
    }
    if (on) store_stream(raw, reinterpret_cast<u32x4*>(out + at));
  }
}

// The attention mask of the prefill and decode graphs in one pass: fused_min_max_triu_te_broadcast_to
// (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py:642-658: [n, n], -65504 above the diagonal, 65504 elsewhere),
// extended to m >= n key positions by extend_te (:68-80: 65504 for the m - n positions already cached, the
// triangle after them) -- and, with n = 1, full (:83-93).  out[i, j] = (j - (m - n) > i) ? -65504 : 65504.
// A thread writes 8 consecutive elements of the flat [n * m] array (16-byte stores whatever m is).
// I = the index type: 32-bit while n * m fits.
template <typename I>
__global__ void __launch_bounds__(kBlock) attn_mask_kernel(half_t* __restrict__ out, I n, I m, I total) {
  const I shift = m - n;
  const I step = static_cast<I>(gridDim.x) * kBlock * 8;
  for (I t = (static_cast<I>(blockIdx.x) * kBlock + threadIdx.x) * 8; t < total; t += step) {
    I i = t / m, jj = t - i * m;
    f16x8 v;
    if (m - jj >= 8) {   // the 8 elements lie in one row: element e is above the diagonal when e > i + shift - jj
      const int64_t last_kept = static_cast<int64_t>(i) + static_cast<int64_t>(shift) - static_cast<int64_t>(jj);
      const int keep = last_kept < 0 ? 0 : last_kept >= 7 ? 8 : static_cast<int>(last_kept) + 1;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = static_cast<half_t>(e < keep ? 65504.f : -65504.f);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        v[e] = static_cast<half_t>(jj > i + shift ? -65504.f : 65504.f);
        if (++jj == m) {
          jj = 0;
          ++i;
        }
      }
    }
    if (total - t >= 8) {
      store_stream(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4*>(out + t));
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (e < total - t) out[t + e] = v[e];
    }
    if (total - t <= step) break;   // t + step would pass total (and, in 32 bits, might wrap)
  }
}

// transpose6 / transpose7 (before_dl.py:1177-1203): [a, b, d] -> [b, a, d], rows of d elements moved whole
// (queries, keys and values between the projection's [n, heads, d] and attention's [heads, n, d]).  A thread
// moves one 16-byte piece; the stores are the contiguous side.
// I = the index type: 32-bit while the piece count fits.
template <typename I>
__global__ void __launch_bounds__(kBlock) swap_axes_kernel(const u32x4* __restrict__ A, u32x4* __restrict__ out, I a, I b,
                                                           I per_row, I total) {
  const I step = static_cast<I>(gridDim.x) * kBlock;
  for (I t = static_cast<I>(blockIdx.x) * kBlock + threadIdx.x; t < total; t += step) {
    const I r = t / per_row, p = t - r * per_row;   // output row r = ib * a + ia
    const I ib = r / a, ia = r - ib * a;
    store_stream(A[(static_cast<int64_t>(ia) * b + ib) * per_row + p], out + t);
    if (total - t <= step) break;   // (t + step might wrap in 32 bits)
  }
}

// The same for rows of up to 1 KiB (the model's are 160 bytes): a workgroup moves the tile of kSwapA consecutive ia by
// kSwapB consecutive ib in the order of the output, so that what it writes (kSwapB runs of kSwapA rows) and what it
// reads (kSwapA runs of kSwapB rows) are both runs of whole 128-byte lines; addresses are a base per workgroup plus
// 32-bit offsets, and a thread loads up to four pieces before it stores them.  At a = 4096, b = 32, d = 80: 8.8 us
// against 9.6 for the kernel above (10.7 before its stores became streaming ones); at a = 1024 4.0 either way.
constexpr int kSwapA = 4, kSwapB = 8;
__global__ void __launch_bounds__(kBlock) swap_axes_tile_kernel(const u32x4* __restrict__ A, u32x4* __restrict__ out, int64_t a,
                                                                int64_t b, uint32_t per_row, uint32_t b_groups) {
  const uint32_t ig = blockIdx.x / b_groups, bg = blockIdx.x - ig * b_groups;
  const int64_t i0 = static_cast<int64_t>(ig) * kSwapA, b0 = static_cast<int64_t>(bg) * kSwapB;
  const uint32_t ni = a - i0 < kSwapA ? static_cast<uint32_t>(a - i0) : kSwapA;
  const uint32_t nb = b - b0 < kSwapB ? static_cast<uint32_t>(b - b0) : kSwapB;
  const uint32_t run = ni * per_row, tile = nb * run;   // pieces of one output run, of the tile
  const u32x4* src = A + (i0 * b + b0) * per_row;
  u32x4* dst = out + (b0 * a + i0) * per_row;
  const uint32_t in_row = static_cast<uint32_t>(b) * per_row, out_plane = static_cast<uint32_t>(a) * per_row;   // (the host checks that they fit)
  for (uint32_t u0 = threadIdx.x; u0 < tile; u0 += 4 * kBlock) {
    u32x4 v[4];
    uint32_t to[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t u = u0 + k * kBlock;
      if (u < tile) {
        const uint32_t jb = u / run, rem = u - jb * run;
        const uint32_t ii = rem / per_row, p = rem - ii * per_row;
        v[k] = src[ii * in_row + jb * per_row + p];
        to[k] = jb * out_plane + rem;
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (u0 + k * kBlock < tile) store_stream(v[k], dst + to[k]);
  }
}

// split (before_dl.py:1099-1125) and fused_reshape7_split1 (:661-688): the fused query / key / value projection
// A[rows, 3 d] (rows = positions x heads, d = 80) cut into three [rows, d] buffers, section s = columns
// [s d, (s + 1) d).  T is a 16-byte piece (d % 8 == 0, aligned buffers) or one element; the loads run
// through A in order, the stores are runs of d elements.
template <typename T, typename I>
__global__ void __launch_bounds__(kBlock) split3_kernel(const T* __restrict__ A, T* __restrict__ o0, T* __restrict__ o1,
                                                        T* __restrict__ o2, I per_sec, I total) {
  const I step = static_cast<I>(gridDim.x) * kBlock;
  for (I t = static_cast<I>(blockIdx.x) * kBlock + threadIdx.x; t < total; t += step) {
    const I r = t / (3 * per_sec), c = t - r * (3 * per_sec);
    const I sec = c / per_sec, j = c - sec * per_sec;
    T* o = sec == 0 ? o0 : sec == 1 ? o1 : o2;
    store_stream(A[t], o + static_cast<int64_t>(r) * per_sec + j);
    if (total - t <= step) break;   // (t + step might wrap in 32 bits)
  }
}

// The same for sections of up to 1 KiB (the model's are 160 bytes), 16-byte pieces: a workgroup takes kSplitRows rows
// of A and walks them section by section, so that its stores are three runs of kSplitRows x d elements, whole
// 128-byte lines; the lines of A are read by the three walks within the one workgroup.  Addresses are a base per
// workgroup plus 32-bit offsets, and a thread loads up to four pieces before it stores them.  At 131072 rows, d = 80:
// 21.8 us against 23.1 for the kernel above (24.4 before its stores became streaming ones), at 32768 rows 7.1 / 7.7.
constexpr int kSplitRows = 8;
__global__ void __launch_bounds__(kBlock) split3_tile_kernel(const u32x4* __restrict__ A, u32x4* __restrict__ o0, u32x4* __restrict__ o1,
                                                             u32x4* __restrict__ o2, int64_t rows, uint32_t per_sec) {
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * kSplitRows;
  const uint32_t nr = rows - r0 < kSplitRows ? static_cast<uint32_t>(rows - r0) : kSplitRows;
  const uint32_t run = nr * per_sec, tile = 3 * run;
  const u32x4* src = A + r0 * 3 * per_sec;
  for (uint32_t u0 = threadIdx.x; u0 < tile; u0 += 4 * kBlock) {
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t u = u0 + k * kBlock;
      if (u < tile) {
        const uint32_t sec = u / run, rem = u - sec * run;
        const uint32_t rr = rem / per_sec, j = rem - rr * per_sec;
        v[k] = src[(rr * 3 + sec) * per_sec + j];
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t u = u0 + k * kBlock;
      if (u < tile) {
        const uint32_t sec = u / run, rem = u - sec * run;
        u32x4* o = sec == 0 ? o0 : sec == 1 ? o1 : o2;
        store_stream(v[k], o + r0 * per_sec + rem);
      }
    }
  }
}

// divide2 (before_dl.py:57-65): T_divide[k] = A[k] / B[()], fp32, the divisor one device scalar (the sampling
// temperature).  The division is the correctly rounded one (no reciprocal shortcut): the result is bit-exact.
__global__ void __launch_bounds__(kBlock) divide_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                            float* __restrict__ out, int64_t count, bool vec) {
  const float b = *B;
  const int64_t step = static_cast<int64_t>(gridDim.x) * kBlock;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (vec) {
    const int64_t nvec = count >> 2;
    for (int64_t t = t0; t < nvec; t += step) {
      f32x4 v = reinterpret_cast<const f32x4*>(A)[t];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = v[e] / b;
      reinterpret_cast<f32x4*>(out)[t] = v;
    }
    for (int64_t k = (nvec << 2) + t0; k < count; k += step) out[k] = A[k] / b;
  } else {
    for (int64_t k = t0; k < count; k += step) out[k] = A[k] / b;
  }
}

}  // namespace

// grid = min(ceil(nvec / (256 * unroll)), grid_cap): the reference's
// ElementwiseConfigEmiter.get_num_blocks (python/dtas/policy/elementwise_config_emiter.py:35-54)
// with the per-thread unroll folded into the tile.
int describe_eltwise(int op, int64_t count, const dtas_config& cfg, int64_t la[7]) {
  EltInfo e;
  if (!elt_info(op, &e)) return fail("elementwise: unknown op %d", op);
  if (cfg.block != kBlock) return fail("%s: block must be %d threads, got %d", e.name, kBlock, cfg.block);
  if (cfg.variant != DTAS_ELT_VECTOR && cfg.variant != DTAS_ELT_SCALAR)
    return fail("%s: unknown variant %d", e.name, cfg.variant);
  if (cfg.unroll != 1 && cfg.unroll != 2 && cfg.unroll != 4 && cfg.unroll != 8)
    return fail("%s: unroll %d is not one of 1, 2, 4, 8", e.name, cfg.unroll);
  const int narrow = e.in_bytes < e.out_bytes ? e.in_bytes : e.out_bytes;
  const int vec = cfg.variant == DTAS_ELT_SCALAR ? 1 : cfg.vec;
  if (cfg.variant == DTAS_ELT_VECTOR && !(vec == 16 / narrow || vec == 8 / narrow || vec == 4 / narrow) )
    return fail("%s: vector width %d not in {%d, %d, %d}", e.name, vec, 16 / narrow, 8 / narrow, 4 / narrow);
  if (vec < 1) return fail("%s: vector width %d", e.name, vec);
  const int64_t nvec = count / vec;
  int64_t grid = ceil_div(nvec > 0 ? nvec : 1, static_cast<int64_t>(kBlock) * cfg.unroll);
  if (cfg.grid_cap > 0 && grid > cfg.grid_cap) grid = cfg.grid_cap;
  if (grid > 0x7fffffff) grid = 0x7fffffff;
  if (grid < 1) grid = 1;
  for (int i = 0; i < 7; ++i) la[i] = 0;
  la[0] = grid; la[1] = 1; la[2] = 1; la[3] = kBlock;
  return 0;
}

}  // namespace dtas

extern "C" {
int dtas_add_f16(const void* A, const void* B, void* T, int64_t n, int64_t H, const dtas_config* cfg, void* stream) {
  return dtas::run_eltwise(DTAS_OP_ADD_F16, A, B, T, n, H, cfg, stream);
}
int dtas_add_f32(const void* A, const void* B, void* T, int64_t n, int64_t H, const dtas_config* cfg, void* stream) {
  return dtas::run_eltwise(DTAS_OP_ADD_F32, A, B, T, n, H, cfg, stream);
}
int dtas_add_i8(const void* A, const void* B, void* T, int64_t n, int64_t H, const dtas_config* cfg, void* stream) {
  return dtas::run_eltwise(DTAS_OP_ADD_I8, A, B, T, n, H, cfg, stream);
}
int dtas_copy_f16(const void* A, void* B, int64_t n, int64_t H, const dtas_config* cfg, void* stream) {
  return dtas::run_eltwise(DTAS_OP_COPY_F16, A, nullptr, B, n, H, cfg, stream);
}
int dtas_copy_f32(const void* A, void* B, int64_t n, int64_t H, const dtas_config* cfg, void* stream) {
  return dtas::run_eltwise(DTAS_OP_COPY_F32, A, nullptr, B, n, H, cfg, stream);
}
int dtas_copy_i8(const void* A, void* B, int64_t n, int64_t H, const dtas_config* cfg, void* stream) {
  return dtas::run_eltwise(DTAS_OP_COPY_I8, A, nullptr, B, n, H, cfg, stream);
}
int dtas_cast_f16_f32(const void* A, void* C, int64_t n, int64_t H, const dtas_config* cfg, void* stream) {
  return dtas::run_eltwise(DTAS_OP_CAST_F16_F32, A, nullptr, C, n, H, cfg, stream);
}
int dtas_cast_f32_f16(const void* A, void* C, int64_t n, int64_t H, const dtas_config* cfg, void* stream) {
  return dtas::run_eltwise(DTAS_OP_CAST_F32_F16, A, nullptr, C, n, H, cfg, stream);
}
int dtas_take_f16(const void* A, const void* ids, void* out, int64_t n, int64_t V, int64_t H, const dtas_config* user,
                  void* stream) {
  using namespace dtas;
  clear_error();
  if (n < 0 || V < 0 || H < 0) return fail("take: negative extent n=%lld V=%lld H=%lld", (long long)n, (long long)V, (long long)H);
  if (H != 0 && (n > INT64_MAX / 4 / H || V > INT64_MAX / 4 / H)) return fail("take: extents overflow");
  if (n == 0 || H == 0) return 0;
  if (V == 0) return fail("take: an empty table has no row to take");
  if (!A || !ids || !out) return fail("take: NULL buffer");
  if (overlaps(out, n * H * 2, A, V * H * 2) || overlaps(out, n * H * 2, ids, n * 4)) return fail("take: output overlaps an input");
  dtas_config cfg = user ? *user : dtas_config{DTAS_ELT_VECTOR, kBlock, 8, 1, {0, 0, 0}, 1, 0};
  if (cfg.block != kBlock) return fail("take: the kernels use %d threads, got %d", kBlock, cfg.block);
  if (cfg.vec != 8 && cfg.vec != 1) return fail("take: vector width must be 8 (128-bit accesses) or 1, got %d", cfg.vec);
  if (cfg.vec == 8 && !(H % 8 == 0 && aligned(A, 16) && aligned(out, 16))) cfg.vec = 1;
  const int64_t items = cfg.vec == 8 ? n * (H / 8) : n * H;
  int64_t grid = ceil_div(items, kBlock);
  const int64_t cap = cfg.grid_cap > 0 ? cfg.grid_cap : kMaxGrid;
  grid = grid > cap ? cap : grid;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (cfg.vec == 8)
    hipLaunchKernelGGL(take_f16_kernel, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, s, static_cast<const u32x4*>(A),
                       static_cast<const int*>(ids), static_cast<u32x4*>(out), items, H / 8, V);
  else
    hipLaunchKernelGGL(take_f16_scalar_kernel, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, s, static_cast<const half_t*>(A),
                       static_cast<const int*>(ids), static_cast<half_t*>(out), items, H, V);
  return check_launch("take");
}
int dtas_rotary_f16(const void* A, const void* cos_t, const void* sin_t, void* out, int64_t n, int64_t m, int64_t heads,
                    int64_t d, int64_t rot, int64_t max_pos, const dtas_config* user, void* stream) {
  using namespace dtas;
  clear_error();
  if (n < 0 || m < 0 || heads < 0 || d < 0 || rot < 0 || max_pos < 0)
    return fail("rotary: negative extent n=%lld m=%lld heads=%lld d=%lld rot=%lld", (long long)n, (long long)m, (long long)heads, (long long)d, (long long)rot);
  if (rot > d || rot % 2 != 0) return fail("rotary: the rotated part (%lld) must be even and at most d (%lld)", (long long)rot, (long long)d);
  if (d % 8 != 0) return fail("rotary: the head dimension must be a multiple of 8 (d=%lld)", (long long)d);
  if (n == 0 || heads == 0 || d == 0) return 0;
  if (heads > INT64_MAX / 4 / d || n > INT64_MAX / 4 / (heads * d)) return fail("rotary: extents overflow");
  // positions m - n .. m - 1 of the tables
  if (m < n || m > max_pos) return fail("rotary: positions %lld .. %lld lie outside the tables' %lld rows", (long long)(m - n), (long long)(m - 1), (long long)max_pos);
  if (!A || !out || (rot > 0 && (!cos_t || !sin_t))) return fail("rotary: NULL buffer");
  if (!aligned(A, 16) || !aligned(out, 16)) return fail("rotary: A and the output must be 16-byte aligned");
  const int64_t bytes = n * heads * d * 2;
  if (overlaps(out, bytes, A, bytes) || overlaps(out, bytes, cos_t, max_pos * rot * 2) || overlaps(out, bytes, sin_t, max_pos * rot * 2))
    return fail("rotary: output overlaps an input");
  // cfg.unroll picks the kernel: 0 (built in) whole rows per wavefront where the shape has that form, 1 a piece per
  // thread with its partners loaded (the model's 20 of d, or a rotated width that is a multiple of 16), 2 the kernel for
  // any rotated width
  dtas_config cfg = user ? *user : dtas_config{DTAS_ELT_VECTOR, kBlock, 8, 0, {0, 0, 0}, 1, 0};
  if (cfg.block != kBlock || cfg.vec != 8) return fail("rotary: the kernel uses %d threads and 8 elements per thread", kBlock);
  const int64_t cap = cfg.grid_cap > 0 ? cfg.grid_cap : kMaxGrid;
  if (rot == 20 && d >= 32 && cfg.unroll <= 1 && aligned(cos_t, 8) && aligned(sin_t, 8)) {  // the model's shape
    const int64_t pieces20 = n * heads * (d / 8);
    int64_t grid = ceil_div(pieces20, kBlock);
    grid = grid > cap ? cap : grid;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half_t* a = static_cast<const half_t*>(A);
    const half_t* c = static_cast<const half_t*>(cos_t);
    const half_t* sn = static_cast<const half_t*>(sin_t);
    if (d <= 512 && cfg.unroll == 0 && n * heads < (int64_t{1} << 31)) {   // rows of up to 64 pieces: whole rows per wavefront
      const int64_t rows = n * heads, per_wave = 64 / (d / 8);
      int64_t g = ceil_div(ceil_div(rows, per_wave), kBlock / 64);
      g = g > cap ? cap : g;
      hipLaunchKernelGGL(rotary20_rows_kernel, dim3(static_cast<unsigned>(g)), dim3(kBlock), 0, st, a, c, sn, static_cast<half_t*>(out),
                         static_cast<uint32_t>(rows), static_cast<uint32_t>(heads), static_cast<uint32_t>(d / 8), m - n);
      return check_launch("rotary");
    }
    if (pieces20 < (int64_t{1} << 31) && heads < (int64_t{1} << 31) && d < (int64_t{1} << 31))
      hipLaunchKernelGGL(rotary20_kernel<uint32_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, a, c, sn, static_cast<half_t*>(out),
                         static_cast<uint32_t>(pieces20), static_cast<uint32_t>(heads), static_cast<uint32_t>(d), m - n);
    else
      hipLaunchKernelGGL(rotary20_kernel<int64_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, a, c, sn, static_cast<half_t*>(out),
                         pieces20, heads, d, m - n);
    return check_launch("rotary");
  }
  const int64_t pieces = n * heads * (d / 8);
  int64_t grid = ceil_div(pieces, kBlock);
  grid = grid > cap ? cap : grid;
  if (rot > 0 && rot % 16 == 0 && cfg.unroll <= 1 && aligned(cos_t, 16) && aligned(sin_t, 16)) {  // partners and table entries in whole pieces
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half_t* a = static_cast<const half_t*>(A);
    const half_t* c = static_cast<const half_t*>(cos_t);
    const half_t* sn = static_cast<const half_t*>(sin_t);
    if (pieces < (int64_t{1} << 31) && heads < (int64_t{1} << 31))
      hipLaunchKernelGGL(rotary16_kernel<uint32_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, a, c, sn, static_cast<half_t*>(out),
                         static_cast<uint32_t>(pieces), static_cast<uint32_t>(heads), static_cast<uint32_t>(d / 8), static_cast<uint32_t>(rot / 8), m - n);
    else
      hipLaunchKernelGGL(rotary16_kernel<int64_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, a, c, sn, static_cast<half_t*>(out),
                         pieces, heads, d / 8, rot / 8, m - n);
    return check_launch("rotary");
  }
  if (rot > 0 && rot % 4 == 0 && cfg.unroll <= 1 && aligned(cos_t, 4) && aligned(sin_t, 4)) {  // partners and table entries in pairs
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half_t* a = static_cast<const half_t*>(A);
    const half_t* c = static_cast<const half_t*>(cos_t);
    const half_t* sn = static_cast<const half_t*>(sin_t);
    if (pieces < (int64_t{1} << 31) && heads < (int64_t{1} << 31) && rot < (int64_t{1} << 31))
      hipLaunchKernelGGL(rotary4_kernel<uint32_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, a, c, sn, static_cast<half_t*>(out),
                         static_cast<uint32_t>(pieces), static_cast<uint32_t>(heads), static_cast<uint32_t>(d / 8), static_cast<uint32_t>(rot), m - n);
    else
      hipLaunchKernelGGL(rotary4_kernel<int64_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, a, c, sn, static_cast<half_t*>(out),
                         pieces, heads, d / 8, rot, m - n);
    return check_launch("rotary");
  }
  hipLaunchKernelGGL(rotary_f16_kernel, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                     static_cast<const half_t*>(A), static_cast<const half_t*>(cos_t), static_cast<const half_t*>(sin_t),
                     static_cast<half_t*>(out), pieces, heads, d, rot, m - n);
  return check_launch("rotary");
}
int dtas_attn_mask_f16(void* out, int64_t n, int64_t m, void* stream) {
  using namespace dtas;
  clear_error();
  if (n < 0 || m < 0) return fail("attn_mask: negative extent n=%lld m=%lld", (long long)n, (long long)m);
  if (m < n) return fail("attn_mask: m (%lld key positions) must be at least n (%lld query positions)", (long long)m, (long long)n);
  if (n == 0 || m == 0) return 0;
  if (n > INT64_MAX / 4 / m) return fail("attn_mask: n*m overflows");
  if (!out) return fail("attn_mask: NULL buffer");
  if (!aligned(out, 16)) return fail("attn_mask: the output must be 16-byte aligned");
  int64_t grid = ceil_div(ceil_div(n * m, 8), kBlock);
  grid = grid > kMaxGrid ? kMaxGrid : grid;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n * m + 8 < (int64_t{1} << 31))   // + 8: the last thread's t stays below 2^31 as well
    hipLaunchKernelGGL(attn_mask_kernel<uint32_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, static_cast<half_t*>(out),
                       static_cast<uint32_t>(n), static_cast<uint32_t>(m), static_cast<uint32_t>(n * m));
  else
    hipLaunchKernelGGL(attn_mask_kernel<int64_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, static_cast<half_t*>(out),
                       n, m, n * m);
  return check_launch("attn_mask");
}
int dtas_swap_axes_f16(const void* A, void* out, int64_t a, int64_t b, int64_t d, void* stream) {
  using namespace dtas;
  clear_error();
  if (a < 0 || b < 0 || d < 0) return fail("swap_axes: negative extent a=%lld b=%lld d=%lld", (long long)a, (long long)b, (long long)d);
  if (a == 0 || b == 0 || d == 0) return 0;
  if (d % 8 != 0) return fail("swap_axes: rows must be a multiple of 8 elements (d=%lld)", (long long)d);
  if (a > INT64_MAX / 4 / d || b > INT64_MAX / 4 / (a * d)) return fail("swap_axes: extents overflow");
  if (!A || !out) return fail("swap_axes: NULL buffer");
  if (!aligned(A, 16) || !aligned(out, 16)) return fail("swap_axes: buffers must be 16-byte aligned");
  if (overlaps(out, a * b * d * 2, A, a * b * d * 2)) return fail("swap_axes: output overlaps the input");
  int64_t grid = ceil_div(a * b * (d / 8), kBlock);
  grid = grid > kMaxGrid ? kMaxGrid : grid;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t total = a * b * (d / 8);
  // rows of up to 1 KiB: by tiles of kSwapA x kSwapB rows (a launch holds fewer than 2^32 threads; the kernel's offsets 32 bits)
  const int64_t groups = ceil_div(a, kSwapA) * ceil_div(b, kSwapB);
  if (d <= 512 && a > 1 && b > 1 && groups < (int64_t{1} << 23) && a * (d / 8) < (int64_t{1} << 28) && b * (d / 8) < (int64_t{1} << 28)) {
    hipLaunchKernelGGL(swap_axes_tile_kernel, dim3(static_cast<unsigned>(groups)), dim3(kBlock), 0, st, static_cast<const u32x4*>(A),
                       static_cast<u32x4*>(out), a, b, static_cast<uint32_t>(d / 8), static_cast<uint32_t>(ceil_div(b, kSwapB)));
    return check_launch("swap_axes");
  }
  if (total < (int64_t{1} << 31))
    hipLaunchKernelGGL(swap_axes_kernel<uint32_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, static_cast<const u32x4*>(A),
                       static_cast<u32x4*>(out), static_cast<uint32_t>(a), static_cast<uint32_t>(b), static_cast<uint32_t>(d / 8),
                       static_cast<uint32_t>(total));
  else
    hipLaunchKernelGGL(swap_axes_kernel<int64_t>, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, st, static_cast<const u32x4*>(A),
                       static_cast<u32x4*>(out), a, b, d / 8, total);
  return check_launch("swap_axes");
}
int dtas_split3_f16(const void* A, void* out0, void* out1, void* out2, int64_t rows, int64_t d, void* stream) {
  using namespace dtas;
  clear_error();
  if (rows < 0 || d < 0) return fail("split3: negative extent rows=%lld d=%lld", (long long)rows, (long long)d);
  if (rows == 0 || d == 0) return 0;
  if (rows > INT64_MAX / 8 / d) return fail("split3: rows*d overflows");
  if (!A || !out0 || !out1 || !out2) return fail("split3: NULL buffer");
  void* outs[3] = {out0, out1, out2};
  const int64_t sec_bytes = rows * d * 2;
  for (int i = 0; i < 3; ++i) {
    if (!aligned(outs[i], 2)) return fail("split3: buffers must be 2-byte aligned");
    if (overlaps(outs[i], sec_bytes, A, 3 * sec_bytes)) return fail("split3: an output overlaps the input");
    for (int j = 0; j < i; ++j)
      if (overlaps(outs[i], sec_bytes, outs[j], sec_bytes)) return fail("split3: two outputs overlap");
  }
  if (!aligned(A, 2)) return fail("split3: buffers must be 2-byte aligned");
  const bool vec = d % 8 == 0 && aligned(A, 16) && aligned(out0, 16) && aligned(out1, 16) && aligned(out2, 16);
  const int64_t per_sec = vec ? d / 8 : d;
  int64_t grid = ceil_div(rows * 3 * per_sec, kBlock);
  grid = grid > kMaxGrid ? kMaxGrid : grid;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t total = rows * 3 * per_sec;
  const bool narrow = total < (int64_t{1} << 31);   // 32-bit indices while they fit
  const dim3 g(static_cast<unsigned>(grid)), blk(kBlock);
  if (vec) {
    const u32x4* a = static_cast<const u32x4*>(A);
    u32x4 *p0 = static_cast<u32x4*>(out0), *p1 = static_cast<u32x4*>(out1), *p2 = static_cast<u32x4*>(out2);
    if (d <= 512 && ceil_div(rows, kSplitRows) < (int64_t{1} << 23)) {   // sections of up to 1 KiB: by tiles of rows (a launch holds fewer than 2^32 threads)
      hipLaunchKernelGGL(split3_tile_kernel, dim3(static_cast<unsigned>(ceil_div(rows, kSplitRows))), blk, 0, st, a, p0, p1, p2, rows,
                         static_cast<uint32_t>(per_sec));
      return check_launch("split3");
    }
    if (narrow) hipLaunchKernelGGL((split3_kernel<u32x4, uint32_t>), g, blk, 0, st, a, p0, p1, p2, static_cast<uint32_t>(per_sec), static_cast<uint32_t>(total));
    else hipLaunchKernelGGL((split3_kernel<u32x4, int64_t>), g, blk, 0, st, a, p0, p1, p2, per_sec, total);
  } else {
    const half_t* a = static_cast<const half_t*>(A);
    half_t *p0 = static_cast<half_t*>(out0), *p1 = static_cast<half_t*>(out1), *p2 = static_cast<half_t*>(out2);
    if (narrow) hipLaunchKernelGGL((split3_kernel<half_t, uint32_t>), g, blk, 0, st, a, p0, p1, p2, static_cast<uint32_t>(per_sec), static_cast<uint32_t>(total));
    else hipLaunchKernelGGL((split3_kernel<half_t, int64_t>), g, blk, 0, st, a, p0, p1, p2, per_sec, total);
  }
  return check_launch("split3");
}
int dtas_divide_f32(const void* A, const void* B, void* out, int64_t count, void* stream) {
  using namespace dtas;
  clear_error();
  if (count < 0) return fail("divide: negative extent %lld", (long long)count);
  if (count == 0) return 0;
  if (count > INT64_MAX / 8) return fail("divide: extent overflows");
  if (!A || !B || !out) return fail("divide: NULL buffer");
  if (!aligned(A, 4) || !aligned(B, 4) || !aligned(out, 4)) return fail("divide: buffers must be 4-byte aligned");
  if (overlaps(out, count * 4, A, count * 4) || overlaps(out, count * 4, B, 4)) return fail("divide: output overlaps an input");
  const bool vec = aligned(A, 16) && aligned(out, 16);
  int64_t grid = ceil_div(vec ? ceil_div(count, 4) : count, kBlock);
  grid = grid > int64_t{kNumCU} * 32 ? int64_t{kNumCU} * 32 : grid;
  hipLaunchKernelGGL(divide_f32_kernel, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                     static_cast<const float*>(A), static_cast<const float*>(B), static_cast<float*>(out), count, vec);
  return check_launch("divide");
}
}

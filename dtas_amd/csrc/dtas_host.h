// Host-side helpers shared by the entry points: thread-local error text, argument
// checks, launch bookkeeping.  Internal to libdtas_gfx950.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/dtas_abi.h"

namespace dtas {

// MI355X (gfx950) constants the launch heuristics use.
constexpr int kNumCU = 256;        // compute units
constexpr int kNumXCD = 8;         // accelerator complex dies, each with its own L2
constexpr int kWave = 64;          // lanes per wavefront
constexpr int kLdsBytes = 160 * 1024;

char* error_buffer();  // thread-local, 512 bytes
int fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
inline bool overlaps(const void* a, int64_t na, const void* b, int64_t nb) {
  const char* pa = static_cast<const char*>(a);
  const char* pb = static_cast<const char*>(b);
  return pa < pb + nb && pb < pa + na;
}

// Reports a failed launch (bad configuration, no code object for the device, ...).
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

// Fills the name field the way the reference names bucket kernels:
// "<func>_<var>_<lo>_to_<hi>__kernel" (python/dtas/common/config.py:28-31).
void bucket_kernel_name(char* dst, size_t cap, const char* func, const char* var, int64_t lo, int64_t hi);

// Built-in bucket tables (dispatch.hip).  `n` is the dynamic extent.
struct Bucketed {
  dtas_config cfg;
  int64_t lo, hi;
  int32_t index, row;
};
Bucketed builtin_config(int op, int64_t n, int64_t d0, int64_t d1);

// Per-family launch resolution: validates cfg for the op and computes grid/block/LDS.
int describe_eltwise(int op, int64_t count, const dtas_config& cfg, int64_t launch_args[7]);
int describe_reduction(int op, int64_t rows, int64_t cols, const dtas_config& cfg, int64_t launch_args[7]);
int describe_gemv(int64_t N, int64_t K, const dtas_config& cfg, int64_t launch_args[7]);
int describe_gemm(int64_t M, int64_t N, int64_t K, const dtas_config& cfg, int64_t launch_args[7]);

// Resolves (once per device) the device address of the scratch array behind dtas_gemm_f16_static; *out may be NULL.
int resolve_static_scratch(void** out);

// split_k = 0 on the 8-wavefront 256x256 GEMM tile: how the tiles of a last, partly filled round are shared.
// *unsplit tiles (whole rounds of the chip) get one workgroup each, the rest *nsplit workgroups each (1 = none).
void tail_split_256(int64_t M, int64_t N, int64_t K, int* nsplit, unsigned* unsplit);

}  // namespace dtas

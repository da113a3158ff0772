// Shared device/host helpers for the gfx950 kernels behind include/e2h_quant.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/e2h_quant.h"

namespace e2h {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kWaveSize = 64;

// ---- bfloat16 <-> float32 (bit exact, round to nearest even; NaN stays a quiet NaN) -----------------

__host__ __device__ inline float bf16_to_f32(uint16_t b) {
  uint32_t u = static_cast<uint32_t>(b) << 16;
  return __builtin_bit_cast(float, u);
}

__host__ __device__ inline uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);  // the rounding add would carry a NaN away
  u += 0x7FFFu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

// float32 value rounded to the nearest bfloat16, kept as float32
__host__ __device__ inline float bf16_round(float f) { return bf16_to_f32(f32_to_bf16_rne(f)); }

// ---- option store (set through e2h_set_option) --------------------------------------------------

struct Options {
  int int4_rows_per_wave;  // 0 = heuristic, else 16/32/64
  int int4_k_slices;       // 0 = heuristic, else 1..16 workgroups along K
  int int4_k_groups;       // 0 = heuristic, else 1/2/4 k-groups inside a workgroup
  int int4_col_waves;      // 0 = heuristic, else 1..4 column waves per k-group
  int int8_rows_per_wave;  // 0 = heuristic, else 16/32/64
  int int8_k_groups;       // 0 = heuristic, else 1/2
  int int8_k_slices;       // 0 = heuristic, else 1..16
  int int8_force_generic;  // 1 = always use the generic (bounds-checked) int8 kernel
  int int4_no_xsum;        // 1 = many-row int4 calls compute the group sums of x inside the matmul (no pre-pass)
  int int4_no_gemm32;      // 1 = many-row calls (int4 and int8) stay on the 16x16-tile kernels
  int int4_gemm32_min_rows;  // 0 = by workgroup count, else rows from which the 32x32-tile kernels take over
  int row_tiles;           // 0 = heuristic, else 1/2/4 tiles of 16 activation rows per workgroup (both matmuls)
  int attention_waves;     // 0 = by cache length, else 4 or 8 waves per decode-attention workgroup
  int attention_no_mfma;   // 1 = grouped-query decode attention stays on the float32 vector kernel
  int int8_gemm_tile;      // 0 = heuristic, else 128 or 256 rows per workgroup in the many-row int8 matmul
  int int4_gemm_tile;      // 0 = heuristic, else 128 or 256 rows per workgroup in the many-row int4 matmul
  int int8_gemm_waves;     // 256-row tiles: 0 = four waves fed by direct-to-LDS loads, 4 = four waves staging through registers, 8 = eight waves
  int int8_gemm_wave_cols; // register-staged four-wave kernel: 0 or 4 = every wave 256 rows x 64 columns, 2 = 128 rows x 128 columns
  int staged_tiles;        // 0 = heuristic, else weight tiles per workgroup of the staged decode-batch int4 kernel
  int staged_slices;       // 0 = heuristic, else workgroups along K of that kernel (partial epilogue)
  int staged_no_rows64;    // 1 = 33 .. 64 rows with K-slice sums out stay on two 32-row slabs of the staged kernel
};
Options &options();

#if defined(__HIPCC__)
// Buffer resource for raw buffer loads: base pointer + byte size (< 4 GB), no swizzle.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() would also drain every outstanding
// global load (loads and stores share one counter on this architecture), which would empty a register
// prefetch pipeline once per use.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
#endif

// many-row int8 matmul on 32x32 MFMA tiles (e2h_int8_gemm.hip); needs no scratch memory
int int8_gemm32(const uint16_t *x, const int8_t *q, const uint16_t *scales, uint16_t *y, int M, int N, int K, hipStream_t stream);

// streaming int8 matmul (e2h_int8_stream.hip)
int int8_stream_mm(const uint16_t *x, const int8_t *q, const uint16_t *scales, uint16_t *y, int M, int N, int K, void *workspace,
                   int64_t workspace_bytes, hipStream_t stream);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int launch_status() { return hipGetLastError() == hipSuccess ? E2H_OK : E2H_ERR_LAUNCH; }

}  // namespace e2h

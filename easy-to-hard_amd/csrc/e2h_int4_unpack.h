// Shared by the int4 matmul kernels: packed word -> bfloat16 MFMA fragment.
#ifndef E2H_INT4_UNPACK_H
#define E2H_INT4_UNPACK_H
#include "e2h_common.h"

namespace e2h {

// (w >> 4i) & 0x000F000F | 0x43004300: two codes -> the bfloat16 pair (128 + q, 128 + q').  The mask lives
// in an SGPR and the magic in a VGPR so that each pair is one v_and_or_b32 (this ISA's VOP3 encoding takes no
// literal and only one scalar operand); the asm statements only keep the compiler from folding them back
// into literals.
struct UnpackConsts {
  uint32_t mask, magic;
};
__device__ __forceinline__ UnpackConsts unpack_consts() {
  UnpackConsts c;
  asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(c.mask));
  asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(c.magic));
  return c;
}
__device__ __forceinline__ bf16x8_t unpack_word(uint32_t w, const UnpackConsts &c) {
  u32x4_t u;
  u[0] = (w & c.mask) | c.magic;
  u[1] = ((w >> 4) & c.mask) | c.magic;
  u[2] = ((w >> 8) & c.mask) | c.magic;
  u[3] = ((w >> 12) & c.mask) | c.magic;
  return __builtin_bit_cast(bf16x8_t, u);
}

// One pass over x: sums over every (row, quantization group), float32, stored group-major [K/G][stride]
// (defined in e2h_int4_mm.hip; groupsize in {32, 64, 128}).
int launch_x_group_sums(const uint16_t *x, float *out, int M, int K, int stride, int groupsize, hipStream_t stream);

// Many-row int4 matmul on 32x32 MFMA tiles (e2h_int4_gemm.hip); xsum as written by launch_x_group_sums.
int int4_gemm32(const uint16_t *x, const int32_t *packed, const uint16_t *sz, uint16_t *y, const float *xsum, int xsum_stride,
                int M, int N, int K, int groupsize, hipStream_t stream);

}  // namespace e2h
#endif

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

// ---- output of the 32x32-tile kernels ----------------------------------------------------------------------------
// A wave holds RT x CT accumulator tiles of v_mfma_f32_32x32x*: lane (h, n) = column n of a tile, element e = row
// 8 (e / 4) + 4 h + e % 4.  Stored straight from that layout every lane writes 2 bytes per instruction; instead each
// 32-row slab goes through a wave-private LDS tile (32 rows x 32 CT columns, row stride kTileStride bytes) and leaves
// as 16-byte pieces of output rows.  Rounding uses the packed hardware convert (round to nearest even, two values per
// instruction).  kScale: the int8 contract y = bf16(bf16(acc) * scale[column]); otherwise y = bf16(acc).
// pieces (uniform): N % 8 == 0 and y 16-byte aligned, so that every piece is one aligned 16-byte store; otherwise the
// eight values of a piece leave one by one, bounds-checked against N.
typedef float e2h_float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 e2h_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float e2h_f32x16_t __attribute__((ext_vector_type(16)));

template <int CT>
struct TileStore {
  static constexpr int kTileStride = 64 * CT + 16;
  static constexpr int kBytesPerWave = 32 * kTileStride;
};

__device__ __forceinline__ uint32_t pack_bf16x2_rne(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(e2h_float2_t{a, b}, e2h_bf16x2_t));
}

template <int RT, int CT, bool kScale>
__device__ __forceinline__ void store_tiles_via_lds(const e2h_f32x16_t (&acc)[CT][RT], const float (&scale)[CT], uint8_t *tile,
                                                    uint16_t *__restrict__ y, int row0, int col0, int M, int N, int lane,
                                                    bool pieces) {
  constexpr int kTileStride = TileStore<CT>::kTileStride;
  constexpr int kPiecesPerRow = 4 * CT;             // 16-byte pieces per tile row
  constexpr int kRowsPerPass = 64 / kPiecesPerRow;  // tile rows one 64-lane read covers
  const int n = lane & 31, h = lane >> 5;
  const bool odd = n & 1;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        // own = (row e, row e + 1) of column n
        uint32_t own = pack_bf16x2_rne(acc[ct][rt][e], acc[ct][rt][e + 1]);
        if (kScale) {
          const float t0 = __builtin_bit_cast(float, own << 16), t1 = __builtin_bit_cast(float, own & 0xFFFF0000u);
          own = pack_bf16x2_rne(t0 * scale[ct], t1 * scale[ct]);
        }
        // neighbouring lanes (columns n, n ^ 1) trade words: even lanes keep row e of both columns (the low halves),
        // odd lanes row e + 1 (the high halves)
        const uint32_t nbr = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(own), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
        const uint32_t word = __builtin_amdgcn_perm(nbr, own, odd ? 0x03020706u : 0x05040100u);
        const int row = 8 * (e >> 2) + 4 * h + (e & 3) + (odd ? 1 : 0);
        *reinterpret_cast<uint32_t *>(tile + row * kTileStride + (32 * ct + (n & ~1)) * 2) = word;
      }
#pragma unroll
    for (int pass = 0; pass < 32 / kRowsPerPass; ++pass) {
      const int trow = pass * kRowsPerPass + lane / kPiecesPerRow, piece = lane % kPiecesPerRow;
      const u32x4_t v = *reinterpret_cast<const u32x4_t *>(tile + trow * kTileStride + piece * 16);
      const int row = row0 + 32 * rt + trow, col = col0 + 8 * piece;
      if (row < M && col < N) {
        uint16_t *dst = y + static_cast<size_t>(row) * N + col;
        if (pieces) {
          __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t *>(dst));  // streamed: the tiles in L2 are the operands
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (col + j < N) dst[j] = static_cast<uint16_t>(v[j >> 1] >> (16 * (j & 1)));
        }
      }
    }
  }
}

// One pass over x: sums over every (row, quantization group), float32, stored group-major [K/G][stride]
// (defined in e2h_int4_mm.hip; groupsize in {32, 64, 128}).
int launch_x_group_sums(const uint16_t *x, float *out, int M, int K, int stride, int groupsize, hipStream_t stream);

// Many-row int4 matmul on 32x32 MFMA tiles (e2h_int4_gemm.hip); xsum as written by launch_x_group_sums.
int int4_gemm32(const uint16_t *x, const int32_t *packed, const uint16_t *sz, uint16_t *y, const float *xsum, int xsum_stride,
                int M, int N, int K, int groupsize, hipStream_t stream);

// Many-row int4 matmul, 256 x 256 outputs per workgroup, weights dequantized to bfloat16 on the way into the matrix
// cores (e2h_int4_gemm128.hip); needs no scratch memory.
int int4_gemm128(const uint16_t *x, const int32_t *packed, const uint16_t *sz, uint16_t *y, int M, int N, int K, int groupsize,
                 hipStream_t stream);

}  // namespace e2h
#endif

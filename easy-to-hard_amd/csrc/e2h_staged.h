// Activations in matrix-core operand order ("staged"), the input format of the decode-batch int4 kernels
// (e2h_int4_staged.hip), and the device helpers with which the kernels that produce activations write it.
//
// One staged buffer for M rows of K values (K % 128 == 0), Mpad = M rounded up to 16:
//   frag  bf16 [K/32][Mpad][32]  at byte 0.  The 64-byte piece of row m and 32-wide k segment p; inside the piece dword
//         4j + i holds the row's original dword j + 4i of the segment (values k = 32p + 2(j + 4i) and the next one).  The
//         four dwords 4j .. 4j+3 are the k values of the packed int4 weight word (j, p) in its nibble-pair order, so lane
//         (b = j, m) of v_mfma_f32_16x16x32_bf16 fetches its A operand with one 16-byte load and a wave-wide load reads
//         1 KB of consecutive memory.
//   sums  f32  [K/128][Mpad][8]  at byte Mpad * K * 2.  Sum of the activations over each run of 16 consecutive k: a balanced
//         binary tree in index order (the two values of a dword; dwords 0+1, 2+3; those two; the two 8-value halves).  The
//         consumer continues the same tree up to its quantization group, so the group sum does not depend on who wrote it.
//   Rows M .. Mpad-1 may hold anything: no result depends on them.
#ifndef E2H_STAGED_H
#define E2H_STAGED_H
#include "e2h_common.h"

namespace e2h {

struct StagedOut {
  uint32_t *frag;  // null: no staged output
  float *sums;
  int mpad;
};

inline int staged_mpad(int64_t m) { return static_cast<int>((m + 15) / 16 * 16); }
inline int64_t staged_bytes(int64_t m, int64_t k) { return static_cast<int64_t>(staged_mpad(m)) * k * 2 + (k / 128) * staged_mpad(m) * 32; }
inline StagedOut staged_out(void *buf, int64_t m, int64_t k) {
  StagedOut o;
  o.frag = static_cast<uint32_t *>(buf);
  o.mpad = staged_mpad(m);
  o.sums = buf ? reinterpret_cast<float *>(static_cast<uint8_t *>(buf) + static_cast<size_t>(o.mpad) * k * 2) : nullptr;
  return o;
}

// 33 .. 64 rows, K-slice sums out, one pass over the weights (e2h_int4_rows64.hip): number of slices (0: not covered)
// and the launch; same arguments and result layout as the partial-sum entry point of e2h_int4_staged.hip.
int rows64_partial_slices(int64_t m, int64_t n, int64_t k, int groupsize);
int rows64_partials(const void *staged, const int32_t *packed, const uint16_t *sz, float *partials, int64_t m, int64_t n, int64_t k,
                    int groupsize, int slices, hipStream_t stream);

#if defined(__HIPCC__)
// Eight consecutive values of row m (16-byte piece number pc of the row, raw = four dwords of two bfloat16 each).  The
// two lanes that hold pieces 2i and 2i + 1 of a row must be neighbours (lane ^ 1) and must both call.
__device__ __forceinline__ void staged_store_piece(const StagedOut &o, int m, int pc, u32x4_t raw) {
  const int seg = pc >> 2, q = pc & 3;
  uint32_t *dst = o.frag + (static_cast<size_t>(seg) * o.mpad + m) * 16 + q;
  float p[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    dst[4 * i] = raw[i];
    p[i] = __builtin_bit_cast(float, raw[i] << 16) + __builtin_bit_cast(float, raw[i] & 0xFFFF0000u);
  }
  float s = (p[0] + p[1]) + (p[2] + p[3]);
  s += __shfl_xor(s, 1);
  if ((pc & 1) == 0) o.sums[(static_cast<size_t>(pc >> 4) * o.mpad + m) * 8 + ((pc >> 1) & 7)] = s;
}

// One value per lane: sixteen neighbouring lanes (an aligned group) hold the sixteen consecutive values k0 .. k0+15 of
// row m, k0 % 16 == 0, lane l of the group the value k0 + l (v = its bfloat16 bits).  All sixteen lanes must call.
__device__ __forceinline__ void staged_store_run16(const StagedOut &o, int m, int k, uint32_t v) {
  const uint32_t other = static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 1));
  float s = __builtin_bit_cast(float, v << 16) + __builtin_bit_cast(float, other << 16);
  s += __shfl_xor(s, 2);
  s += __shfl_xor(s, 4);
  s += __shfl_xor(s, 8);
  if ((k & 1) == 0) {
    const int d = (k & 31) >> 1;  // dword of the 32-wide segment
    o.frag[(static_cast<size_t>(k >> 5) * o.mpad + m) * 16 + 4 * (d & 3) + (d >> 2)] = v | (other << 16);
  }
  if ((k & 15) == 0) o.sums[(static_cast<size_t>(k >> 7) * o.mpad + m) * 8 + ((k >> 4) & 7)] = s;
}
#endif

}  // namespace e2h
#endif

// int4 group-wise matmul for many rows of x (prefill, scoring), 256 x 256 outputs per workgroup of four waves.
//
// Same contract and data layouts as e2h_int4_mm.hip (torch.ops.aten._weight_int4pack_mm as called by
// linear_forward_int4, reference models/quantize.py:445-453), inner_k_tiles = 8, group size 32 / 64 / 128.
//
// Dequantize-to-bfloat16 form: every weight becomes a bfloat16 value w = bf16( fma(128 + q, s, fma(-136, s, z)) ) on its
// way into the matrix cores (two float32 FMAs: the constant z - 136 s is rounded to float32 once per group, then one FMA
// per weight, then round to nearest even; within one bfloat16 ulp of the single-rounded bf16(s * (q - 8) + z) and equal
// to it whenever z - 136 s is exact in float32), and the products accumulate in float32 -- the arithmetic of the
// kernel the reference calls, up to that ulp.  With 256 accumulator registers per lane there is no
// room for per-group partial sums, and none are needed this way: no pass over x for group sums, no accumulator
// prologue, no scaling of accumulators inside the loop.
//
// Main loop, v_mfma_f32_32x32x16_bf16 (A = activations, 32 rows; B = weights, 32 columns; 16 k per instruction), k in
// natural order: lane L = 32 h + n supplies column n0 + n and the eight k values 16 s + 8 h .. + 7 of step s.
//   Activations are staged per 64-wide k chunk into LDS in fragment order by plain 16-byte copies (double buffered,
//   one LDS barrier per chunk): the fragment of lane (h, m) for step s is x[m][16 s + 8 h .. + 7].
//   Weights never touch LDS.  A packed word (column, j, span p) holds the codes at k = 32 p + 8 i + 2 j + {0, 1} in
//   nibbles i and i + 4 (i = 0 .. 3), and the checkpoint stores the four spans of a 128-wide k block next to each
//   other: the lane loads, per column tile and block, the four 16-byte pieces j = 0 .. 3 of its column (32 registers
//   for both column tiles, the next block's in flight meanwhile) and forms the operand of step s = 2 p' + a as
//   dword j = ((word[j][p'] >> (8 a + 4 h)) & 0x000F000F) | 0x43004300 = the bfloat16 pair (128 + q, 128 + q') of
//   k = 16 s + 8 h + 2 j + {0, 1}.  Every wave owns its 64 columns alone, so no two waves convert the same fragment,
//   and a converted fragment feeds eight MFMAs.
// With one wave per SIMD nothing else covers latencies, so the wave pipelines itself: each MFMA (32 cycles of the
// matrix pipeline) is followed by at most a quarter of the next fragment's conversion and one or two memory
// instructions, fenced in place.
#include "e2h_common.h"
#include "e2h_int4_unpack.h"

namespace e2h {
namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

// One 32-row x 16-k A fragment block in LDS: lane (h, r) at h * kHalfA + 16 r.  A 16-lane group of the staging stores
// covers 2 rows x 8 pieces = 4 steps x 2 halves, 32 bytes each; with these strides (5 * 32 and 128 mod 256) the 16 stores
// fall into 16 different 16-byte bank groups of the 256-byte LDS row, as the fragment reads (256 contiguous bytes per
// 16 lanes) always do.
constexpr int kFragA = 1184, kHalfA = 640;

template <int G>
__global__ __launch_bounds__(256) void int4_gemm128_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ wp,
                                                           const uint32_t *__restrict__ sz, uint16_t *__restrict__ y, int M, int N, int K,
                                                           int n_col_blocks, int cbx) {
  constexpr int RT = 8, CT = 2;        // 32 x 32 tiles per wave: 256 rows x 64 columns
  constexpr int CK = 64;               // k per staged activation chunk
  constexpr int SPC = CK / 16;         // MFMA steps per chunk
  constexpr int NGRP = 128 / G;        // quantization groups per 128-wide weight block
  constexpr int kStageX = RT * SPC * kFragA;
  constexpr int kXPieces = 8;          // 256 rows x 8 pieces of 16 bytes per chunk, 256 threads
  static_assert(G == 32 || G == 64 || G == 128, "group sizes of the packed format up to one weight block");
  __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kStageX];
  static_assert(2 * kStageX >= 4 * TileStore<CT>::kBytesPerWave, "the output tiles reuse the stages");

  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int cb = xcd + 8 * (slot % cbx);
  const int rb = slot / cbx;
  if (cb >= n_col_blocks) return;  // grid padding; uniform, before any barrier

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int row0 = rb * 256;
  const int col0 = cb * 256 + wave * 64;
  const int KT = K / 128;          // weight blocks along K
  const int nchunks = K / CK;      // a multiple of 4: K % 256 == 0

  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(wp, static_cast<uint32_t>(static_cast<size_t>(N) * K / 2));
  const __amdgpu_buffer_rsrc_t sz_rsrc = make_rsrc(sz, static_cast<uint32_t>(static_cast<size_t>(K / G) * N * 4));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));

  f32x16_t acc[CT][RT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[ct][rt][e] = 0.f;

  // ---- activation staging: piece (row, w), k = 8 w .. 8 w + 7, goes to fragment (row tile, step w / 2), lane (w % 2, row % 32)
  const int xr0 = tid >> 3, xw = tid & 7;
  uint32_t xsrc[kXPieces];
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) {
    int row = row0 + xr0 + 32 * i;
    row = row < M ? row : M - 1;
    xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + xw * 8) * 2);
  }
  const int xdst0 = (xw >> 1) * kFragA + (xw & 1) * kHalfA + xr0 * 16;  // pass i covers row tile i

  // ---- weights: byte offset of piece j = 0 of this lane's column inside block 0; (scale, zero) column offset
  uint32_t wlane[CT], szlane[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    int col = col0 + 32 * ct + n;
    col = col < N ? col : N - 1;
    wlane[ct] = static_cast<uint32_t>((static_cast<size_t>(col >> 3) * KT * 32 + (col & 7) * 4) * 16);
    szlane[ct] = static_cast<uint32_t>(col) * 4u;
  }
  struct WSet {
    u32x4_t q[CT][4];       // [column tile][j]: the words of the four 32-wide spans of a block
    uint32_t sz[CT][NGRP];  // raw (scale, zero) pairs of the block's groups
  };
  const int nblocks = KT;
  auto load_w = [&](WSet &w, int blk, int i) {  // i = 0 .. 7
    const int bb = blk < nblocks ? blk : nblocks - 1;
    w.q[i >> 2][i & 3] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wlane[i >> 2] + (i & 3) * 16, static_cast<uint32_t>(bb) * 512u, 0);
  };
  auto load_sz = [&](WSet &w, int blk, int i) {  // i = 0 .. CT * NGRP - 1
    const int bb = blk < nblocks ? blk : nblocks - 1;
    w.sz[i / NGRP][i % NGRP] = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, szlane[i / NGRP], static_cast<uint32_t>(bb * NGRP + i % NGRP) * N * 4u, 0);
  };

  struct Staged {
    u32x4_t p[kXPieces];
  };
  auto load_piece = [&](Staged &r, int ci, int i) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
    r.p[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xsrc[i], static_cast<uint32_t>(cc) * (CK * 2), 0);
  };
  auto store_piece = [&](const Staged &r, int parity, int i) {
    *reinterpret_cast<u32x4_t *>(lds + (parity & 1) * kStageX + xdst0 + i * (SPC * kFragA)) = r.p[i];
  };
  bf16x8_t af[RT];  // fragment rt is re-read for the next step right after its last MFMA of this one
  auto read_a = [&](int parity, int s, int rt) {
    return *reinterpret_cast<const bf16x8_t *>(lds + (parity & 1) * kStageX + h * kHalfA + n * 16 + (rt * SPC + s) * kFragA);
  };

  // ---- conversion of one operand in four parts (dword j each): unpack, two float32 FMAs, one packed round ----------
  const UnpackConsts uc = unpack_consts();
  const uint32_t shift0 = 4u * h, shift1 = 8u + 4u * h;
  uint32_t cv[4];
  float cscale = 0.f, czc = 0.f;
  auto convert_part = [&](const WSet &w, int ct, int sa, int j) {  // sa = step within the block, 0 .. 7
    if (j == 0) {
      const uint32_t szw = w.sz[ct][(16 * sa) / G];
      cscale = __builtin_bit_cast(float, szw << 16);
      czc = __builtin_fmaf(-136.0f, cscale, __builtin_bit_cast(float, szw & 0xFFFF0000u));
    }
    const uint32_t word = w.q[ct][j][sa >> 1];
    const uint32_t v = ((word >> ((sa & 1) ? shift1 : shift0)) & uc.mask) | uc.magic;
    const float lo = __builtin_fmaf(__builtin_bit_cast(float, v << 16), cscale, czc);
    const float hi = __builtin_fmaf(__builtin_bit_cast(float, v & 0xFFFF0000u), cscale, czc);
    cv[j] = pack_bf16x2_rne(lo, hi);
  };
  bf16x8_t wf;  // converted operand of the column tile whose MFMAs come next

  // Slot j = 0 .. 15 of step s of chunk ci (half hf of its weight block), whose register set r holds chunk ci + 1:
  //   j >= 8 (second column tile, the fragment's last use in this step): activation fragment j - 8 of the next step
  //   s < 2, j = 0 .. 3: staging store of piece 4 s + j;  j = 4 .. 7: load of that piece of chunk ci + 3
  //   s = 2 of a block's first half: the eight weight loads (j < 8) and the (scale, zero) loads (j >= 8) of the next block
  // The last step's fragment reads address the next chunk's stage, behind the chunk's only barrier.
  auto slot_op = [&](int ci, Staged &r, WSet &nxt, int hf, int s, int j) {
    const bool last = s + 1 == SPC;
    if (j >= RT) af[j - RT] = last ? read_a(ci + 1, 0, j - RT) : read_a(ci, s + 1, j - RT);
    if (s < 2 && j < 4) store_piece(r, ci + 1, 4 * s + j);
    if (s < 2 && j >= 4 && j < 8) load_piece(r, ci + 3, 4 * s + j - 4);
    if (s == 2 && hf == 0) {
      if (j < 8) load_w(nxt, (ci >> 1) + 1, j);
      if (j >= 8 && j - 8 < CT * NGRP) load_sz(nxt, (ci >> 1) + 1, j - 8);
    }
  };
  auto chunk = [&](int ci, Staged &r, const WSet &cur, WSet &nxt, int hf) {
#pragma unroll
    for (int s = 0; s < SPC; ++s) {
      const int sa = 4 * hf + s;
      if (s + 1 == SPC) lds_barrier();  // staging stores of this chunk visible, every wave done reading this stage
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        // the operand to convert meanwhile: the next column tile's, or the first one of the following step
        const int nct = ct + 1 < CT ? ct + 1 : 0;
        const int nsa = ct + 1 < CT ? sa : sa + 1;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          acc[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[rt], wf, acc[ct][rt], 0, 0, 0);
          if (rt & 1) {
            if (nsa < 8) convert_part(cur, nct, nsa, rt >> 1);
            else convert_part(nxt, nct, 0, rt >> 1);
          }
          slot_op(ci, r, nxt, hf, s, ct * RT + rt);
          __builtin_amdgcn_sched_barrier(0);
        }
        wf = __builtin_bit_cast(bf16x8_t, u32x4_t{cv[0], cv[1], cv[2], cv[3]});
      }
    }
  };

  Staged st[2];
  WSet ws[2];
#pragma unroll
  for (int i = 0; i < 8; ++i) load_w(ws[0], 0, i);
#pragma unroll
  for (int i = 0; i < CT * NGRP; ++i) load_sz(ws[0], 0, i);
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) load_piece(st[0], 0, i);
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) store_piece(st[0], 0, i);
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) load_piece(st[1], 1, i);
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) load_piece(st[0], 2, i);
  lds_barrier();
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) af[rt] = read_a(0, 0, rt);
#pragma unroll
  for (int j = 0; j < 4; ++j) convert_part(ws[0], 0, 0, j);
  wf = __builtin_bit_cast(bf16x8_t, u32x4_t{cv[0], cv[1], cv[2], cv[3]});
  for (int blk = 0; blk < nblocks; blk += 2) {  // two blocks per trip (K % 256 == 0): the register sets are compile-time names
    chunk(2 * blk, st[1], ws[0], ws[1], 0);
    chunk(2 * blk + 1, st[0], ws[0], ws[1], 1);
    chunk(2 * blk + 2, st[1], ws[1], ws[0], 0);
    chunk(2 * blk + 3, st[0], ws[1], ws[0], 1);
  }

  // ---- store: lane (h, n) holds column col0 + 32 ct + n, rows 8 (e / 4) + 4 h + e % 4 of each tile -----------------
  lds_barrier();  // the staging stages are dead from here on
  const float no_scale[CT] = {};
  store_tiles_via_lds<RT, CT, false>(acc, no_scale, lds + wave * TileStore<CT>::kBytesPerWave, y, row0, col0, M, N, lane,
                                    (N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0);
}

}  // namespace

int int4_gemm128(const uint16_t *x, const int32_t *packed, const uint16_t *sz, uint16_t *y, int M, int N, int K, int groupsize,
                 hipStream_t stream) {
  if (K % 256 != 0 || N % 8 != 0) return E2H_ERR_BAD_SHAPE;  // the loop takes two 128-wide weight blocks per trip
  const int n_col_blocks = (N + 255) / 256, n_row_blocks = (M + 255) / 256;
  const int cbx = (n_col_blocks + 7) / 8;
  const long long wgs = 8LL * cbx * n_row_blocks;
  if (wgs > 0x7FFFFFFFLL) return E2H_ERR_BAD_SHAPE;
  dim3 grid(static_cast<unsigned>(wgs)), block(256);
  const uint32_t *w = reinterpret_cast<const uint32_t *>(packed);
  const uint32_t *s = reinterpret_cast<const uint32_t *>(sz);
  switch (groupsize) {
    case 32: hipLaunchKernelGGL(int4_gemm128_kernel<32>, grid, block, 0, stream, x, w, s, y, M, N, K, n_col_blocks, cbx); break;
    case 64: hipLaunchKernelGGL(int4_gemm128_kernel<64>, grid, block, 0, stream, x, w, s, y, M, N, K, n_col_blocks, cbx); break;
    case 128: hipLaunchKernelGGL(int4_gemm128_kernel<128>, grid, block, 0, stream, x, w, s, y, M, N, K, n_col_blocks, cbx); break;
    default: return E2H_ERR_BAD_GROUPSIZE;
  }
  return launch_status();
}

}  // namespace e2h

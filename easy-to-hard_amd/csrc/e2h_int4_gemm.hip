// int4 group-wise matmul for many rows of x (prefill, scoring): MFMA-bound, 32x32 tiles.
//
// Same contract and data layouts as e2h_int4_mm.hip (torch.ops.aten._weight_int4pack_mm as called by
// linear_forward_int4, reference models/quantize.py:445-453), inner_k_tiles = 8, group size 32 / 64 / 128.
//
//   y[m,n] = sum_g  s[g,n] * sum_{k in g} x[m,k] * (128 + q[n,k])  +  sum_g (z[g,n] - 136 s[g,n]) * X[m,g]
//
// with X[m,g] = sum_{k in g} x[m,k] taken from a pre-pass (launch_x_group_sums).  The second sum is a small float32
// matmul over the groups; it initialises the accumulators through v_mfma_f32_32x32x2_f32 (two groups per
// instruction) before the main loop, so the loop itself carries no zero-point work at all.
//
// Main loop, v_mfma_f32_32x32x16_bf16 (A = activations, 32 rows; B = weights, 32 columns; 16 k per instruction):
// lane L = 32*h + n supplies column n0 + n and k-half h.  A packed word holds 8 codes of one column at
// k0 + {2j, 2j+1, 2j+8, 2j+9, 2j+16, ...} (j = 0..3); the lane loads the words with j = h (first 16-byte load)
// and j = 2 + h (second), four 32-wide k spans p each.  Step (p, jp) multiplies the words (j = 2 jp + h, p) with
// the activation fragment gathered in the same k order, so weights are never shuffled: one word is one B operand.
// A workgroup of WR x WC waves owns 64 WR rows x 64 WC columns (each wave 64 x 64 = 2 x 2 tiles, 64 accumulator
// registers).  Activations and packed weights are both staged per 128-wide k chunk into LDS in fragment order (double
// buffered, one LDS barrier per chunk): the global loads then cover whole contiguous 512-byte weight blocks and whole
// activation rows, every A fragment read feeds two column tiles and every unpacked word two row tiles.
//
// Workgroup -> tile mapping: workgroup w runs on XCD w % 8; each XCD owns the column blocks cb = xcd (mod 8) and
// walks them for one row block before moving to the next, so its L2 keeps that slice of the weights.
#include "e2h_common.h"
#include "e2h_int4_unpack.h"

namespace e2h {
namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kChunkK = 128;
constexpr int kFragB = 1024 + 32;                   // one 32-row x 16-k A fragment block in LDS (64 lanes x 16 B) + skew
constexpr int kRT = 2, kCT = 2;                     // 32x32 tiles per wave: rows x columns

template <int G, int WR, int WC>
__global__ __launch_bounds__(64 * WR * WC) void int4_gemm32_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ wp,
                                                                   const uint32_t *__restrict__ sz, uint16_t *__restrict__ y,
                                                                   const float *__restrict__ xsum, int xsum_stride, int M, int N, int K,
                                                                   int n_col_blocks, int cbx) {
  constexpr int NGRP = kChunkK / G;   // groups per chunk
  constexpr int SPG = G / 16;         // MFMA steps per group
  constexpr int kThreads = 64 * WR * WC;
  constexpr int kRows = 64 * WR, kCols = 64 * WC;
  constexpr int kStageX = (2 * WR) * 8 * kFragB;      // kRows x 128 k of activations, 8 fragments per 32-row tile
  constexpr int kStageW = (2 * WC) * 2 * kFragB;      // kCols x 128 k of packed weights, 2 fragments (j pairs) per 32-column tile
  constexpr int kXRowsPerPass = kThreads / 16;        // 16 pieces of 16 bytes per activation row
  constexpr int kXPieces = kRows / kXRowsPerPass;
  constexpr int kWTilesPerPass = kThreads / 32;       // 32 pieces of 16 bytes per 8-column weight block
  constexpr int kWPieces = (kCols / 8) / kWTilesPerPass;
  static_assert(kXRowsPerPass % 32 == 0 && kWTilesPerPass % 4 == 0, "staging passes cover whole 32-wide tiles");
  __shared__ __attribute__((aligned(16))) uint8_t lds[2 * (kStageX + kStageW)];
  uint8_t *const lds_w = lds + 2 * kStageX;

  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int cb = xcd + 8 * (slot % cbx);
  const int rb = slot / cbx;
  if (cb >= n_col_blocks) return;  // grid padding; uniform, before any barrier

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave / WC, wc = wave % WC;
  const int n = lane & 31, h = lane >> 5;
  const int row0 = rb * kRows + wr * 64;
  const int col0 = cb * kCols + wc * 64;
  const int KT = K / kChunkK;
  const int nchunks = K / kChunkK;
  const int ngroups = K / G;

  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(wp, static_cast<uint32_t>(static_cast<size_t>(N) * K / 2));
  const __amdgpu_buffer_rsrc_t sz_rsrc = make_rsrc(sz, static_cast<uint32_t>(static_cast<size_t>(ngroups) * N * 4));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));
  const __amdgpu_buffer_rsrc_t xs_rsrc = make_rsrc(xsum, static_cast<uint32_t>(static_cast<size_t>(ngroups) * xsum_stride * 4));

  uint32_t szlane[kCT];  // byte offset of this lane's column inside one [N] row of (scale, zero) pairs
#pragma unroll
  for (int ct = 0; ct < kCT; ++ct) {
    int col = col0 + 32 * ct + n;
    col = col < N ? col : N - 1;
    szlane[ct] = static_cast<uint32_t>(col) * 4u;
  }

  // ---- accumulators start as the zero-point term: sum_g X[m,g] * (z - 136 s)[g,n] in float32 MFMAs --------
  f32x16_t acc[kCT][kRT];
#pragma unroll
  for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
    for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[ct][rt][e] = 0.f;
  {
    uint32_t xslane[kRT];
#pragma unroll
    for (int rt = 0; rt < kRT; ++rt) xslane[rt] = static_cast<uint32_t>(h * xsum_stride + row0 + 32 * rt + n) * 4u;
    uint32_t zlane[kCT];
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct) zlane[ct] = szlane[ct] + static_cast<uint32_t>(h) * static_cast<uint32_t>(N) * 4u;
#pragma unroll 4
    for (int g0 = 0; g0 < ngroups; g0 += 2) {  // lanes with h = 1 take group g0 + 1 (reads past the last group return 0)
      float a[kRT], zc[kCT];
#pragma unroll
      for (int rt = 0; rt < kRT; ++rt)
        a[rt] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xs_rsrc, xslane[rt], static_cast<uint32_t>(g0) * xsum_stride * 4u, 0));
#pragma unroll
      for (int ct = 0; ct < kCT; ++ct) {
        const uint32_t szw = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, zlane[ct], static_cast<uint32_t>(g0) * N * 4u, 0);
        const float scale = __builtin_bit_cast(float, szw << 16), zero = __builtin_bit_cast(float, szw & 0xFFFF0000u);
        zc[ct] = __builtin_fmaf(-136.0f, scale, zero);
      }
#pragma unroll
      for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
        for (int rt = 0; rt < kRT; ++rt) acc[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rt], zc[ct], acc[ct][rt], 0, 0, 0);
    }
  }

  // ---- staging.  Activations: piece (row, within): span p = within / 4 of 32 k, quarter u = within % 4; its dword e
  // belongs to the fragment of step (p, e / 2), lane (h = e % 2, row % 32), register u.  Weights: piece (8-column block,
  // t) of a 512-byte block = the four words (column 8 blk + t / 4, j = t % 4): fragment (column tile, j / 2), lane
  // (h = j % 2, column % 32).
  const int xr0 = tid >> 4, xw = tid & 15;
  uint32_t xsrc[kXPieces];
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) {
    int row = rb * kRows + xr0 + kXRowsPerPass * i;
    row = row < M ? row : M - 1;
    xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + xw * 8) * 2);
  }
  const int xdst0 = ((xr0 >> 5) * 8 + 2 * (xw >> 2)) * kFragB + (xr0 & 31) * 16 + (xw & 3) * 4;
  const int wb0 = tid >> 5, wt = tid & 31;  // 8-column block within the pass, piece within the block
  uint32_t wsrc[kWPieces];
#pragma unroll
  for (int i = 0; i < kWPieces; ++i) {
    int nt8 = cb * (kCols / 8) + wb0 + kWTilesPerPass * i;
    nt8 = nt8 < (N >> 3) ? nt8 : (N >> 3) - 1;
    wsrc[i] = static_cast<uint32_t>((static_cast<size_t>(nt8) * KT * 32 + wt) * 16);
  }
  const int wdst0 = ((wb0 >> 2) * 2 + ((wt & 3) >> 1)) * kFragB + ((wt & 1) * 32 + 8 * (wb0 & 3) + (wt >> 2)) * 16;

  struct Staged {
    u32x4_t x[kXPieces], w[kWPieces];
  };
  auto load_next = [&](Staged &r, int ci) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
#pragma unroll
    for (int i = 0; i < kXPieces; ++i) r.x[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xsrc[i], static_cast<uint32_t>(cc) * (kChunkK * 2), 0);
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) r.w[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wsrc[i], static_cast<uint32_t>(cc) * 512u, 0);
  };
  auto store_next = [&](const Staged &r, int parity) {
    uint8_t *bx = lds + (parity & 1) * kStageX + xdst0;
#pragma unroll
    for (int i = 0; i < kXPieces; ++i) {
      uint8_t *d = bx + i * (kXRowsPerPass / 32) * (8 * kFragB);
#pragma unroll
      for (int e = 0; e < 4; ++e) *reinterpret_cast<uint32_t *>(d + (e >> 1) * kFragB + (e & 1) * (32 * 16)) = r.x[i][e];
    }
    uint8_t *bw = lds_w + (parity & 1) * kStageW + wdst0;
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) *reinterpret_cast<u32x4_t *>(bw + i * (kWTilesPerPass / 4) * (2 * kFragB)) = r.w[i];
  };
  auto load_scales = [&](uint32_t (&r)[kCT][NGRP], int ci) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
      for (int g = 0; g < NGRP; ++g)
        r[ct][g] = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, szlane[ct], static_cast<uint32_t>(cc * NGRP + g) * N * 4u, 0);
  };

  const UnpackConsts uc = unpack_consts();
  auto compute = [&](const uint32_t (&sc)[kCT][NGRP], int parity) {
    const uint8_t *bx = lds + (parity & 1) * kStageX + (wr * kRT) * (8 * kFragB) + lane * 16;
    const uint8_t *bw = lds_w + (parity & 1) * kStageW + (wc * kCT) * (2 * kFragB) + lane * 16;
    u32x4_t wq[kCT][2];  // [column tile][j pair]: words of the four 32-wide k spans
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
      for (int ld = 0; ld < 2; ++ld) wq[ct][ld] = *reinterpret_cast<const u32x4_t *>(bw + (ct * 2 + ld) * kFragB);
#pragma unroll
    for (int g = 0; g < NGRP; ++g) {
      f32x16_t part[kCT][kRT];
#pragma unroll
      for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
        for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
          for (int e = 0; e < 16; ++e) part[ct][rt][e] = 0.f;
#pragma unroll
      for (int sg = 0; sg < SPG; ++sg) {
        const int s = g * SPG + sg;  // step = 2 p + jp
        bf16x8_t af[kRT];
#pragma unroll
        for (int rt = 0; rt < kRT; ++rt) af[rt] = *reinterpret_cast<const bf16x8_t *>(bx + (rt * 8 + s) * kFragB);
#pragma unroll
        for (int ct = 0; ct < kCT; ++ct) {
          const bf16x8_t wf = unpack_word(wq[ct][s & 1][s >> 1], uc);
#pragma unroll
          for (int rt = 0; rt < kRT; ++rt) part[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[rt], wf, part[ct][rt], 0, 0, 0);
        }
      }
#pragma unroll
      for (int ct = 0; ct < kCT; ++ct) {
        const float scale = __builtin_bit_cast(float, sc[ct][g] << 16);
#pragma unroll
        for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[ct][rt][e] = __builtin_fmaf(scale, part[ct][rt][e], acc[ct][rt][e]);
      }
    }
  };

  // ---- main loop, two chunks per trip so that the scale registers are compile-time names -----------------
  Staged st;
  uint32_t sc[2][kCT][NGRP];
  load_next(st, 0);
  load_scales(sc[0], 0);
  store_next(st, 0);
  lds_barrier();
  for (int ci = 0; ci < nchunks; ci += 2) {
    load_next(st, ci + 1);       // in flight during the arithmetic of this chunk
    load_scales(sc[1], ci + 1);
    __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the arithmetic: the scheduler would sink it to its first use
    compute(sc[0], 0);
    store_next(st, 1);           // the other stage: everybody left it at the previous barrier
    lds_barrier();
    if (ci + 1 >= nchunks) break;  // uniform
    load_next(st, ci + 2);
    load_scales(sc[0], ci + 2);
    __builtin_amdgcn_sched_barrier(0);
    compute(sc[1], 1);
    store_next(st, 0);
    lds_barrier();
  }

  // ---- store: lane (h, n) holds column col0 + 32 ct + n, rows 8 (e / 4) + 4 h + e % 4 of each tile -----------
  // (the barrier that ended the last chunk left every wave done with the stages)
  const float no_scale[kCT] = {};
  store_tiles_via_lds<kRT, kCT, false>(acc, no_scale, lds + wave * TileStore<kCT>::kBytesPerWave, y, row0, col0, M, N, lane,
                                    (N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0);
}

}  // namespace

int int4_gemm32(const uint16_t *x, const int32_t *packed, const uint16_t *sz, uint16_t *y, const float *xsum, int xsum_stride,
                int M, int N, int K, int groupsize, hipStream_t stream) {
  if (K % kChunkK != 0 || N % 8 != 0) return E2H_ERR_BAD_SHAPE;
  constexpr int WR = 2, WC = 4;  // 128 rows x 256 columns per workgroup of 8 waves, one workgroup per CU (101 KB of LDS)
  const int n_col_blocks = (N + 64 * WC - 1) / (64 * WC), n_row_blocks = (M + 64 * WR - 1) / (64 * WR);
  const int cbx = (n_col_blocks + 7) / 8;
  const long long wgs = 8LL * cbx * n_row_blocks;
  if (wgs > 0x7FFFFFFFLL) return E2H_ERR_BAD_SHAPE;
  // the pre-pass pads its rows to 64; this kernel's lanes read whole row blocks: rows past the pad return 0 from the
  // buffer bound or belong to other groups' rows of the same array -- they only ever reach rows >= M, which are not stored
  dim3 grid(static_cast<unsigned>(wgs)), block(64 * WR * WC);
  const uint32_t *w = reinterpret_cast<const uint32_t *>(packed);
  const uint32_t *s = reinterpret_cast<const uint32_t *>(sz);
  switch (groupsize) {
    case 32: hipLaunchKernelGGL((int4_gemm32_kernel<32, WR, WC>), grid, block, 0, stream, x, w, s, y, xsum, xsum_stride, M, N, K, n_col_blocks, cbx); break;
    case 64: hipLaunchKernelGGL((int4_gemm32_kernel<64, WR, WC>), grid, block, 0, stream, x, w, s, y, xsum, xsum_stride, M, N, K, n_col_blocks, cbx); break;
    case 128: hipLaunchKernelGGL((int4_gemm32_kernel<128, WR, WC>), grid, block, 0, stream, x, w, s, y, xsum, xsum_stride, M, N, K, n_col_blocks, cbx); break;
    default: return E2H_ERR_BAD_GROUPSIZE;
  }
  return launch_status();
}

}  // namespace e2h

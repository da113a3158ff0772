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
// A workgroup of 4 waves owns 128 rows x 128 columns (each wave 64 x 64 = 2 x 2 tiles, 64 accumulator registers);
// activations are staged per 128-wide k chunk into LDS in fragment order (double buffered, one LDS barrier per
// chunk); every A fragment read feeds two column tiles and every unpacked word two row tiles.
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
constexpr int kStageB = 4 * 8 * kFragB;             // 128 rows x 128 k
constexpr int kRT = 2, kCT = 2;                     // 32x32 tiles per wave: rows x columns

template <int G>
__global__ __launch_bounds__(256) void int4_gemm32_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ wp,
                                                          const uint32_t *__restrict__ sz, uint16_t *__restrict__ y,
                                                          const float *__restrict__ xsum, int xsum_stride, int M, int N, int K,
                                                          int n_col_blocks, int cbx) {
  constexpr int NGRP = kChunkK / G;   // groups per chunk
  constexpr int SPG = G / 16;         // MFMA steps per group
  __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kStageB];

  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int cb = xcd + 8 * (slot % cbx);
  const int rb = slot / cbx;
  if (cb >= n_col_blocks) return;  // grid padding; uniform, before any barrier

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave >> 1, wc = wave & 1;
  const int n = lane & 31, h = lane >> 5;
  const int row0 = rb * 128 + wr * 64;
  const int col0 = cb * 128 + wc * 64;
  const int KT = K / kChunkK;
  const int nchunks = K / kChunkK;
  const int ngroups = K / G;

  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(wp, static_cast<uint32_t>(static_cast<size_t>(N) * K / 2));
  const __amdgpu_buffer_rsrc_t sz_rsrc = make_rsrc(sz, static_cast<uint32_t>(static_cast<size_t>(ngroups) * N * 4));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));
  const __amdgpu_buffer_rsrc_t xs_rsrc = make_rsrc(xsum, static_cast<uint32_t>(static_cast<size_t>(ngroups) * xsum_stride * 4));

  // per-lane constant byte offsets
  uint32_t wlane[kCT][2], szlane[kCT];
#pragma unroll
  for (int ct = 0; ct < kCT; ++ct) {
    int col = col0 + 32 * ct + n;
    col = col < N ? col : N - 1;
    szlane[ct] = static_cast<uint32_t>(col) * 4u;
#pragma unroll
    for (int ld = 0; ld < 2; ++ld) {
      const int j = 2 * ld + h;
      wlane[ct][ld] = static_cast<uint32_t>((static_cast<size_t>(col >> 3) * KT * 32 + ((col & 7) * 4 + j)) * 16);
    }
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

  // ---- activation staging: 2048 16-byte pieces per chunk, 8 per thread ------------------------------
  // piece (row, within): span p = within / 4 of 32 k, quarter u = within % 4; its dword e belongs to the fragment
  // of step (p, e / 2), lane (h = e % 2, row % 32), register u.
  const int r0 = tid >> 4, within = tid & 15;
  uint32_t xsrc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int row = rb * 128 + r0 + 16 * i;
    row = row < M ? row : M - 1;
    xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + within * 8) * 2);
  }
  const int xdst0 = (2 * (within >> 2)) * kFragB + r0 * 16 + (within & 3) * 4;
  auto load_x = [&](u32x4_t (&r)[8], int ci) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xsrc[i], static_cast<uint32_t>(cc) * (kChunkK * 2), 0);
  };
  auto store_x = [&](const u32x4_t (&r)[8], int parity) {
    uint8_t *buf = lds + (parity & 1) * kStageB + xdst0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // row = r0 + 16 i: row tile i / 2, row within the tile r0 + 16 (i % 2)
      uint8_t *d = buf + (i >> 1) * (8 * kFragB) + (i & 1) * (16 * 16);
#pragma unroll
      for (int e = 0; e < 4; ++e) *reinterpret_cast<uint32_t *>(d + (e >> 1) * kFragB + (e & 1) * (32 * 16)) = r[i][e];
    }
  };

  struct WRegs {
    u32x4_t w[kCT][2];
    uint32_t s[kCT][NGRP];
  };
  auto load_w = [&](WRegs &r, int ci) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
    const uint32_t so = static_cast<uint32_t>(cc) * 512u;
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct) {
#pragma unroll
      for (int ld = 0; ld < 2; ++ld) r.w[ct][ld] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wlane[ct][ld], so, 0);
#pragma unroll
      for (int g = 0; g < NGRP; ++g)
        r.s[ct][g] = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, szlane[ct], static_cast<uint32_t>(cc * NGRP + g) * N * 4u, 0);
    }
  };

  const UnpackConsts uc = unpack_consts();
  auto compute = [&](const WRegs &r, int parity) {
    const uint8_t *buf = lds + (parity & 1) * kStageB + (wr * kRT) * (8 * kFragB) + lane * 16;
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
        for (int rt = 0; rt < kRT; ++rt) af[rt] = *reinterpret_cast<const bf16x8_t *>(buf + (rt * 8 + s) * kFragB);
#pragma unroll
        for (int ct = 0; ct < kCT; ++ct) {
          const bf16x8_t wf = unpack_word(r.w[ct][s & 1][s >> 1], uc);
#pragma unroll
          for (int rt = 0; rt < kRT; ++rt) part[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[rt], wf, part[ct][rt], 0, 0, 0);
        }
      }
#pragma unroll
      for (int ct = 0; ct < kCT; ++ct) {
        const float scale = __builtin_bit_cast(float, r.s[ct][g] << 16);
#pragma unroll
        for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[ct][rt][e] = __builtin_fmaf(scale, part[ct][rt][e], acc[ct][rt][e]);
      }
    }
  };

  // ---- main loop, two chunks per trip so that the register buffers are compile-time names ------------
  WRegs ring[2];
  u32x4_t xst[8];
  load_x(xst, 0);
  load_w(ring[0], 0);
  store_x(xst, 0);
  lds_barrier();
  for (int ci = 0; ci < nchunks; ci += 2) {
    load_x(xst, ci + 1);
    load_w(ring[1], ci + 1);
    compute(ring[0], 0);
    store_x(xst, 1);
    lds_barrier();
    if (ci + 1 >= nchunks) break;  // uniform
    load_x(xst, ci + 2);
    load_w(ring[0], ci + 2);
    compute(ring[1], 1);
    store_x(xst, 0);
    lds_barrier();
  }

  // ---- store: lane (h, n) holds column col0 + 32 ct + n, rows 8 (e / 4) + 4 h + e % 4 of each tile -----------
#pragma unroll
  for (int ct = 0; ct < kCT; ++ct) {
    const int col = col0 + 32 * ct + n;
#pragma unroll
    for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = row0 + 32 * rt + 8 * (e >> 2) + 4 * h + (e & 3);
        if (row < M && col < N) y[static_cast<size_t>(row) * N + col] = f32_to_bf16_rne(acc[ct][rt][e]);
      }
  }
}

}  // namespace

int int4_gemm32(const uint16_t *x, const int32_t *packed, const uint16_t *sz, uint16_t *y, const float *xsum, int xsum_stride,
                int M, int N, int K, int groupsize, hipStream_t stream) {
  if (K % kChunkK != 0 || N % 8 != 0) return E2H_ERR_BAD_SHAPE;
  const int n_col_blocks = (N + 127) / 128, n_row_blocks = (M + 127) / 128;
  const int cbx = (n_col_blocks + 7) / 8;
  const long long wgs = 8LL * cbx * n_row_blocks;
  if (wgs > 0x7FFFFFFFLL) return E2H_ERR_BAD_SHAPE;
  // the pre-pass pads its rows to 64; this kernel's lanes read 128-row blocks: rows past the pad return 0 from the
  // buffer bound or belong to other groups' rows of the same array -- they only ever reach rows >= M, which are not stored
  dim3 grid(static_cast<unsigned>(wgs));
  const uint32_t *w = reinterpret_cast<const uint32_t *>(packed);
  const uint32_t *s = reinterpret_cast<const uint32_t *>(sz);
  switch (groupsize) {
    case 32: hipLaunchKernelGGL(int4_gemm32_kernel<32>, grid, dim3(256), 0, stream, x, w, s, y, xsum, xsum_stride, M, N, K, n_col_blocks, cbx); break;
    case 64: hipLaunchKernelGGL(int4_gemm32_kernel<64>, grid, dim3(256), 0, stream, x, w, s, y, xsum, xsum_stride, M, N, K, n_col_blocks, cbx); break;
    case 128: hipLaunchKernelGGL(int4_gemm32_kernel<128>, grid, dim3(256), 0, stream, x, w, s, y, xsum, xsum_stride, M, N, K, n_col_blocks, cbx); break;
    default: return E2H_ERR_BAD_GROUPSIZE;
  }
  return launch_status();
}

}  // namespace e2h

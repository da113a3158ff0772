// int8 per-channel matmul for many rows of x (reward scoring, prefill): MFMA-bound, 32x32 tiles.
//
// Same contract as e2h_int8_mm (WeightOnlyInt8Linear.forward, reference models/quantize.py:428-429):
//   y = bf16( bf16( x @ q^T ) * scales ),   q int8 [N][K] row-major, K % 128 == 0, 16-byte aligned rows.
//
// int8 -> bfloat16 without sign handling: u = q + 128 (one XOR per four codes) lies in [0, 255] and is exactly
// representable in bfloat16's 8 significant bits, so each code costs one byte-to-float convert and half a byte
// permute.  The offset is taken back out through the accumulators' initial value
//   acc0[m,n] = -128 * sum_k x[m,k],
// built before the main loop from per-128 sums of x (a one-pass pre-kernel) with v_mfma_f32_32x32x2_f32.
//
// Main loop, v_mfma_f32_32x32x16_bf16: lane L = 32*h + n supplies weight row n0 + n; per 32-wide k span t it loads
// the 16 bytes k = 32 t + 16 h .. +15 (one 128-bit load), bytes 0..7 feeding step (t, 0) and bytes 8..15 step
// (t, 1).  The activation fragment of lane (h, m) for step (t, a) is then the 16 contiguous bytes
// x[m][32 t + 16 h + 8 a .. +7]: staging into LDS is a plain 16-byte copy per piece.  A workgroup of 4 waves owns
// 128 rows x 128 columns, each wave 2 x 2 tiles accumulating straight into its 64 accumulator registers (no
// per-group scale to apply); workgroups are laid out over the XCDs as in the int4 kernel of the same shape.
#include "e2h_common.h"
#include "e2h_int4_unpack.h"

namespace e2h {
namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kChunkK8 = 128;
constexpr int kFragB8 = 1024 + 32;
constexpr int kStageB8 = 4 * 8 * kFragB8;
constexpr int kRT8 = 2, kCT8 = 2;

// four codes (one dword, already offset to unsigned) -> two dwords of bfloat16 pairs
__device__ __forceinline__ void bytes4_to_bf16(uint32_t t, uint32_t &lo, uint32_t &hi) {
  const float f0 = static_cast<float>(t & 0xFFu), f1 = static_cast<float>((t >> 8) & 0xFFu);
  const float f2 = static_cast<float>((t >> 16) & 0xFFu), f3 = static_cast<float>(t >> 24);
  // high halves of two floats (exact: the values have at most 8 significant bits)
  lo = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
  hi = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2), 0x07060302u);
}

__global__ __launch_bounds__(256) void int8_gemm32_kernel(const uint16_t *__restrict__ x, const int8_t *__restrict__ q,
                                                          const uint16_t *__restrict__ scales, uint16_t *__restrict__ y,
                                                          const float *__restrict__ xsum, int xsum_stride, int M, int N, int K,
                                                          int n_col_blocks, int cbx) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kStageB8];

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
  const int nchunks = K / kChunkK8;

  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(q, static_cast<uint32_t>(static_cast<size_t>(N) * K));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));
  const __amdgpu_buffer_rsrc_t xs_rsrc = make_rsrc(xsum, static_cast<uint32_t>(static_cast<size_t>(nchunks) * xsum_stride * 4));

  uint32_t wlane[kCT8];
#pragma unroll
  for (int ct = 0; ct < kCT8; ++ct) {
    int col = col0 + 32 * ct + n;
    col = col < N ? col : N - 1;
    wlane[ct] = static_cast<uint32_t>(static_cast<size_t>(col) * K + 16 * h);
  }

  // ---- accumulators start at -128 * sum_k x[m,k] (float32 MFMAs over the per-chunk sums of x) ------------------
  f32x16_t acc[kCT8][kRT8];
#pragma unroll
  for (int ct = 0; ct < kCT8; ++ct)
#pragma unroll
    for (int rt = 0; rt < kRT8; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[ct][rt][e] = 0.f;
  {
    uint32_t xslane[kRT8];
#pragma unroll
    for (int rt = 0; rt < kRT8; ++rt) xslane[rt] = static_cast<uint32_t>(h * xsum_stride + row0 + 32 * rt + n) * 4u;
#pragma unroll 4
    for (int g0 = 0; g0 < nchunks; g0 += 2) {  // lanes with h = 1 take chunk g0 + 1 (reads past the last one return 0)
      float a[kRT8];
#pragma unroll
      for (int rt = 0; rt < kRT8; ++rt)
        a[rt] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xs_rsrc, xslane[rt], static_cast<uint32_t>(g0) * xsum_stride * 4u, 0));
#pragma unroll
      for (int ct = 0; ct < kCT8; ++ct)
#pragma unroll
        for (int rt = 0; rt < kRT8; ++rt) acc[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rt], -128.0f, acc[ct][rt], 0, 0, 0);
    }
  }

  // ---- activation staging: piece (row, w): k = 8 w .. 8 w + 7 = 32 t + 16 h + 8 a with w = 4 t + 2 h + a -------------
  const int r0 = tid >> 4, within = tid & 15;
  uint32_t xsrc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int row = rb * 128 + r0 + 16 * i;
    row = row < M ? row : M - 1;
    xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + within * 8) * 2);
  }
  const int xdst0 = (2 * (within >> 2) + (within & 1)) * kFragB8 + (((within >> 1) & 1) * 32 + r0) * 16;
  auto load_x = [&](u32x4_t (&r)[8], int ci) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xsrc[i], static_cast<uint32_t>(cc) * (kChunkK8 * 2), 0);
  };
  auto store_x = [&](const u32x4_t (&r)[8], int parity) {
    uint8_t *buf = lds + (parity & 1) * kStageB8 + xdst0;
#pragma unroll
    for (int i = 0; i < 8; ++i)  // row = r0 + 16 i: row tile i / 2, row within the tile r0 + 16 (i % 2)
      *reinterpret_cast<u32x4_t *>(buf + (i >> 1) * (8 * kFragB8) + (i & 1) * (16 * 16)) = r[i];
  };

  struct WRegs {
    u32x4_t w[kCT8][4];
  };
  auto load_w = [&](WRegs &r, int ci) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
#pragma unroll
    for (int ct = 0; ct < kCT8; ++ct)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        r.w[ct][t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wlane[ct], static_cast<uint32_t>(cc) * kChunkK8 + 32u * t, 0);
  };

  auto compute = [&](const WRegs &r, int parity) {
    const uint8_t *buf = lds + (parity & 1) * kStageB8 + (wr * kRT8) * (8 * kFragB8) + lane * 16;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int s = 2 * t + a;
        bf16x8_t af[kRT8];
#pragma unroll
        for (int rt = 0; rt < kRT8; ++rt) af[rt] = *reinterpret_cast<const bf16x8_t *>(buf + (rt * 8 + s) * kFragB8);
#pragma unroll
        for (int ct = 0; ct < kCT8; ++ct) {
          uint32_t u0, u1, u2, u3;
          bytes4_to_bf16(r.w[ct][t][2 * a] ^ 0x80808080u, u0, u1);
          bytes4_to_bf16(r.w[ct][t][2 * a + 1] ^ 0x80808080u, u2, u3);
          const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, u32x4_t{u0, u1, u2, u3});
#pragma unroll
          for (int rt = 0; rt < kRT8; ++rt) acc[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[rt], wf, acc[ct][rt], 0, 0, 0);
        }
      }
    }
  };

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

  // ---- store with the reference's two roundings: bf16(acc), then bf16(t * scale) ----------------------------------
#pragma unroll
  for (int ct = 0; ct < kCT8; ++ct) {
    const int col = col0 + 32 * ct + n;
    const float scale = bf16_to_f32(scales[col < N ? col : N - 1]);
#pragma unroll
    for (int rt = 0; rt < kRT8; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = row0 + 32 * rt + 8 * (e >> 2) + 4 * h + (e & 3);
        if (row < M && col < N) y[static_cast<size_t>(row) * N + col] = f32_to_bf16_rne(bf16_round(acc[ct][rt][e]) * scale);
      }
  }
}

}  // namespace

int int8_gemm32(const uint16_t *x, const int8_t *q, const uint16_t *scales, uint16_t *y, float *xsum, int64_t xsum_bytes, int M,
                int N, int K, hipStream_t stream) {
  if (K % kChunkK8 != 0) return E2H_ERR_BAD_SHAPE;
  const int stride = ((M + 63) / 64) * 64;
  if (static_cast<int64_t>(K / kChunkK8) * stride * 4 > xsum_bytes) return E2H_ERR_BAD_SHAPE;
  const int rc = launch_x_group_sums(x, xsum, M, K, stride, 128, stream);
  if (rc != E2H_OK) return rc;
  const int n_col_blocks = (N + 127) / 128, n_row_blocks = (M + 127) / 128;
  const int cbx = (n_col_blocks + 7) / 8;
  const long long wgs = 8LL * cbx * n_row_blocks;
  if (wgs > 0x7FFFFFFFLL) return E2H_ERR_BAD_SHAPE;
  hipLaunchKernelGGL(int8_gemm32_kernel, dim3(static_cast<unsigned>(wgs)), dim3(256), 0, stream, x, q, scales, y, xsum, stride, M, N, K,
                     n_col_blocks, cbx);
  return launch_status();
}

}  // namespace e2h

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
// Main loop, v_mfma_f32_32x32x16_bf16: lane L = 32*h + n supplies weight row n0 + n; per 32-wide k span t its B
// operands are the 16 bytes k = 32 t + 16 h .. +15, bytes 0..7 feeding step (t, 0) and bytes 8..15 step (t, 1).  The
// activation fragment of lane (h, m) for step (t, a) is then the 16 contiguous bytes x[m][32 t + 16 h + 8 a .. +7].
// Both operands are staged per 128-wide k chunk into LDS in fragment order by plain 16-byte copies (double buffered,
// one LDS barrier per chunk): read straight from memory, a weight fragment would touch 32 different rows per load
// instruction, and that address traffic -- not the arithmetic -- bounded an earlier form of this kernel (measured:
// 38 % of its time).  Staged, every global load covers whole 128-byte rows.  A workgroup of WR x WC waves owns
// 64 WR rows x 64 WC columns, each wave 2 x 2 tiles accumulating straight into its 64 accumulator registers (no
// per-group scale to apply); workgroups are laid out over the XCDs as in the int4 kernel of the same shape.
#include "e2h_common.h"
#include "e2h_int4_unpack.h"

namespace e2h {
namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kFragB8 = 1024 + 32;

// four codes (one dword, already offset to unsigned) -> two dwords of bfloat16 pairs
__device__ __forceinline__ void bytes4_to_bf16(uint32_t t, uint32_t &lo, uint32_t &hi) {
  const float f0 = static_cast<float>(t & 0xFFu), f1 = static_cast<float>((t >> 8) & 0xFFu);
  const float f2 = static_cast<float>((t >> 16) & 0xFFu), f3 = static_cast<float>(t >> 24);
  // high halves of two floats (exact: the values have at most 8 significant bits)
  lo = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
  hi = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2), 0x07060302u);
}

// WR x WC waves per workgroup, RT x CT tiles of 32 x 32 outputs per wave, CK = k per staged chunk (64 or 128).
// <2, 4, 2, 2, 128>: 8 waves, 128 x 256 outputs per workgroup.  <2, 4, 4, 2, 64>: 8 waves, 256 x 256 outputs per
// workgroup, every wave 128 rows x 64 columns (128 accumulator registers): a converted weight fragment feeds four row
// tiles instead of two, so conversions and LDS reads per MFMA drop by 40 %; the k chunk halves to keep both stages
// within the LDS.  (Four waves with 4 x 4 tiles and the accumulators in the accumulation registers measured slower:
// one wave per SIMD leaves nothing to cover its LDS and conversion latencies.)
template <int WR, int WC, int RT, int CT, int CK>
__global__ __launch_bounds__(64 * WR * WC) void int8_gemm32_kernel(const uint16_t *__restrict__ x, const int8_t *__restrict__ q,
                                                                   const uint16_t *__restrict__ scales, uint16_t *__restrict__ y,
                                                                   const float *__restrict__ xsum, int xsum_stride, int M, int N, int K,
                                                                   int n_col_blocks, int cbx) {
  constexpr int kThreads = 64 * WR * WC;
  constexpr int kRows = 32 * RT * WR, kCols = 32 * CT * WC;
  constexpr int SPC = CK / 16;                        // MFMA steps per chunk = activation fragments per 32-row tile
  constexpr int TPC = CK / 32;                        // 32-wide k spans per chunk = weight fragments per 32-column tile
  constexpr int kStageX = (RT * WR) * SPC * kFragB8;  // kRows x CK of activations
  constexpr int kStageW = (CT * WC) * TPC * kFragB8;  // kCols x CK of weights
  constexpr int PX = CK / 8, PW = CK / 16;            // 16-byte pieces per activation row / weight row and chunk
  constexpr int kXRowsPerPass = kThreads / PX;
  constexpr int kXPieces = kRows / kXRowsPerPass;
  constexpr int kWColsPerPass = kThreads / PW;
  constexpr int kWPieces = kCols / kWColsPerPass;
  static_assert(kXRowsPerPass % 32 == 0 && kWColsPerPass % 32 == 0, "staging passes cover whole 32-wide tiles");
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
  const int row0 = rb * kRows + wr * (32 * RT);
  const int col0 = cb * kCols + wc * (32 * CT);
  const int nchunks = K / CK;
  const int nsums = K / 128;  // the pre-pass leaves sums of x over spans of 128

  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(q, static_cast<uint32_t>(static_cast<size_t>(N) * K));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));
  const __amdgpu_buffer_rsrc_t xs_rsrc = make_rsrc(xsum, static_cast<uint32_t>(static_cast<size_t>(nsums) * xsum_stride * 4));

  // ---- accumulators start at -128 * sum_k x[m,k] (float32 MFMAs over the per-chunk sums of x) ------------------
  // (the value does not depend on the column: one MFMA chain per row tile, copied to the tile's columns)
  f32x16_t acc[CT][RT];
  {
    f32x16_t init[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) init[rt][e] = 0.f;
    uint32_t xslane[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) xslane[rt] = static_cast<uint32_t>(h * xsum_stride + row0 + 32 * rt + n) * 4u;
#pragma unroll 4
    for (int g0 = 0; g0 < nsums; g0 += 2) {  // lanes with h = 1 take span g0 + 1 (reads past the last one return 0)
      float a[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
        a[rt] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xs_rsrc, xslane[rt], static_cast<uint32_t>(g0) * xsum_stride * 4u, 0));
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) init[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rt], -128.0f, init[rt], 0, 0, 0);
    }
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) acc[ct][rt] = init[rt];
  }

  // ---- staging.  Activations: piece (row, w), k = 8 w .. 8 w + 7 = 32 t + 16 h + 8 a with w = 4 t + 2 h + a, goes to
  // fragment (row tile, step 2 t + a), lane (h, row % 32).  Weights: piece (col, pc), bytes 16 pc .. 16 pc + 15 =
  // 32 t + 16 h with pc = 2 t + h, goes to fragment (column tile, t), lane (h, col % 32).
  const int xr0 = tid / PX, xw = tid % PX;
  uint32_t xsrc[kXPieces];
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) {
    int row = rb * kRows + xr0 + kXRowsPerPass * i;
    row = row < M ? row : M - 1;
    xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + xw * 8) * 2);
  }
  const int xdst0 = ((xr0 >> 5) * SPC + 2 * (xw >> 2) + (xw & 1)) * kFragB8 + (((xw >> 1) & 1) * 32 + (xr0 & 31)) * 16;
  const int wc0 = tid / PW, wpc = tid % PW;
  uint32_t wsrc[kWPieces];
#pragma unroll
  for (int i = 0; i < kWPieces; ++i) {
    int col = cb * kCols + wc0 + kWColsPerPass * i;
    col = col < N ? col : N - 1;
    wsrc[i] = static_cast<uint32_t>(static_cast<size_t>(col) * K + wpc * 16);
  }
  const int wdst0 = ((wc0 >> 5) * TPC + (wpc >> 1)) * kFragB8 + ((wpc & 1) * 32 + (wc0 & 31)) * 16;

  struct Staged {
    u32x4_t x[kXPieces], w[kWPieces];
  };
  auto load_next = [&](Staged &r, int ci) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
#pragma unroll
    for (int i = 0; i < kXPieces; ++i) r.x[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xsrc[i], static_cast<uint32_t>(cc) * (CK * 2), 0);
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) r.w[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wsrc[i], static_cast<uint32_t>(cc) * CK, 0);
  };
  auto store_next = [&](const Staged &r, int parity) {
    uint8_t *bx = lds + (parity & 1) * kStageX + xdst0;
#pragma unroll
    for (int i = 0; i < kXPieces; ++i) *reinterpret_cast<u32x4_t *>(bx + i * (kXRowsPerPass / 32) * (SPC * kFragB8)) = r.x[i];
    uint8_t *bw = lds_w + (parity & 1) * kStageW + wdst0;
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) *reinterpret_cast<u32x4_t *>(bw + i * (kWColsPerPass / 32) * (TPC * kFragB8)) = r.w[i];
  };

  auto compute = [&](int parity) {
    const uint8_t *bx = lds + (parity & 1) * kStageX + (wr * RT) * (SPC * kFragB8) + lane * 16;
    const uint8_t *bw = lds_w + (parity & 1) * kStageW + (wc * CT) * (TPC * kFragB8) + lane * 16;
#pragma unroll
    for (int t = 0; t < TPC; ++t) {
      u32x4_t wq[CT];
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) wq[ct] = *reinterpret_cast<const u32x4_t *>(bw + (ct * TPC + t) * kFragB8);
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int s = 2 * t + a;
        bf16x8_t af[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) af[rt] = *reinterpret_cast<const bf16x8_t *>(bx + (rt * SPC + s) * kFragB8);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          uint32_t u0, u1, u2, u3;
          bytes4_to_bf16(wq[ct][2 * a] ^ 0x80808080u, u0, u1);
          bytes4_to_bf16(wq[ct][2 * a + 1] ^ 0x80808080u, u2, u3);
          const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, u32x4_t{u0, u1, u2, u3});
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) acc[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[rt], wf, acc[ct][rt], 0, 0, 0);
        }
      }
    }
  };

  Staged st;
  load_next(st, 0);
  store_next(st, 0);
  lds_barrier();
  for (int ci = 0; ci < nchunks; ++ci) {
    load_next(st, ci + 1);       // in flight during the arithmetic of this chunk ...
    __builtin_amdgcn_sched_barrier(0);  // ... which the scheduler would otherwise undo by sinking the loads to their first use
    compute(ci);
    store_next(st, ci + 1);      // the other stage: everybody left it at the previous barrier
    lds_barrier();
  }

  // ---- store with the reference's two roundings: bf16(acc), then bf16(t * scale) ----------------------------------
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col = col0 + 32 * ct + n;
    const float scale = bf16_to_f32(scales[col < N ? col : N - 1]);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
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
  if (K % 128 != 0) return E2H_ERR_BAD_SHAPE;
  const int stride = ((M + 63) / 64) * 64;
  if (static_cast<int64_t>(K / 128) * stride * 4 > xsum_bytes) return E2H_ERR_BAD_SHAPE;
  const int rc = launch_x_group_sums(x, xsum, M, K, stride, 128, stream);
  if (rc != E2H_OK) return rc;
  // 256 x 256 or 128 x 256 outputs per workgroup (one workgroup per CU either way).  A 256-row workgroup takes
  // about 1.8 x as long as a 128-row one (measured: 10 % more throughput), so it wins exactly when it needs fewer than
  // 1 / 1.8 as many rounds of workgroups over the chip's 256 CUs.
  const long long wgs256 = static_cast<long long>((M + 255) / 256) * ((N + 255) / 256);
  const long long wgs128 = static_cast<long long>((M + 127) / 128) * ((N + 255) / 256);
  const long long rounds256 = (wgs256 + 255) / 256, rounds128 = (wgs128 + 255) / 256;
  const bool big = options().int8_gemm_tile ? options().int8_gemm_tile == 256 : rounds256 * 20 <= rounds128 * 11;
  const int rows = big ? 256 : 128;
  const int n_col_blocks = (N + 255) / 256, n_row_blocks = (M + rows - 1) / rows;
  const int cbx = (n_col_blocks + 7) / 8;
  const long long wgs = 8LL * cbx * n_row_blocks;
  if (wgs > 0x7FFFFFFFLL) return E2H_ERR_BAD_SHAPE;
  if (big)
    hipLaunchKernelGGL((int8_gemm32_kernel<2, 4, 4, 2, 64>), dim3(static_cast<unsigned>(wgs)), dim3(512), 0, stream, x, q, scales, y, xsum,
                       stride, M, N, K, n_col_blocks, cbx);
  else
    hipLaunchKernelGGL((int8_gemm32_kernel<2, 4, 2, 2, 128>), dim3(static_cast<unsigned>(wgs)), dim3(512), 0, stream, x, q, scales, y, xsum,
                       stride, M, N, K, n_col_blocks, cbx);
  return launch_status();
}

}  // namespace e2h

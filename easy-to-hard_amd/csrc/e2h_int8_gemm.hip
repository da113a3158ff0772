// int8 per-channel matmul for many rows of x (reward scoring, prefill): MFMA-bound, 32x32 tiles.
//
// Same contract as e2h_int8_mm (WeightOnlyInt8Linear.forward, reference models/quantize.py:428-429):
//   y = bf16( bf16( x @ q^T ) * scales ),   q int8 [N][K] row-major, K % 128 == 0, 16-byte aligned rows.
//
// int8 -> bfloat16: a sign-extending byte-to-float convert per code (the value has at most 8 significant bits, so
// the high half of the float is the exact bfloat16) and half a byte permute to pack two of them.
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
#include <algorithm>

#include "e2h_common.h"
#include "e2h_int4_unpack.h"

namespace e2h {
namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kFragB8 = 1024 + 32;

// four codes (one dword) -> two dwords of bfloat16 pairs
__device__ __forceinline__ void bytes4_to_bf16(uint32_t t, uint32_t &lo, uint32_t &hi) {
  const float f0 = static_cast<float>(static_cast<int8_t>(t & 0xFFu)), f1 = static_cast<float>(static_cast<int8_t>((t >> 8) & 0xFFu));
  const float f2 = static_cast<float>(static_cast<int8_t>((t >> 16) & 0xFFu)), f3 = static_cast<float>(static_cast<int8_t>(t >> 24));
  // high halves of two floats (exact: the values have at most 8 significant bits)
  lo = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
  hi = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2), 0x07060302u);
}

// WR x WC waves per workgroup, RT x CT tiles of 32 x 32 outputs per wave, CK = k per staged chunk (64 or 128).
// <2, 4, 2, 2, 128>: 8 waves, 128 x 256 outputs per workgroup, the form for row counts that leave CUs idle with
// 256-row workgroups.  <2, 4, 4, 2, 64>: 8 waves, 256 x 256 outputs per workgroup, every wave 128 rows x 64 columns
// (128 accumulator registers); kept selectable as the comparison for int8_gemm128_kernel below, which replaced it.
template <int WR, int WC, int RT, int CT, int CK>
__global__ __launch_bounds__(64 * WR * WC) void int8_gemm32_kernel(const uint16_t *__restrict__ x, const int8_t *__restrict__ q,
                                                                   const uint16_t *__restrict__ scales, uint16_t *__restrict__ y, int M, int N,
                                                                   int K, int n_col_blocks, int cbx) {
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

  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(q, static_cast<uint32_t>(static_cast<size_t>(N) * K));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));

  f32x16_t acc[CT][RT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[ct][rt][e] = 0.f;

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
          bytes4_to_bf16(wq[ct][2 * a], u0, u1);
          bytes4_to_bf16(wq[ct][2 * a + 1], u2, u3);
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
  float scale[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col = col0 + 32 * ct + n;
    scale[ct] = bf16_to_f32(scales[col < N ? col : N - 1]);
  }
  // (the barrier that ended the last chunk left every wave done with the stages)
  store_tiles_via_lds<RT, CT, true>(acc, scale, lds + wave * TileStore<CT>::kBytesPerWave, y, row0, col0, M, N, lane,
                                    (N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0);
}


// Four waves, 256 x 256 outputs per workgroup: <2, 2> every wave 128 rows x 128 columns, <1, 4> 256 rows x 64
// columns (the default: a converted weight fragment then feeds eight MFMAs and no two waves convert the same one).
// 256 accumulator registers per lane: one wave per SIMD owns the whole 512-register budget, each fragment read from
// LDS feeds more MFMAs, and the LDS carries about half the bytes per MFMA of the eight-wave forms.  With nothing else
// on the SIMD to cover latencies the wave pipelines itself (see the slot schedule in the body).  Codes are converted
// with sign-extending byte-to-float instructions, so there is no +128 offset to take back out: no pass over x
// beforehand, no accumulator prologue.  Measured against the eight-wave 256-row form on the same GPU, 7B shapes at
// 8192 rows: 4 % (12288 x 4096) to 14 % (4096 x 11008) less time.  What bounds it: with every matrix pipeline busy
// the chip clocks near 1.6 GHz (the same loop with the MFMAs alone reaches 1650 TFLOP/s, which the bfloat16 library
// matmul nearly attains); LDS reads, staging stores and loads each add 8 - 14 % on top when timed by omission.
template <int WR, int WC, int CK>
__global__ __launch_bounds__(256) void int8_gemm128_kernel(const uint16_t *__restrict__ x, const int8_t *__restrict__ q,
                                                           const uint16_t *__restrict__ scales, uint16_t *__restrict__ y, int M, int N, int K,
                                                           int n_col_blocks, int cbx) {
  static_assert(WR * WC == 4, "four waves");
  constexpr int RT = 8 / WR, CT = 8 / WC;  // 256 x 256 outputs per workgroup
  constexpr int kThreads = 256;
  constexpr int kRows = 256, kCols = 256;
  constexpr int SPC = CK / 16, TPC = CK / 32;
  // A fragment block in LDS: lanes (h, r) at h * half + 16 r.  The strides are chosen for the staging stores, which a
  // 16-lane group issues as 2 rows x 8 pieces (activations: 4 steps x 2 halves, 32 bytes each) or 4 rows x 4 pieces
  // (weights: 2 spans x 2 halves, 64 bytes each): with these strides the 16 stores of a group fall into 16 different
  // 16-byte bank groups of the 256-byte LDS row, as the fragment reads (16 lanes, 256 contiguous bytes) always do.
  constexpr int kFragX = 1184, kHalfX = 640;  // 1184 = 5 * 32 mod 256, 640 = 128 mod 256
  constexpr int kFragW = 1152, kHalfW = 576;  // 1152 = 128 mod 256, 576 = 64 mod 256
  constexpr int kStageX = (RT * WR) * SPC * kFragX;
  constexpr int kStageW = (CT * WC) * TPC * kFragW;
  constexpr int PX = CK / 8, PW = CK / 16;
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

  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(q, static_cast<uint32_t>(static_cast<size_t>(N) * K));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));

  f32x16_t acc[CT][RT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[ct][rt][e] = 0.f;

  // staging: the same piece -> fragment maps as in int8_gemm32_kernel
  const int xr0 = tid / PX, xw = tid % PX;
  uint32_t xsrc[kXPieces];
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) {
    int row = rb * kRows + xr0 + kXRowsPerPass * i;
    row = row < M ? row : M - 1;
    xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + xw * 8) * 2);
  }
  const int xdst0 = ((xr0 >> 5) * SPC + 2 * (xw >> 2) + (xw & 1)) * kFragX + ((xw >> 1) & 1) * kHalfX + (xr0 & 31) * 16;
  const int wc0 = tid / PW, wpc = tid % PW;
  uint32_t wsrc[kWPieces];
#pragma unroll
  for (int i = 0; i < kWPieces; ++i) {
    int col = cb * kCols + wc0 + kWColsPerPass * i;
    col = col < N ? col : N - 1;
    wsrc[i] = static_cast<uint32_t>(static_cast<size_t>(col) * K + wpc * 16);
  }
  const int wdst0 = ((wc0 >> 5) * TPC + (wpc >> 1)) * kFragW + (wpc & 1) * kHalfW + (wc0 & 31) * 16;

  static_assert(kXPieces + kWPieces == 12 && SPC == 4, "the slot schedule below is written for 64-wide chunks");
  struct Staged {
    u32x4_t p[kXPieces + kWPieces];  // activation pieces, then weight pieces
  };
  auto load_piece = [&](Staged &r, int ci, int i) {
    const int cc = ci < nchunks ? ci : nchunks - 1;
    if (i < kXPieces)
      r.p[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xsrc[i], static_cast<uint32_t>(cc) * (CK * 2), 0);
    else
      r.p[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wsrc[i - kXPieces], static_cast<uint32_t>(cc) * CK, 0);
  };
  auto store_piece = [&](const Staged &r, int parity, int i) {
    if (i < kXPieces)
      *reinterpret_cast<u32x4_t *>(lds + (parity & 1) * kStageX + xdst0 + i * (kXRowsPerPass / 32) * (SPC * kFragX)) = r.p[i];
    else
      *reinterpret_cast<u32x4_t *>(lds_w + (parity & 1) * kStageW + wdst0 + (i - kXPieces) * (kWColsPerPass / 32) * (TPC * kFragW)) = r.p[i];
  };

  const int x_frag0 = (wr * RT) * (SPC * kFragX) + h * kHalfX + n * 16;
  const int w_frag0 = (wc * CT) * (TPC * kFragW) + h * kHalfW + n * 16;
  bf16x8_t af[2][RT];
  u32x4_t wq[2][CT];
  auto read_a = [&](int parity, int s, int rt) {
    return *reinterpret_cast<const bf16x8_t *>(lds + (parity & 1) * kStageX + x_frag0 + (rt * SPC + s) * kFragX);
  };
  auto read_w = [&](int parity, int t, int ct) {
    return *reinterpret_cast<const u32x4_t *>(lds_w + (parity & 1) * kStageW + w_frag0 + (ct * TPC + t) * kFragW);
  };

  // One MFMA occupies the matrix pipeline for 32 cycles and the wave issues in order, with no second wave on its SIMD
  // to fill gaps.  So everything else is cut into pieces that fit behind one MFMA each and fenced there: the
  // conversion of the next weight fragment (14 vector instructions in four parts), and one memory instruction per
  // slot -- a fragment read for the next step, a staging store of the next chunk, or a load two chunks ahead.
  uint32_t cv[4];  // the fragment being converted
  auto convert_part = [&](uint32_t d0, uint32_t d1, int part) {
    // sign-extending byte-to-float converts (one instruction per code), high halves of two floats per permute: exact,
    // |q| <= 128 has at most 8 significant bits
    const uint32_t t = part < 2 ? d0 : d1;
    if ((part & 1) == 0) {
      const float f0 = static_cast<float>(static_cast<int8_t>(t & 0xFFu)), f1 = static_cast<float>(static_cast<int8_t>((t >> 8) & 0xFFu));
      cv[part] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
    } else {
      const float f2 = static_cast<float>(static_cast<int8_t>((t >> 16) & 0xFFu)), f3 = static_cast<float>(static_cast<int8_t>(t >> 24));
      cv[part] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2), 0x07060302u);
    }
  };
  bf16x8_t wf;  // converted fragment of the column tile whose MFMAs come next

  // Slot j = 0 .. 15 of step s of chunk ci, whose register set r holds chunk ci + 1 (loaded two chunks ago: the
  // memory round trip under load is longer than one chunk):
  //   j < RT: activation fragment j of the next step           j < CT, s odd: weight codes of the next 32-wide span
  //   j = 8 .. 11, s < 3: staging store of piece 4 s + j - 8     j = 12 .. 15, s < 3: load of that piece of chunk ci + 3
  // The last step's reads address the next chunk's stage, behind the chunk's only barrier.
  auto slot_op = [&](int ci, Staged &r, int s, int j) {
    const int t = s >> 1;
    const bool last = s + 1 == SPC;
    if (j < RT) af[(s + 1) & 1][j] = last ? read_a(ci + 1, 0, j) : read_a(ci, s + 1, j);
    if (j < CT && (s & 1)) wq[(t + 1) & 1][j] = last ? read_w(ci + 1, 0, j) : read_w(ci, t + 1, j);
    if (!last && j >= 8 && j < 12) store_piece(r, ci + 1, 4 * s + j - 8);
    if (!last && j >= 12) load_piece(r, ci + 3, 4 * s + j - 12);
  };
  auto chunk = [&](int ci, Staged &r) {
#pragma unroll
    for (int s = 0; s < SPC; ++s) {
      const int t = s >> 1, a = s & 1;
      if (s + 1 == SPC) lds_barrier();  // staging stores of this chunk visible, every wave done reading this stage
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        // the fragment to convert meanwhile: the next column tile's, or the first one of the following step
        const u32x4_t &nx = ct + 1 < CT ? wq[t & 1][ct + 1] : (a ? wq[(t + 1) & 1][0] : wq[t & 1][0]);
        const int na = ct + 1 < CT ? a : (a ^ 1);
        const uint32_t d0 = nx[2 * na], d1 = nx[2 * na + 1];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          acc[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[s & 1][rt], wf, acc[ct][rt], 0, 0, 0);
          constexpr int kEvery = RT / 4;  // conversion parts per column tile: 4, spread over its RT MFMAs
          if (rt % kEvery == kEvery - 1) convert_part(d0, d1, rt / kEvery);
          slot_op(ci, r, s, ct * RT + rt);
          __builtin_amdgcn_sched_barrier(0);
        }
        wf = __builtin_bit_cast(bf16x8_t, u32x4_t{cv[0], cv[1], cv[2], cv[3]});
      }
    }
  };

  Staged st[2];
#pragma unroll
  for (int i = 0; i < 12; ++i) load_piece(st[0], 0, i);
#pragma unroll
  for (int i = 0; i < 12; ++i) store_piece(st[0], 0, i);
#pragma unroll
  for (int i = 0; i < 12; ++i) load_piece(st[1], 1, i);
#pragma unroll
  for (int i = 0; i < 12; ++i) load_piece(st[0], 2, i);
  lds_barrier();
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) af[0][rt] = read_a(0, 0, rt);
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) wq[0][ct] = read_w(0, 0, ct);
#pragma unroll
  for (int part = 0; part < 4; ++part) convert_part(wq[0][0][0], wq[0][0][1], part);
  wf = __builtin_bit_cast(bf16x8_t, u32x4_t{cv[0], cv[1], cv[2], cv[3]});
  for (int ci = 0; ci < nchunks; ci += 2) {  // K % 128 == 0: an even number of 64-wide chunks
    chunk(ci, st[1]);
    chunk(ci + 1, st[0]);
  }

  // ---- store with the reference's two roundings: bf16(acc), then bf16(t * scale) ----------------------------------
  float scale[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col = col0 + 32 * ct + n;
    scale[ct] = bf16_to_f32(scales[col < N ? col : N - 1]);
  }
  lds_barrier();  // the staging stages are dead from here on
  store_tiles_via_lds<RT, CT, true>(acc, scale, lds + wave * TileStore<CT>::kBytesPerWave, y, row0, col0, M, N, lane,
                                    (N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0);
}


// Four waves, 256 x 256 outputs per tile, every wave 256 rows x 64 columns, like int8_gemm128_kernel<1, 4, 64>, with two
// differences.
// How the operands reach LDS: 16-byte buffer loads that write LDS directly (lane L of an instruction lands at
// base + 16 L), so no operand passes through registers on its way in, there are no staging stores, and three 48 KB
// stages (the chunk in use and two in flight) take the place of two stages and two register sets.
//   Activations, 256 rows x 64 k per chunk: 1 KB block b holds rows 8 b .. 8 b + 7, 128 bytes each (eight lanes read one
//   whole 128-byte row segment); within a row the 16-byte pieces are stored at position piece ^ ((row >> 1) & 7), so the
//   fragment read of 16 consecutive rows at one piece index touches 16 different bank groups.  Wave w loads blocks
//   w, w + 4, ..
//   Weights, 256 columns x 64 k (bytes) per chunk: block b holds columns 16 b .. 16 b + 15, 64 bytes each, pieces at
//   position piece ^ ((column >> 2) & 3).  Wave w loads (and alone reads) blocks 4 w .. 4 w + 3: its own columns.
// How tiles follow each other: one workgroup per CU walks its XCD's tiles, and the chunk pipeline runs across tile
// boundaries -- the loads two chunks ahead simply move on to the next tile's first chunks, so a tile's output
// conversion and stores run while the next tile's first operands are in flight, and no tile starts with an empty
// pipeline.  The output tiles pass through the stage that the next loads will target, hence one extra barrier per tile.
// Fragment contents, conversion and the slot schedule are those of int8_gemm128_kernel.
__global__ __launch_bounds__(256) void int8_gemm_dl_kernel(const uint16_t *__restrict__ x, const int8_t *__restrict__ q,
                                                           const uint16_t *__restrict__ scales, uint16_t *__restrict__ y, int M, int N, int K,
                                                           int n_col_blocks, int n_row_blocks, int cbx) {
  constexpr int RT = 8, CT = 2, CK = 64, SPC = 4, TPC = 2;
  constexpr int kStageX = 256 * 128, kStageW = 256 * 64, kStage = kStageX + kStageW, kStages = 3;
  constexpr int kXLoads = 8, kWLoads = 4;
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kStages * kStage];
  static_assert(kStage >= 4 * TileStore<CT>::kBytesPerWave, "the output tiles fit one stage");
  typedef __attribute__((address_space(3))) void lds_void;

  // ---- this workgroup's tiles: slot sl of XCD blockIdx.x % 8 is column block xcd + 8 (sl % cbx), row block sl / cbx
  const int xcd = blockIdx.x & 7;
  const int stride = gridDim.x >> 3;
  const int slots = cbx * n_row_blocks;
  auto next_slot = [&](int sl) {  // the next slot of this workgroup that names a column block of the matrix (uniform)
    do sl += stride;
    while (sl < slots && xcd + 8 * (sl % cbx) >= n_col_blocks);
    return sl;
  };
  int sl = next_slot(static_cast<int>(blockIdx.x >> 3) - stride);
  if (sl >= slots) return;  // uniform, before any barrier

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int nchunks = K / CK;

  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(q, static_cast<uint32_t>(static_cast<size_t>(N) * K));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));

  // ---- what this lane loads for a tile: activation block w + 4 i, row 8 (w + 4 i) + lane / 8, the piece that belongs at
  // position lane % 8; weight block 4 w + i, column 16 (4 w + i) + lane / 4, the piece that belongs at position lane % 4
  uint32_t xsrc[kXLoads], wsrc[kWLoads];
  const int xpiece = (lane & 7) ^ (((lane >> 4) + 4 * wave) & 7);  // ((row >> 1) & 7) of this lane's rows, the same for every i
  const int wpiece = (lane & 3) ^ ((lane >> 4) & 3);               // ((column >> 2) & 3)
  auto aim_loads_at = [&](int slot_) {
    const int cb = xcd + 8 * (slot_ % cbx), rb = slot_ / cbx;
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      int row = rb * 256 + 8 * (wave + 4 * i) + (lane >> 3);
      row = row < M ? row : M - 1;
      xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + xpiece * 8) * 2);
    }
#pragma unroll
    for (int i = 0; i < kWLoads; ++i) {
      int col = cb * 256 + wave * 64 + 16 * i + (lane >> 2);
      col = col < N ? col : N - 1;
      wsrc[i] = static_cast<uint32_t>(static_cast<size_t>(col) * K + wpiece * 16);
    }
  };
  auto load_piece = [&](int lchunk, uint32_t stage_off, int i) {  // stage_off: byte offset of the receiving stage (uniform)
    if (i < kXLoads)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (lds_void *)(lds + stage_off + (wave + 4 * i) * 1024), 16, xsrc[i],
                                               static_cast<uint32_t>(lchunk) * (CK * 2), 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_void *)(lds + stage_off + kStageX + (4 * wave + (i - kXLoads)) * 1024), 16,
                                               wsrc[i - kXLoads], static_cast<uint32_t>(lchunk) * CK, 0, 0);
  };

  // ---- fragment reads.  Activation fragment (row tile rt, step s = 2 t + a): lane (h, r) reads row 32 rt + r, piece
  // p = 4 t + 2 h + a, stored at position p ^ ((r >> 1) & 7).  Weight fragment (column tile ct, span t): lane (h, c) reads
  // column 64 w + 32 ct + c, piece 2 t + h, stored at position (2 t + h) ^ ((c >> 2) & 3).
  uint32_t a_lane[SPC], w_lane[TPC];
#pragma unroll
  for (int s2 = 0; s2 < SPC; ++s2) {
    const int p = 4 * (s2 >> 1) + 2 * h + (s2 & 1);
    a_lane[s2] = static_cast<uint32_t>(n * 128 + ((p ^ ((n >> 1) & 7)) << 4));
  }
#pragma unroll
  for (int t = 0; t < TPC; ++t)
    w_lane[t] = static_cast<uint32_t>(kStageX + (64 * wave + n) * 64 + (((2 * t + h) ^ ((n >> 2) & 3)) << 4));
  bf16x8_t af[2][RT];
  u32x4_t wq[2][CT];
  auto read_a = [&](uint32_t stage_off, int s2, int rt) {
    return *reinterpret_cast<const bf16x8_t *>(lds + stage_off + a_lane[s2] + rt * 4096);
  };
  auto read_w = [&](uint32_t stage_off, int t, int ct) {
    return *reinterpret_cast<const u32x4_t *>(lds + stage_off + w_lane[t] + ct * 2048);
  };

  uint32_t cv[4];
  auto convert_part = [&](uint32_t d0, uint32_t d1, int part) {
    const uint32_t t = part < 2 ? d0 : d1;
    if ((part & 1) == 0) {
      const float f0 = static_cast<float>(static_cast<int8_t>(t & 0xFFu)), f1 = static_cast<float>(static_cast<int8_t>((t >> 8) & 0xFFu));
      cv[part] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
    } else {
      const float f2 = static_cast<float>(static_cast<int8_t>((t >> 16) & 0xFFu)), f3 = static_cast<float>(static_cast<int8_t>(t >> 24));
      cv[part] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2), 0x07060302u);
    }
  };
  bf16x8_t wf;

  f32x16_t acc[CT][RT];

  // Slot j = 0 .. 15 of step s of a chunk (stage cur; the chunk after it sits in stage nxt; the one after that, chunk
  // lchunk of the tile the loads are aimed at, goes to stage far, which every wave left before the previous barrier):
  //   j < RT: activation fragment j of the next step           j < CT, s odd: weight codes of the next 32-wide span
  //   j = 12 .. 15, s < 3: load 4 s + j - 12 of the chunk two ahead
  auto slot_op = [&](int lchunk, uint32_t cur, uint32_t nxt, uint32_t far, int s2, int j) {
    const int t = s2 >> 1;
    const bool last = s2 + 1 == SPC;
    if (j < RT) af[(s2 + 1) & 1][j] = last ? read_a(nxt, 0, j) : read_a(cur, s2 + 1, j);
    if (j < CT && (s2 & 1)) wq[(t + 1) & 1][j] = last ? read_w(nxt, 0, j) : read_w(cur, t + 1, j);
    if (!last && j >= 12) load_piece(lchunk, far, 4 * s2 + j - 12);
  };
  auto chunk = [&](int lchunk, uint32_t cur, uint32_t nxt, uint32_t far) {
#pragma unroll
    for (int s2 = 0; s2 < SPC; ++s2) {
      const int t = s2 >> 1, a = s2 & 1;
      if (s2 + 1 == SPC) {
        // the next chunk (loaded during the previous one) has landed once at most this chunk's 12 loads are outstanding;
        // behind the barrier every wave is done with this stage (the last step's fragments are in registers)
        asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      }
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const u32x4_t &nx = ct + 1 < CT ? wq[t & 1][ct + 1] : (a ? wq[(t + 1) & 1][0] : wq[t & 1][0]);
        const int na = ct + 1 < CT ? a : (a ^ 1);
        const uint32_t d0 = nx[2 * na], d1 = nx[2 * na + 1];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          acc[ct][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[s2 & 1][rt], wf, acc[ct][rt], 0, 0, 0);
          if (rt % 2 == 1) convert_part(d0, d1, rt / 2);
          slot_op(lchunk, cur, nxt, far, s2, ct * RT + rt);
          __builtin_amdgcn_sched_barrier(0);
        }
        wf = __builtin_bit_cast(bf16x8_t, u32x4_t{cv[0], cv[1], cv[2], cv[3]});
      }
    }
  };

  // ---- pipeline start: the first tile's chunks 0 and 1 (K % 128 == 0: at least two chunks per tile)
  aim_loads_at(sl);
#pragma unroll
  for (int i = 0; i < 12; ++i) load_piece(0, 0, i);
#pragma unroll
  for (int i = 0; i < 12; ++i) load_piece(1, kStage, i);
  int lsl = sl, lchunk = 2;  // where the loads are aimed: tile slot and chunk
  if (lchunk == nchunks) {
    lchunk = 0;
    lsl = next_slot(lsl);
    if (lsl < slots) aim_loads_at(lsl);  // else: keep re-reading the last tile, nobody uses it
  }
  asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) af[0][rt] = read_a(0, 0, rt);
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) wq[0][ct] = read_w(0, 0, ct);
#pragma unroll
  for (int part = 0; part < 4; ++part) convert_part(wq[0][0][0], wq[0][0][1], part);
  wf = __builtin_bit_cast(bf16x8_t, u32x4_t{cv[0], cv[1], cv[2], cv[3]});
  uint32_t cur = 0, nxt = kStage, far = 2 * kStage;

  while (true) {
    const int cb = xcd + 8 * (sl % cbx), rb = sl / cbx;
    const int row0 = rb * 256, col0 = cb * 256 + wave * 64;
    uint16_t scale_raw[CT];  // requested now, needed after the tile's last chunk
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int col = col0 + 32 * ct + n;
      scale_raw[ct] = scales[col < N ? col : N - 1];
    }
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[ct][rt][e] = 0.f;
    for (int ci = 0; ci < nchunks; ++ci) {
      chunk(lchunk, cur, nxt, far);
      const uint32_t tmp = cur;
      cur = nxt;
      nxt = far;
      far = tmp;
      if (++lchunk == nchunks) {  // uniform; once per tile
        lchunk = 0;
        lsl = next_slot(lsl);
        if (lsl < slots) aim_loads_at(lsl);
      }
    }
    // ---- store with the reference's two roundings: bf16(acc), then bf16(t * scale).  The stage just left (far) is free
    // until the next chunk's loads target it; the next tile's first fragments are already in registers.
    float scale[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) scale[ct] = bf16_to_f32(scale_raw[ct]);
    store_tiles_via_lds<RT, CT, true>(acc, scale, lds + far + wave * TileStore<CT>::kBytesPerWave, y, row0, col0, M, N, lane,
                                      (N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0);
    sl = next_slot(sl);
    if (sl >= slots) break;  // uniform
    lds_barrier();  // every wave's output tiles have left the stage before anybody's loads write it
  }
  // the loads aimed past the last tile still write LDS: they must land before the workgroup's LDS is given away
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace

int int8_gemm32(const uint16_t *x, const int8_t *q, const uint16_t *scales, uint16_t *y, int M, int N, int K, hipStream_t stream) {
  if (K % 128 != 0) return E2H_ERR_BAD_SHAPE;
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
  if (big && options().int8_gemm_waves == 0) {
    // one workgroup per CU, an equal share per XCD, each walking its XCD's tiles
    static const int cus = [] {
      int dev = 0, v = 0;
      if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v < 8) v = 256;
      return v;
    }();
    const long long per_xcd = std::min<long long>(cus / 8, static_cast<long long>(cbx) * n_row_blocks);
    hipLaunchKernelGGL(int8_gemm_dl_kernel, dim3(static_cast<unsigned>(8 * per_xcd)), dim3(256), 0, stream, x, q, scales, y, M, N, K,
                       n_col_blocks, n_row_blocks, cbx);
    return launch_status();
  }
  if (big && options().int8_gemm_waves != 8) {
    if (options().int8_gemm_wave_cols == 2)
      hipLaunchKernelGGL((int8_gemm128_kernel<2, 2, 64>), dim3(static_cast<unsigned>(wgs)), dim3(256), 0, stream, x, q, scales, y, M, N, K,
                         n_col_blocks, cbx);
    else
      hipLaunchKernelGGL((int8_gemm128_kernel<1, 4, 64>), dim3(static_cast<unsigned>(wgs)), dim3(256), 0, stream, x, q, scales, y, M, N, K,
                         n_col_blocks, cbx);
    return launch_status();
  }
  if (big)
    hipLaunchKernelGGL((int8_gemm32_kernel<2, 4, 4, 2, 64>), dim3(static_cast<unsigned>(wgs)), dim3(512), 0, stream, x, q, scales, y, M, N, K,
                       n_col_blocks, cbx);
  else
    hipLaunchKernelGGL((int8_gemm32_kernel<2, 4, 2, 2, 128>), dim3(static_cast<unsigned>(wgs)), dim3(512), 0, stream, x, q, scales, y, M, N, K,
                       n_col_blocks, cbx);
  return launch_status();
}

}  // namespace e2h

// int4 group-wise matmul for many rows of x (prefill, scoring), 256 x 256 outputs per workgroup of four waves.
//
// Same contract and data layouts as e2h_int4_mm.hip (torch.ops.aten._weight_int4pack_mm as called by
// linear_forward_int4, reference models/quantize.py:445-453), inner_k_tiles = 8, group size 32 / 64 / 128.
//
// Dequantize-to-bfloat16 form: every weight becomes a bfloat16 value w = bf16( fma(128 + q, s, fma(-136, s, z)) ) on its
// way into the matrix cores (two float32 FMAs: the constant z - 136 s is rounded to float32 once per group, then one FMA
// per weight, then round to nearest even.  Against the single-rounded bf16(s * (q - 8) + z) this is off by at most
// 2^-22 (|z| + 136 |s|) in front of the last rounding: the same bfloat16 value except at near-ties of that rounding
// (one ulp then) and for weights that nearly cancel, |w| << |z - 136 s|), and the products accumulate in float32 -- the
// arithmetic of the kernel the reference calls, up to that difference.  With 256 accumulator registers per lane there is no
// room for per-group partial sums, and none are needed this way: no pass over x for group sums, no accumulator
// prologue, no scaling of accumulators inside the loop.
//
// Main loop, v_mfma_f32_32x32x16_bf16 (A = activations, 32 rows; B = weights, 32 columns; 16 k per instruction), k in
// natural order: lane L = 32 h + n supplies column n0 + n and the eight k values 16 s + 8 h .. + 7 of step s.
//   Activations reach LDS per 64-wide k chunk by 16-byte buffer loads that write LDS directly (lane L of an
//   instruction lands at base + 16 L; no staging registers, no staging stores), three 32 KB stages: the chunk in use and
//   two in flight, one barrier per chunk.  1 KB block b holds rows 8 b .. 8 b + 7, 128 bytes each (eight lanes read one
//   whole row segment); within a row the 16-byte pieces sit at position piece ^ ((row >> 1) & 7), so the fragment read
//   of 16 consecutive rows at one piece index touches 16 different bank groups.  The fragment of lane (h, m) for step
//   s is x[m][16 s + 8 h .. + 7] = piece 2 s + h.
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

template <int G>
__global__ __launch_bounds__(256) void int4_gemm128_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ wp,
                                                           const uint32_t *__restrict__ sz, uint16_t *__restrict__ y, int M, int N, int K,
                                                           int n_col_blocks, int cbx) {
  constexpr int RT = 8, CT = 2;        // 32 x 32 tiles per wave: 256 rows x 64 columns
  constexpr int CK = 64;               // k per staged activation chunk
  constexpr int SPC = CK / 16;         // MFMA steps per chunk
  constexpr int NGRP = 128 / G;        // quantization groups per 128-wide weight block
  constexpr int kStageX = 256 * 128;   // 256 rows x 64 k of bfloat16
  constexpr int kXPieces = 8;          // 256 rows x 8 pieces of 16 bytes per chunk, 256 threads
  static_assert(G == 32 || G == 64 || G == 128, "group sizes of the packed format up to one weight block");
  __shared__ __attribute__((aligned(1024))) uint8_t lds[3 * kStageX];
  static_assert(kStageX >= 4 * TileStore<CT>::kBytesPerWave, "the output tiles reuse a stage");
  typedef __attribute__((address_space(3))) void lds_void;

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

  // ---- what this lane loads: activation block w + 4 i, row 8 (w + 4 i) + lane / 8, the piece that belongs at position
  // lane % 8 (the swizzle term ((row >> 1) & 7) is the same for every i)
  uint32_t xsrc[kXPieces];
  {
    const int xpiece = (lane & 7) ^ (((lane >> 4) + 4 * wave) & 7);
#pragma unroll
    for (int i = 0; i < kXPieces; ++i) {
      int row = row0 + 8 * (wave + 4 * i) + (lane >> 3);
      row = row < M ? row : M - 1;
      xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + xpiece * 8) * 2);
    }
  }

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

  auto load_piece = [&](int ci, uint32_t stage_off, int i) {  // stage_off: byte offset of the stage that receives chunk ci (uniform)
    const int cc = ci < nchunks ? ci : nchunks - 1;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (lds_void *)(lds + stage_off + (wave + 4 * i) * 1024), 16, xsrc[i],
                                             static_cast<uint32_t>(cc) * (CK * 2), 0, 0);
  };
  uint32_t a_lane[SPC];  // lane (h, r), step s: row r, piece 2 s + h at position (2 s + h) ^ ((r >> 1) & 7)
#pragma unroll
  for (int s2 = 0; s2 < SPC; ++s2) a_lane[s2] = static_cast<uint32_t>(n * 128 + (((2 * s2 + h) ^ ((n >> 1) & 7)) << 4));
  bf16x8_t af[RT];  // fragment rt is re-read for the next step right after its last MFMA of this one
  auto read_a = [&](uint32_t stage_off, int s2, int rt) {
    return *reinterpret_cast<const bf16x8_t *>(lds + stage_off + a_lane[s2] + rt * 4096);
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

  // Slot j = 0 .. 15 of step s of chunk ci (half hf of its weight block; stage scur, the next chunk in stage snxt, chunk
  // ci + 2 goes to stage sfar, which every wave left before the previous barrier):
  //   j >= 8 (second column tile, the fragment's last use in this step): activation fragment j - 8 of the next step
  //   s < 2, j = 4 .. 7: load 4 s + j - 4 of chunk ci + 2
  //   s = 2 of a block's first half: the eight weight loads (j < 8) and the (scale, zero) loads (j >= 8) of the next block
  // The last step's fragment reads address the next chunk's stage, behind the chunk's only barrier.
  auto slot_op = [&](int ci, uint32_t scur, uint32_t snxt, uint32_t sfar, WSet &nxt, int hf, int s, int j) {
    const bool last = s + 1 == SPC;
    if (j >= RT) af[j - RT] = last ? read_a(snxt, 0, j - RT) : read_a(scur, s + 1, j - RT);
    if (s < 2 && j >= 4 && j < 8) load_piece(ci + 2, sfar, 4 * s + j - 4);
    if (s == 2 && hf == 0) {
      if (j < 8) load_w(nxt, (ci >> 1) + 1, j);
      if (j >= 8 && j - 8 < CT * NGRP) load_sz(nxt, (ci >> 1) + 1, j - 8);
    }
  };
  // Memory instructions issued after the activation loads of chunk ci + 1 when chunk ci reaches its barrier: this chunk's
  // eight activation loads and one weight block's loads (issued in this chunk or the one before, whichever is a block's
  // first half).  Loads complete in order, so that many may still be outstanding once chunk ci + 1 has landed.
  constexpr int kLoadsBehind = kXPieces + 8 + CT * NGRP;
  auto chunk = [&](int ci, uint32_t scur, uint32_t snxt, uint32_t sfar, const WSet &cur, WSet &nxt, int hf) {
#pragma unroll
    for (int s = 0; s < SPC; ++s) {
      const int sa = 4 * hf + s;
      if (s + 1 == SPC)  // the next chunk has landed; behind the barrier every wave is done reading this stage
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(kLoadsBehind) : "memory");
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
          slot_op(ci, scur, snxt, sfar, nxt, hf, s, ct * RT + rt);
          __builtin_amdgcn_sched_barrier(0);
        }
        wf = __builtin_bit_cast(bf16x8_t, u32x4_t{cv[0], cv[1], cv[2], cv[3]});
      }
    }
  };

  WSet ws[2];
#pragma unroll
  for (int i = 0; i < 8; ++i) load_w(ws[0], 0, i);
#pragma unroll
  for (int i = 0; i < CT * NGRP; ++i) load_sz(ws[0], 0, i);
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) load_piece(0, 0, i);
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) load_piece(1, kStageX, i);
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kXPieces) : "memory");  // the weights of block 0 and chunk 0 are in
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) af[rt] = read_a(0, 0, rt);
#pragma unroll
  for (int j = 0; j < 4; ++j) convert_part(ws[0], 0, 0, j);
  wf = __builtin_bit_cast(bf16x8_t, u32x4_t{cv[0], cv[1], cv[2], cv[3]});
  uint32_t s0 = 0, s1 = kStageX, s2 = 2 * kStageX;  // stage of the chunk in use, of the next one, of the one after
  for (int blk = 0; blk < nblocks; blk += 2) {  // two blocks per trip (K % 256 == 0): the weight register sets are compile-time names
    chunk(2 * blk, s0, s1, s2, ws[0], ws[1], 0);
    chunk(2 * blk + 1, s1, s2, s0, ws[0], ws[1], 1);
    chunk(2 * blk + 2, s2, s0, s1, ws[1], ws[0], 0);
    chunk(2 * blk + 3, s0, s1, s2, ws[1], ws[0], 1);
    const uint32_t t0 = s0;  // four chunks on: the rotation by three stages has advanced by one
    s0 = s1;
    s1 = s2;
    s2 = t0;
  }

  // ---- store: lane (h, n) holds column col0 + 32 ct + n, rows 8 (e / 4) + 4 h + e % 4 of each tile -----------------
  // the loads issued past the last chunk still write LDS: drain them before the stages are reused
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
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

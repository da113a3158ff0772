// int4 group-wise dequant GEMV / skinny GEMM for gfx950, reading the tile-packed checkpoint layout directly.
//
// Replaces torch.ops.aten._weight_int4pack_mm as called by linear_forward_int4
// (reference models/quantize.py:445-453).
//
// Data layout (all in HBM, untouched checkpoint format):
//   packed  int32 [N/8][K/(16*ikt)][32][ikt/2]   word (nTile, kOuter, t, p) holds 8 codes of row
//           n = 8*nTile + t/4: with j = t%4 and k0 = (kOuter*ikt + 2p)*16 the nibbles 0..7 are the codes at
//           k0 + {2j, 2j+8, 16+2j, 24+2j, 2j+1, 2j+9, 17+2j, 25+2j}.
//   sz      bf16  [K/g][N][2]                    (scale, zero) pairs, read as one dword per (group, n).
//   x       bf16  [M][K] row-major,  y bf16 [M][N] row-major.
//
// Mapping to v_mfma_f32_16x16x32_bf16 (A = activations, rows m; B = weights, columns n):
//   lane L = 16*b + c supplies, for column n = n0 + c, the 8 k-values of k-block b.  One packed word is
//   exactly such a fragment: (word >> 4i) & 0x000F000F is the code pair (k0+8i+2j, k0+8i+2j+1), and
//   OR-ing 0x43004300 turns it into the bfloat16 pair (128+q, 128+q') with no arithmetic.  A dot product
//   is invariant under a common permutation of k, so the activation fragment of lane (b, m) is gathered
//   with the same k order (dwords b, b+4, b+8, b+12 of each 64-byte activation segment) and the weights
//   are never re-packed.
//   The scale and zero are applied to the float32 accumulators once per group:
//     y[m,n] += s * sum_k x[m,k]*(128+q[n,k]) + (z - 136*s) * sum_k x[m,k]
//   (the group sums of x come from one extra MFMA against an all-ones fragment, which lands them in the
//   accumulator layout).  bf16*bf16 products are exact in float32, so this is more accurate than a
//   dequantize-to-bf16 kernel.
//
// Work decomposition: a workgroup of 4 waves owns 64*T output columns (each wave T tiles of 16 weight rows),
// 16*MT rows of x and one of S contiguous slices of K.  Per 128-wide k chunk the workgroup stages the
// activation chunk once into LDS (coalesced 16-byte global loads, scattered so that every MFMA fragment is
// one conflict-free ds_read_b128), while every wave streams its own packed weights with 128-bit loads kept
// several chunks ahead in registers.  With S > 1 the slices meet in a workspace: each workgroup stores its
// float32 partial tile, takes a ticket, and the last one to arrive adds the S partials in slice order -- a
// fixed order, so results are deterministic -- and writes bf16.
#include <atomic>

#include "e2h_common.h"
#include "e2h_int4_unpack.h"

namespace e2h {
namespace {

template <int G, int IKT>
struct Int4Geom {
  static constexpr int WORDS = IKT / 2;                  // packed words per lane per k-block
  static constexpr int KBLK = 16 * IKT;                  // k covered by one packed k-block
  static constexpr int CHUNK = (G > KBLK) ? G : KBLK;    // k per pipeline chunk
  static constexpr int NBLK = CHUNK / KBLK;              // packed k-blocks per chunk
  static constexpr int STEPS = CHUNK / 32;               // 32-wide MFMA steps per chunk
  static constexpr int NGRP = CHUNK / G;                 // quantization groups per chunk
  static constexpr int SPG = G / 32;                     // MFMA steps per group
  static constexpr int PPR = CHUNK / 8;                  // 16-byte activation pieces per row per chunk
};

template <int N> struct WordVec;
template <> struct WordVec<1> { typedef uint32_t type; };
template <> struct WordVec<2> { typedef u32x2_t type; };
template <> struct WordVec<4> { typedef u32x4_t type; };

constexpr int kFragBytes = 1024 + 64;   // one MFMA A-fragment block in LDS; the pad skews banks between steps

template <int G, int IKT, int T, int XS>
struct WeightRegs {
  typedef Int4Geom<G, IKT> Geo;
  uint32_t w[T][Geo::STEPS];
  uint32_t sz[T][Geo::NGRP];
  f32x4_t xs[XS > 0 ? XS : 1][Geo::NGRP];  // precomputed group sums of x for the chunk (XS = row tiles), else unused
};

constexpr int kWeightCachePolicy = 2;  // "nt": weights are streamed once, keep them from displacing x and qparams


// Weight prefetch: a ring of NB register buffers per wave, NB - 1 chunks in flight beyond the one being
// consumed (about 8 KB per wave: HBM latency here is well over a microsecond, so a CU needs tens of KB in
// flight).  The main loop is unrolled NB times so that ring slots are compile-time registers.
template <int G, int IKT, int MT, int T, int WN, int WK>
struct Tuning {
  static constexpr int kChunkWords = T * Int4Geom<G, IKT>::STEPS;  // weight registers per chunk
  // few waves per workgroup: deep ring; many waves: the other waves of the SIMD cover the latency
  static constexpr int NB = MT >= 4 ? 2 : (kChunkWords <= 4 ? (WN * WK <= 4 ? 8 : 4) : (kChunkWords <= 8 ? 4 : 2));
  // Activations are staged into LDS one phase (CPP chunks) at a time, a whole phase ahead of their use, so
  // the workgroup meets at a barrier once per phase instead of once per chunk.
  static constexpr int kChunkLds = MT * Int4Geom<G, IKT>::STEPS * kFragBytes;  // one chunk of x in LDS
  static constexpr int kLdsBudget = (WK >= 4 ? 144 : 72) * 1024;               // both stages of all k-groups
  static constexpr int CPP = (WK * 2 * 4 * kChunkLds <= kLdsBudget) ? 4 : ((WK * 2 * 2 * kChunkLds <= kLdsBudget) ? 2 : 1);
  // Loads return in issue order, so waiting for an activation load also waits for every weight load issued
  // before it.  The activation loads of a phase are therefore issued XD phases ahead -- at least as far
  // ahead (in chunks) as the weight ring -- and by the time they are needed everything older has been
  // consumed anyway.
  static constexpr int XD = (NB + CPP - 1) / CPP;
};

// WN = waves that share one activation stream and split the workgroup's columns; WK = number of k-groups
// inside the workgroup (each group = WN waves with its own activation stream over a contiguous part of the
// workgroup's K slice); the k-groups' accumulators are added through LDS at the end.
//
// GATE: the two "tiles" of a wave are the same 16 columns of two weight matrices of equal shape (wp / sz and
// wp2 / sz2, the gate and up projections of a feed-forward block); the epilogue writes
// bf16(bf16(silu(bf16(gate))) * bf16(up)), the rounding points of  F.silu(w1(x)) * w3(x)  on bfloat16 tensors
// (reference models/model.py:343-344).  Both products share one activation stream.
//
// ROPE (one new token per sequence, x row m = sequence m): the product is the fused q | k | v projection; the
// epilogue rounds it to bfloat16, rotates the interleaved pairs of the q and k heads in float32 by the angle of
// position input_pos[0] (reference models/model.py:400-412), and writes q to q_out [B, H, D] and k, v straight
// into the caches [B, Hkv, S, D] at that position (KVCache.update, reference models/model.py:94-104).
//
// PARTIAL: the workgroup's float32 sums over its K slice go to slice blockIdx.y of a row-major [S][M][N] array and the
// launch ends there: no tickets, no meeting of the slices.  The consumer (the residual add + RMSNorm that follows the
// wo and w2 projections of a decoder block, reference models/model.py:279-282) adds the slices in slice order.
enum Epilogue { kPlain = 0, kGate = 1, kRope = 2, kPartial = 3 };

struct RopeArgs {
  const uint16_t *freqs;     // [>= S, D/2, 2] bf16 (cos, sin)
  uint16_t *q_out, *kc, *vc;
  const int64_t *input_pos;  // [1] on the device
  int H, Hkv, S, D;
};

template <int G, int IKT, int MT, int T, int WN, int WK, int EPI = kPlain, bool XSUM = false>
__global__ __launch_bounds__(64 * WN * WK) void int4_skinny_mm_kernel(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ wp, const uint32_t *__restrict__ sz,
    const uint32_t *__restrict__ wp2, const uint32_t *__restrict__ sz2,
    uint16_t *__restrict__ y, float *__restrict__ ws_partial, unsigned *__restrict__ ws_ticket, int M, int N, int K,
    int slabs_in_x, RopeArgs rope, const float *__restrict__ xsum, int xsum_stride) {
  constexpr bool GATE = EPI == kGate;
  static_assert(!GATE || T == 2, "gate mode pairs exactly two weight matrices");
  constexpr int TC = GATE ? 1 : T;  // distinct column tiles per wave
  typedef Int4Geom<G, IKT> Geo;
  typedef WeightRegs<G, IKT, T, XSUM ? MT : 0> wregs_t;
  constexpr int kWavesN = WN;
  constexpr int kGroupThreads = WN * 64;
  constexpr int NB = Tuning<G, IKT, MT, T, WN, WK>::NB;
  constexpr int PD = NB - 1;
  constexpr int CPP = Tuning<G, IKT, MT, T, WN, WK>::CPP;
  constexpr int XD = Tuning<G, IKT, MT, T, WN, WK>::XD;
  constexpr int U = NB > CPP * XD ? NB : CPP * XD;                  // chunks per unrolled loop body
  constexpr int kPieces = 16 * MT * Geo::PPR;                       // 16-byte pieces of x per chunk
  constexpr int kPhasePieces = CPP * kPieces;
  constexpr int kPiecesPerThread = (kPhasePieces + kGroupThreads - 1) / kGroupThreads;
  constexpr int kBufBytes = MT * Geo::STEPS * kFragBytes;           // one activation chunk in fragment order
  constexpr int kStageBytes = CPP * kBufBytes;                      // one phase
  constexpr int kSlots = T * MT * 4;                                // accumulator registers per lane
  constexpr int kXBytes = WK * 2 * kStageBytes;
  constexpr int kRedBytes = (WK - 1) * kWavesN * kSlots * 64 * 4;
  constexpr int kLdsBytes = kXBytes > kRedBytes ? kXBytes : kRedBytes;

  __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsBytes];
  __shared__ unsigned s_ticket;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: everything derived from it stays in SGPRs
  const int wave_n = wave % kWavesN;
  const int kg = wave / kWavesN;          // k-group of this wave
  const int tid_g = tid % kGroupThreads;  // thread index within the k-group
  const int c = lane & 15;  // column of the MFMA tile (weight row within the 16-row tile)
  const int b = lane >> 4;  // k-block of the MFMA
  const int n_tiles8 = N >> 3;
  const int KT = K / Geo::KBLK;
  const int nchunks = K / Geo::CHUNK;
  const int S = gridDim.y;
  const int ks = blockIdx.y;
  // workgroup slice [C0, C1) of the chunks, then this k-group's part [c0, c1) of it
  // (32-bit arithmetic: nchunks < 2^24 and S <= 64 on every path the host takes)
  const int C0 = S == 1 ? 0 : static_cast<int>((static_cast<unsigned>(nchunks) * static_cast<unsigned>(ks)) / static_cast<unsigned>(S));
  const int C1 = S == 1 ? nchunks : static_cast<int>((static_cast<unsigned>(nchunks) * static_cast<unsigned>(ks + 1)) / static_cast<unsigned>(S));
  const int c0 = C0 + ((C1 - C0) * kg) / WK;
  const int c1 = C0 + ((C1 - C0) * (kg + 1)) / WK;
  const int nloc = c1 - c0;
  const int nloc_max = (C1 - C0 + WK - 1) / WK;  // trip count, uniform over the workgroup
  // Column block and row slab of this workgroup.  A few row slabs (decode batches of 33 .. 128 rows) are folded into
  // blockIdx.x so that the slabs of one column block are dispatched together AND land on the same XCD (workgroup
  // i goes to XCD i % 8): the second slab then finds the weights in that XCD's L2 instead of fetching them again.
  const int n_blocks = ((N + 15) / 16 + kWavesN * TC - 1) / (kWavesN * TC);
  int col_block = blockIdx.x, row_slab = blockIdx.z;
  if (slabs_in_x > 1) {
    row_slab = (blockIdx.x >> 3) % slabs_in_x;
    col_block = (blockIdx.x / (8 * slabs_in_x)) * 8 + (blockIdx.x & 7);
    if (col_block >= n_blocks) return;  // padding of the folded grid; uniform over the workgroup, before any barrier
  }
  const int tile16_0 = (col_block * kWavesN + wave_n) * TC;
  const int m_base = row_slab * (16 * MT);
  uint8_t *const xlds = lds + kg * (2 * kStageBytes);

  // ---- addressing: uniform (scalar) base per chunk + constant 32-bit per-lane byte offsets ------------
  uint32_t wlane[T];   // byte offset of this lane's 16 (or 8 / 4) bytes inside chunk 0 of the packed tensor
  uint32_t szlane[T];  // byte offset of this lane's column inside one [N] row of (scale, zero) pairs
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int tcol = tile16_0 + (GATE ? 0 : t);
    int nt8 = 2 * tcol + (c >> 3);
    nt8 = nt8 < n_tiles8 ? nt8 : n_tiles8 - 1;
    wlane[t] = static_cast<uint32_t>((static_cast<size_t>(nt8) * KT * 32 + ((c & 7) * 4 + b)) * Geo::WORDS * 4);
    int ncol = 16 * tcol + c;
    ncol = ncol < N ? ncol : N - 1;
    szlane[t] = static_cast<uint32_t>(ncol) * 4u;
  }
  // Buffer addressing: resource (scalar) + scalar byte offset of the chunk + the lane's constant offset,
  // so a load costs no vector ALU work at all.  Every tensor is smaller than 4 GB (checked on the host).
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(wp, static_cast<uint32_t>(static_cast<size_t>(N) * K / 2));
  const __amdgpu_buffer_rsrc_t sz_rsrc = make_rsrc(sz, static_cast<uint32_t>(static_cast<size_t>(K / G) * N * 4));
  const __amdgpu_buffer_rsrc_t w2_rsrc = make_rsrc(GATE ? wp2 : wp, static_cast<uint32_t>(static_cast<size_t>(N) * K / 2));
  const __amdgpu_buffer_rsrc_t sz2_rsrc = make_rsrc(GATE ? sz2 : sz, static_cast<uint32_t>(static_cast<size_t>(K / G) * N * 4));
  // XSUM: the sums of x over every (row, quantization group) were computed once by a pre-pass, laid out
  // [K/G][xsum_stride] float32; each lane fetches the four rows of its accumulator registers per row tile
  const __amdgpu_buffer_rsrc_t xs_rsrc = make_rsrc(XSUM ? xsum : reinterpret_cast<const float *>(x),
                                                   XSUM ? static_cast<uint32_t>(static_cast<size_t>(K / G) * xsum_stride * 4) : 0u);
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));

  auto load_weights = [&](wregs_t &r, int ci) {
    const uint32_t wchunk = static_cast<uint32_t>(ci) * (Geo::NBLK * 32 * Geo::WORDS * 4);
    const uint32_t szchunk = static_cast<uint32_t>(ci) * Geo::NGRP * N * 4;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const __amdgpu_buffer_rsrc_t wr = (GATE && t == 1) ? w2_rsrc : w_rsrc;
      const __amdgpu_buffer_rsrc_t sr = (GATE && t == 1) ? sz2_rsrc : sz_rsrc;
#pragma unroll
      for (int blk = 0; blk < Geo::NBLK; ++blk) {
        const uint32_t so = wchunk + blk * (32 * Geo::WORDS * 4);
        if constexpr (Geo::WORDS == 4) {
          const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(wr, wlane[t], so, kWeightCachePolicy);
#pragma unroll
          for (int p = 0; p < 4; ++p) r.w[t][blk * 4 + p] = v[p];
        } else if constexpr (Geo::WORDS == 2) {
          const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(wr, wlane[t], so, kWeightCachePolicy);
          r.w[t][blk * 2] = v[0];
          r.w[t][blk * 2 + 1] = v[1];
        } else {
          r.w[t][blk] = __builtin_amdgcn_raw_buffer_load_b32(wr, wlane[t], so, kWeightCachePolicy);
        }
      }
#pragma unroll
      for (int g = 0; g < Geo::NGRP; ++g)
        r.sz[t][g] = __builtin_amdgcn_raw_buffer_load_b32(sr, szlane[t], szchunk + g * N * 4, 0);
    }
    if constexpr (XSUM) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int g = 0; g < Geo::NGRP; ++g) {
          const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(
              xs_rsrc, static_cast<uint32_t>((m_base + 16 * mt + 4 * b) * 4), static_cast<uint32_t>(ci * Geo::NGRP + g) * static_cast<uint32_t>(xsum_stride) * 4u, 0);
          r.xs[mt][g] = __builtin_bit_cast(f32x4_t, v);
        }
    }
  };

  // ---- cooperative activation staging (per k-group) ------------------------------------------------
  // piece p of a phase: chunk q = p / kPieces of the phase; within the chunk row = p' / PPR and 16-byte piece
  // `within` = p' % PPR of that row's CHUNK-wide segment; step s = within / 4, u = within % 4.  Its dword j
  // belongs to lane (b = j, m = row % 16), register u.
  uint32_t xsrc[kPiecesPerThread];  // byte offset of the piece inside chunk 0 of x
  int xdst[kPiecesPerThread];
  int xq[kPiecesPerThread];
#pragma unroll
  for (int i = 0; i < kPiecesPerThread; ++i) {
    const int p = tid_g + i * kGroupThreads;
    const int q = (p / kPieces) < CPP ? (p / kPieces) : CPP - 1;
    const int pc = p % kPieces;
    int row = pc / Geo::PPR;
    const int within = pc % Geo::PPR;
    const int s = within >> 2, u = within & 3;
    xq[i] = q;
    xdst[i] = q * kBufBytes + ((row >> 4) * Geo::STEPS + s) * kFragBytes + (row & 15) * 16 + u * 4;
    row += m_base;
    row = row < M ? row : M - 1;
    xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + within * 8) * 2);
  }
  auto chunk_at = [&](int i) {
    const int ci = c0 + (i < nloc ? i : nloc - 1);
    return ci < C0 ? C0 : ci;  // a group without chunks re-reads the first chunk of the slice
  };
  auto load_x = [&](u32x4_t (&r)[kPiecesPerThread], int phase) {
#pragma unroll
    for (int i = 0; i < kPiecesPerThread; ++i)
      if (kPhasePieces % kGroupThreads == 0 || tid_g + i * kGroupThreads < kPhasePieces)
        r[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xsrc[i], static_cast<uint32_t>(chunk_at(phase * CPP + xq[i])) * (Geo::CHUNK * 2), 0);
  };
  auto store_x = [&](const u32x4_t (&r)[kPiecesPerThread], int parity) {
    uint8_t *buf = xlds + (parity & 1) * kStageBytes;
#pragma unroll
    for (int i = 0; i < kPiecesPerThread; ++i)
      if (kPhasePieces % kGroupThreads == 0 || tid_g + i * kGroupThreads < kPhasePieces) {
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<uint32_t *>(buf + xdst[i] + j * 256) = r[i][j];
      }
  };

  f32x4_t acc[T][MT];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const UnpackConsts uc = unpack_consts();
  const bf16x8_t ones = __builtin_bit_cast(bf16x8_t, u32x4_t{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});

  auto compute_chunk = [&](const wregs_t &r, int parity, int q, uint32_t live) {
    const uint8_t *buf = xlds + (parity & 1) * kStageBytes + q * kBufBytes + lane * 16;
    bf16x8_t xf[MT][Geo::STEPS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int s = 0; s < Geo::STEPS; ++s)
        xf[mt][s] = *reinterpret_cast<const bf16x8_t *>(buf + (mt * Geo::STEPS + s) * kFragBytes);
    // group sums of x, already in accumulator layout (every column holds the same sum)
    f32x4_t xs[MT][Geo::NGRP];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int g = 0; g < Geo::NGRP; ++g) {
        if constexpr (XSUM) {
          xs[mt][g] = r.xs[mt][g];
        } else {
          f32x4_t s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < Geo::SPG; ++s)
            s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[mt][g * Geo::SPG + s], ones, s4, 0, 0, 0);
          xs[mt][g] = s4;
        }
      }
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
      for (int g = 0; g < Geo::NGRP; ++g) {
        f32x4_t part[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) part[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < Geo::SPG; ++s) {
          const bf16x8_t wf = unpack_word(r.w[t][g * Geo::SPG + s], uc);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            part[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[mt][g * Geo::SPG + s], wf, part[mt], 0, 0, 0);
        }
        const uint32_t szw = r.sz[t][g] & live;  // live == 0 turns the chunk into a no-op (scale = zero = 0)
        const float scale = __builtin_bit_cast(float, szw << 16);
        const float zero = __builtin_bit_cast(float, szw & 0xFFFF0000u);
        const float zc = __builtin_fmaf(-136.0f, scale, zero);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float a = acc[t][mt][q];
            a = __builtin_fmaf(scale, part[mt][q], a);
            a = __builtin_fmaf(zc, xs[mt][g][q], a);
            acc[t][mt][q] = a;
          }
        }
      }
    }
  };

  // ---- main pipeline -----------------------------------------------------------------------------
  // The loop body is branch-free so that the compiler can count outstanding loads exactly and never waits
  // for younger prefetches: chunk indices past the end of the group's part are clamped to a valid chunk (the
  // loads hit cache, the arithmetic is neutralised with live = 0), and the trip count is rounded up to U.
  wregs_t ring[NB];
  u32x4_t xstage[XD][kPiecesPerThread];
  int rope_pos = -1;
  float rope_cs[TC], rope_sn[TC];
#pragma unroll
  for (int t = 0; t < TC; ++t) {
    rope_cs[t] = 1.f;
    rope_sn[t] = 0.f;
  }
  if (C1 > C0) {
#pragma unroll
    for (int d = 0; d < XD; ++d) load_x(xstage[d], d);
#pragma unroll
    for (int i = 0; i < PD; ++i) load_weights(ring[i], chunk_at(i));
    if constexpr (EPI == kRope) {
      // the rotation's cos / sin depend on a position read from memory: fetch both now, behind the first
      // weight loads, instead of as two dependent round trips at the very end
      rope_pos = static_cast<int>(rope.input_pos[0]);
#pragma unroll
      for (int t = 0; t < TC; ++t) {
        const int ncol = 16 * (tile16_0 + t) + c;
        if (ncol < N && rope_pos >= 0 && rope_pos < rope.S && ncol < (rope.H + rope.Hkv) * rope.D) {
          const uint32_t f = reinterpret_cast<const uint32_t *>(rope.freqs)[static_cast<size_t>(rope_pos) * (rope.D / 2) + ((ncol % rope.D) >> 1)];
          rope_cs[t] = __builtin_bit_cast(float, f << 16);
          rope_sn[t] = __builtin_bit_cast(float, f & 0xFFFF0000u);
        }
      }
    }
    store_x(xstage[0], 0);
    lds_barrier();
    // invariant at the top of phase ph: LDS stage (ph & 1) holds the activations of phase ph, register set
    // (ph + d) % XD holds (or is still receiving) phase ph + d for d = 1 .. XD-1, set ph % XD is free
    for (int base = 0; base < nloc_max; base += U) {
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const int i = base + j;
        const int phase = i / CPP;
        const uint32_t live = i < nloc ? 0xFFFFFFFFu : 0u;
        if (j % CPP == 0) load_x(xstage[(j / CPP) % XD], phase + XD);
        load_weights(ring[(j + PD) % NB], chunk_at(i + PD));
        compute_chunk(ring[j % NB], phase, j % CPP, live);
        if (j % CPP == CPP - 1) {
          store_x(xstage[(j / CPP + 1) % XD], phase + 1);
          lds_barrier();
        }
      }
    }
  }

  // ---- epilogue 1: add the k-groups of this workgroup through LDS (fixed order) --------------------
  if constexpr (WK > 1) {
    float *red = reinterpret_cast<float *>(lds);
    if (kg > 0) {
      float *mine = red + (static_cast<size_t>(kg - 1) * kWavesN + wave_n) * kSlots * 64 + lane;
#pragma unroll
      for (int t = 0; t < T; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int q = 0; q < 4; ++q) mine[((t * MT + mt) * 4 + q) * 64] = acc[t][mt][q];
    }
    lds_barrier();
    if (kg == 0) {
#pragma unroll
      for (int g2 = 1; g2 < WK; ++g2) {
        const float *other = red + (static_cast<size_t>(g2 - 1) * kWavesN + wave_n) * kSlots * 64 + lane;
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[t][mt][q] += other[((t * MT + mt) * 4 + q) * 64];
      }
    }
  }

  if constexpr (EPI == kPartial) {
    if (kg != 0) return;
    float *out = ws_partial + static_cast<size_t>(ks) * M * N;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const int n = 16 * (tile16_0 + t) + c;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = m_base + 16 * mt + 4 * b + q;
          if (n < N && m < M) out[static_cast<size_t>(m) * N + n] = acc[t][mt][q];
        }
    }
    return;
  }

  // ---- epilogue 2: combine the K slices of different workgroups ------------------------------------
  // Partial tiles and the ticket travel as device-scope relaxed atomics (written through to, and read from,
  // the memory side, so no cache write-back or invalidate is needed); the stores are complete before the
  // ticket is taken, and the loads are issued after it has been observed.
  if (S > 1) {
    const size_t tile_floats = static_cast<size_t>(kWavesN) * kSlots * 64;
    const size_t wg_tile = static_cast<size_t>(row_slab) * n_blocks + col_block;
    if (kg == 0) {
      float *mine = ws_partial + (wg_tile * S + ks) * tile_floats + static_cast<size_t>(wave_n) * kSlots * 64 + lane;
#pragma unroll
      for (int t = 0; t < T; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            __hip_atomic_store(mine + ((t * MT + mt) * 4 + q) * 64, acc[t][mt][q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(ws_ticket + wg_tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != static_cast<unsigned>(S - 1)) return;
    if (tid == 0) __hip_atomic_store(ws_ticket + wg_tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    if (kg == 0) {
      const float *all = ws_partial + wg_tile * S * tile_floats + static_cast<size_t>(wave_n) * kSlots * 64 + lane;
      // slice order 0, 1, .., S-1 for every element, whichever workgroup arrived last.  The loads of four slices are
      // issued before the first addition (one round trip to the memory side instead of one per slice).
      for (int s0 = 0; s0 < S; s0 += 4) {
        float v[4][kSlots];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int s2 = s0 + u < S ? s0 + u : S - 1;  // past the end: a slice read again and not added
#pragma unroll
          for (int slot = 0; slot < kSlots; ++slot)
            v[u][slot] = __hip_atomic_load(all + s2 * tile_floats + slot * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (s0 + u >= S) break;  // uniform
#pragma unroll
          for (int t = 0; t < T; ++t)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const int slot = (t * MT + mt) * 4 + q;
                acc[t][mt][q] = s0 + u == 0 ? v[u][slot] : acc[t][mt][q] + v[u][slot];
              }
        }
      }
    }
  }
  if (kg != 0) return;
  if constexpr (EPI == kRope) {
    const int D = rope.D, H = rope.H, Hkv = rope.Hkv;
    const int pos = rope_pos;
#pragma unroll
    for (int t = 0; t < TC; ++t) {
      const int n = 16 * (tile16_0 + t) + c;
      const int head = n / D, d = n % D;
      const bool in_range = n < N && pos >= 0 && pos < rope.S;
      const bool rotated = head < H + Hkv;
      const float cs = rope_cs[t], sn = rope_sn[t];
      uint16_t *dst;  // element (m = 0) of this lane's column; rows are row_stride apart
      size_t row_stride;
      if (head < H) {
        dst = rope.q_out + static_cast<size_t>(head) * D + d;
        row_stride = static_cast<size_t>(H) * D;
      } else {
        const int hk = rotated ? head - H : head - H - Hkv;
        dst = (rotated ? rope.kc : rope.vc) + (static_cast<size_t>(hk) * rope.S + pos) * D + d;
        row_stride = static_cast<size_t>(Hkv) * rope.S * D;
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = m_base + 16 * mt + 4 * b + q;
          const float own = bf16_round(acc[t][mt][q]);
          const float other = __shfl_xor(own, 1);  // the pair's other column lives in the neighbouring lane
          // even column: x0 * cos - x1 * sin; odd column: x1 * cos + x0 * sin (two rounded products, then the sum)
          const float r = (c & 1) ? own * cs + other * sn : own * cs - other * sn;
          if (in_range && m < M) dst[static_cast<size_t>(m) * row_stride] = f32_to_bf16_rne(rotated ? r : own);
        }
    }
    return;
  }
  if constexpr (GATE) {
    const int n = 16 * tile16_0 + c;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = m_base + 16 * mt + 4 * b + q;
        const float gate = bf16_round(acc[0][mt][q]), up = bf16_round(acc[1][mt][q]);
        const float act = bf16_round(gate / (1.0f + expf(-gate)));
        if (n < N && m < M) y[static_cast<size_t>(m) * N + n] = f32_to_bf16_rne(act * up);
      }
    return;
  }
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int n = 16 * (tile16_0 + t) + c;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = m_base + 16 * mt + 4 * b + q;
        if (n < N && m < M) y[static_cast<size_t>(m) * N + n] = f32_to_bf16_rne(acc[t][mt][q]);
      }
  }
}

// Pre-pass for many-row calls: sums of x over every (row, quantization group), float32, stored group-major
// [K/G][stride] so that the matmul's lanes read four consecutive rows with one 16-byte load.  Reads x once
// (2 M K bytes); the matmul then needs no arithmetic at all for the zero-point term's x side.
template <int G>
__global__ __launch_bounds__(256) void x_group_sums_kernel(const uint16_t *__restrict__ x, float *__restrict__ out, int M, int K, int stride) {
  constexpr int PG = G / 8;  // 16-byte pieces per group (4 .. 32 lanes of one wave)
  const int m = blockIdx.x;
  const uint16_t *row = x + static_cast<size_t>(m) * K;
  for (int piece = threadIdx.x; piece < K / 8; piece += 256) {  // K % G == 0, so whole groups stay inside one wave's lanes
    const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(row + piece * 8);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) s += __builtin_bit_cast(float, raw[j] << 16) + __builtin_bit_cast(float, raw[j] & 0xFFFF0000u);
#pragma unroll
    for (int off = 1; off < PG; off <<= 1) s += __shfl_xor(s, off);
    if ((piece % PG) == 0) out[static_cast<size_t>(piece / PG) * stride + m] = s;
  }
}

struct LaunchArgs {
  const uint16_t *x;
  const int32_t *packed;
  const uint16_t *sz;
  const int32_t *packed2;  // second weight matrix of the gated form, else null
  const uint16_t *sz2;
  uint16_t *y;
  RopeArgs rope;
  const float *xsum;  // group sums of x from the pre-pass (large M), else null
  int xsum_stride;
  float *ws_partial;
  unsigned *ws_ticket;
  int M, N, K, S;
  hipStream_t stream;
};

template <int G, int IKT, int MT, int T, int WN, int WK, int EPI = kPlain, bool XSUM = false>
int launch(const LaunchArgs &a) {
  const int tiles16 = (a.N + 15) / 16;
  constexpr int TC = EPI == kGate ? 1 : T;
  const int n_blocks = (tiles16 + WN * TC - 1) / (WN * TC);
  const int m_chunks = (a.M + 16 * MT - 1) / (16 * MT);
  const int slabs_in_x = (m_chunks > 1 && m_chunks <= 4) ? m_chunks : 1;
  dim3 grid(n_blocks, a.S, m_chunks);
  if (slabs_in_x > 1) grid = dim3(((n_blocks + 7) / 8) * 8 * slabs_in_x, a.S, 1);
  hipLaunchKernelGGL((int4_skinny_mm_kernel<G, IKT, MT, T, WN, WK, EPI, XSUM>), grid, dim3(64 * WN * WK), 0, a.stream, a.x,
                     reinterpret_cast<const uint32_t *>(a.packed), reinterpret_cast<const uint32_t *>(a.sz),
                     reinterpret_cast<const uint32_t *>(a.packed2), reinterpret_cast<const uint32_t *>(a.sz2), a.y,
                     a.ws_partial, a.ws_ticket, a.M, a.N, a.K, slabs_in_x, a.rope, a.xsum, a.xsum_stride);
  return launch_status();
}

// (T, WN, WK) shapes instantiated for the common geometry (inner_k_tiles 8, group size <= 128)
struct Shape {
  int t, wn, wk;
};
constexpr Shape kShapes[] = {{1, 4, 1}, {1, 4, 2}, {1, 2, 2}, {2, 4, 1}, {2, 4, 2}, {2, 2, 2}, {4, 4, 1}};

template <int G, int IKT>
int dispatch_shape(int mt, Shape sh, const LaunchArgs &a) {
  if constexpr (IKT == 8 && G <= 128) {
#define E2H_CASE(TV, WNV, WKV)                                                  \
  if (sh.t == TV && sh.wn == WNV && sh.wk == WKV) {                             \
    if (mt == 1) return launch<G, IKT, 1, TV, WNV, WKV>(a);                     \
    if (mt == 2) return launch<G, IKT, 2, TV, WNV, WKV>(a);                     \
  }
    E2H_CASE(1, 4, 1) E2H_CASE(1, 4, 2) E2H_CASE(1, 2, 2)
    E2H_CASE(2, 4, 1) E2H_CASE(2, 4, 2) E2H_CASE(2, 2, 2) E2H_CASE(4, 4, 1)
#undef E2H_CASE
    if (a.xsum) {
      if (sh.t == 2) return launch<G, IKT, 4, 2, 4, 1, kPlain, true>(a);
      if (sh.t == 1) return launch<G, IKT, 4, 1, 4, 1, kPlain, true>(a);
    }
    if (sh.t == 4) return launch<G, IKT, 4, 4, 4, 1>(a);
    if (sh.t == 2) return launch<G, IKT, 4, 2, 4, 1>(a);
    return launch<G, IKT, 4, 1, 4, 1>(a);
  } else {
    // rarely used geometries: one column tile per wave keeps the register footprint small
    if (mt == 1) return launch<G, IKT, 1, 1, 4, 1>(a);
    if constexpr (G == 256) {
      return launch<G, IKT, 2, 1, 4, 1>(a);  // 256-wide chunks: four row tiles of x would not fit the LDS budget
    } else {
      if (mt == 2) return launch<G, IKT, 2, 1, 4, 1>(a);
      return launch<G, IKT, 4, 1, 4, 1>(a);
    }
  }
}

template <int G>
int dispatch_ikt(int ikt, int mt, Shape sh, const LaunchArgs &a) {
  switch (ikt) {
    case 2: return dispatch_shape<G, 2>(mt, sh, a);
    case 4: return dispatch_shape<G, 4>(mt, sh, a);
    default: return dispatch_shape<G, 8>(mt, sh, a);
  }
}

constexpr size_t kTicketBytes = 64 * 1024;  // 16384 tickets
constexpr int kCUs = 256;

// K slices for the 32-row decode shape (4 column waves x 2 k-groups): narrow matrices split K over S workgroups as long
// as that does not exceed one workgroup per CU and leaves every k-group at least four chunks
inline int decode_k_slices(int blocks, int nchunks) {
  int s = 1;
  while (s < 4 && blocks * s * 2 <= kCUs && nchunks / (2 * s * 2) >= 4) s *= 2;
  return s;
}

}  // namespace
}  // namespace e2h

namespace e2h {
int launch_x_group_sums(const uint16_t *x, float *out, int M, int K, int stride, int groupsize, hipStream_t stream) {
  switch (groupsize) {
    case 32: hipLaunchKernelGGL(x_group_sums_kernel<32>, dim3(M), dim3(256), 0, stream, x, out, M, K, stride); break;
    case 64: hipLaunchKernelGGL(x_group_sums_kernel<64>, dim3(M), dim3(256), 0, stream, x, out, M, K, stride); break;
    case 128: hipLaunchKernelGGL(x_group_sums_kernel<128>, dim3(M), dim3(256), 0, stream, x, out, M, K, stride); break;
    default: return E2H_ERR_BAD_GROUPSIZE;
  }
  return launch_status();
}
}  // namespace e2h

extern "C" int64_t e2h_workspace_bytes(void) { return static_cast<int64_t>(e2h::kTicketBytes) + (int64_t{32} << 20); }

namespace e2h {
namespace {

// strict_scratch: fail with E2H_ERR_SCRATCH_TOO_SMALL where the launch geometry chosen for the shape needs more scratch
// than was passed, instead of falling back to a geometry that needs none
int int4_mm_impl(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros, uint16_t *y, int64_t m, int64_t n,
                 int64_t k, int groupsize, int inner_k_tiles, void *workspace, int64_t workspace_bytes, void *stream,
                 bool strict_scratch) {
  if (!x || !packed || !scales_and_zeros || !y) return E2H_ERR_NULL_POINTER;
  if (groupsize != 32 && groupsize != 64 && groupsize != 128 && groupsize != 256) return E2H_ERR_BAD_GROUPSIZE;
  if (inner_k_tiles != 2 && inner_k_tiles != 4 && inner_k_tiles != 8) return E2H_ERR_BAD_INNER_K_TILES;
  if (m < 1 || n < 8 || k < 1 || (n % 8) != 0 || m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if (k % groupsize != 0) return E2H_ERR_BAD_GROUPSIZE;
  if (k % (16 * inner_k_tiles) != 0) return E2H_ERR_BAD_INNER_K_TILES;
  if (!aligned16(x) || !aligned16(packed) || !aligned16(scales_and_zeros) || (reinterpret_cast<uintptr_t>(y) & 1u))
    return E2H_ERR_MISALIGNED;
  if (workspace && !aligned16(workspace)) return E2H_ERR_MISALIGNED;
  if (n * k / 2 >= (int64_t{1} << 32) || (k / groupsize) * n * 4 >= (int64_t{1} << 32)) return E2H_ERR_BAD_SHAPE;
  LaunchArgs a;
  a.x = x; a.packed = packed; a.sz = scales_and_zeros; a.y = y;
  a.packed2 = nullptr; a.sz2 = nullptr; a.rope = RopeArgs{}; a.xsum = nullptr; a.xsum_stride = 0;
  a.M = static_cast<int>(m); a.N = static_cast<int>(n); a.K = static_cast<int>(k);
  a.stream = static_cast<hipStream_t>(stream);
  // up to 64 rows (decode batches): 32-row workgroups with the K-split shapes, two row slabs per column block
  // when M > 32 (measured 1.4x ... 3.9x faster at M = 64 than the 64-row large-M shape, which has no K split)
  int mt = a.M <= 16 ? 1 : (a.M <= 64 ? 2 : 4);
  if (options().row_tiles) mt = options().row_tiles;
  if (groupsize == 256 && mt == 4) mt = 2;
  const int m_chunks = (a.M + 16 * mt - 1) / (16 * mt);
  const int tiles16 = (a.N + 15) / 16;
  const int chunk = groupsize > 16 * inner_k_tiles ? groupsize : 16 * inner_k_tiles;
  const int nchunks = a.K / chunk;
  const bool wide_ok = inner_k_tiles == 8 && groupsize <= 128;

  // Decomposition: a workgroup = WN column waves x WK k-groups, each wave T tiles of 16 weight rows; S
  // workgroups share a column block along K.
  const bool have_ws = workspace && workspace_bytes >= static_cast<int64_t>(kTicketBytes) + (int64_t{1} << 20);
  // Measured on MI355X: 8 waves per workgroup (4 column waves x 2 k-groups, one tile each) is the best
  // all-round shape -- two waves per SIMD overlap arithmetic with memory waits -- and narrow matrices
  // additionally split K over S workgroups as long as that does not exceed one workgroup per CU (measured: 172
  // column blocks run faster unsplit than as 344 half-length workgroups; 64 blocks run fastest split four ways).
  Shape sh = {1, 4, 1};
  int s = 1;
  if (wide_ok && mt <= 2) {
    sh = Shape{1, 4, 2};
    const int blocks = ((tiles16 + 3) / 4) * m_chunks;
    if (have_ws) s = decode_k_slices(blocks, nchunks);
    // More column blocks than CUs: a wave with two column tiles takes about 1.5x as long as with one, and halving the
    // number of workgroups saves more than that whenever one tile per wave needs a second round of workgroups
    // (measured: 10240 x 8192 at 64 rows 32.9 instead of 44.5 us, 32000 x 8192 71.5 instead of 97.7,
    // 32000 x 4096 at 32 rows 24.8 instead of 27.2; with 16-row workgroups one tile per wave stays ahead)
    if (mt == 2 && blocks > kCUs) sh.t = 2;
  } else if (wide_ok) {
    // many rows of x (prefill, scoring): every weight fragment feeds four row tiles straight from registers;
    // wide column blocks keep the LDS traffic for activation fragments below the MFMA rate
    const int opt_t4 = options().int4_rows_per_wave / 16;
    // two weight tiles per wave once that still leaves a workgroup per CU (measured best of T = 1 / 2 / 4)
    sh = Shape{opt_t4 ? opt_t4 : (static_cast<long long>((tiles16 + 7) / 8) * m_chunks >= kCUs ? 2 : 1), 4, 1};
  }
  const int opt_t = options().int4_rows_per_wave / 16, opt_wk = options().int4_k_groups, opt_wn = options().int4_col_waves;
  if (wide_ok && mt <= 2 && (opt_t || opt_wk || opt_wn)) {
    Shape want = {opt_t ? opt_t : sh.t, opt_wn ? opt_wn : sh.wn, opt_wk ? opt_wk : sh.wk};
    for (const Shape &cand : kShapes)
      if (cand.t == want.t && cand.wn == want.wn && cand.wk == want.wk) sh = cand;
  }
  if (options().int4_k_slices > 0) s = options().int4_k_slices;
  if (s > nchunks) s = nchunks;
  const int n_blocks = (tiles16 + sh.wn * sh.t - 1) / (sh.wn * sh.t);
  if (s > 1) {
    // workspace layout: [tickets | float partial tiles]
    const int64_t tile_floats = static_cast<int64_t>(sh.wn) * sh.t * mt * 4 * 64;
    const int64_t need = static_cast<int64_t>(kTicketBytes) + static_cast<int64_t>(n_blocks) * m_chunks * s * tile_floats * 4;
    if (!have_ws || need > workspace_bytes || static_cast<int64_t>(n_blocks) * m_chunks * 4 > static_cast<int64_t>(kTicketBytes)) {
      if (strict_scratch) return E2H_ERR_SCRATCH_TOO_SMALL;
      s = 1;
    }
  }
  a.S = s;
  a.ws_ticket = reinterpret_cast<unsigned *>(workspace);
  a.ws_partial = workspace ? reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + kTicketBytes) : nullptr;
  // The kernels address x through a 32-bit buffer descriptor: slice M so that every launch sees < 4 GB
  // of activations (and a grid within limits).  Decode-sized calls take a single pass.
  const int64_t rows_by_bytes = ((int64_t{1} << 32) - 1) / (2 * static_cast<int64_t>(a.K));
  const int64_t rows_by_grid = int64_t{65535} * 16 * mt;
  int64_t max_rows = rows_by_bytes < rows_by_grid ? rows_by_bytes : rows_by_grid;
  max_rows -= max_rows % (16 * mt);
  if (max_rows < 16 * mt) return E2H_ERR_BAD_SHAPE;
  // Many rows run on the 128-row kernel (exact products, scale and zero applied to float32 group sums: the arithmetic of
  // every other int4 kernel here, so a row's result does not depend on how many rows share the call).  The 256 x 256
  // kernel that dequantizes to bfloat16 on the way into the matrix cores (the reference kernel's arithmetic, 15-20 %
  // faster at thousands of rows) is taken only on request, option "int4_gemm_tile" = 256, and then for every slice of
  // the call alike.
  const auto takes_256_row_kernel = [&](int64_t) {
    return mt == 4 && wide_ok && !options().int4_no_gemm32 && a.K % 256 == 0 && options().int4_gemm_tile == 256;
  };
  if (mt == 4 && wide_ok && workspace && !options().int4_no_xsum && !takes_256_row_kernel(a.M)) {
    // many rows: the pre-pass keeps (K / g) sums per row in the workspace; slice M so that they fit rather than fall
    // back to the kernels that form the sums themselves (K = 22016 at g = 64: 24k rows per slice with 32 MB)
    const int64_t avail = workspace_bytes - static_cast<int64_t>(kTicketBytes);
    const int64_t rows_by_xsum = avail / (static_cast<int64_t>(a.K / groupsize) * 4) / 256 * 256;
    if (rows_by_xsum >= 2048 && rows_by_xsum < max_rows) max_rows = rows_by_xsum;
  }
  const int m_total = a.M;
  for (int64_t m0 = 0; m0 < m_total; m0 += max_rows) {
    a.x = x + m0 * a.K;
    a.y = y + m0 * a.N;
    a.M = static_cast<int>(m_total - m0 < max_rows ? m_total - m0 : max_rows);
    a.xsum = nullptr;
    if (takes_256_row_kernel(a.M)) {
      const int rc128 = int4_gemm128(a.x, a.packed, a.sz, a.y, a.M, a.N, a.K, groupsize, a.stream);
      if (rc128 != E2H_OK) return rc128;
      continue;
    }
    if (mt == 4 && wide_ok && (sh.t == 1 || sh.t == 2) && workspace && !options().int4_no_xsum) {
      // many rows: one pass over x leaves its group sums in the workspace's partial-tile area (unused here: no K split)
      const int stride = ((a.M + 63) / 64) * 64;
      const int64_t need = static_cast<int64_t>(kTicketBytes) + static_cast<int64_t>(a.K / groupsize) * stride * 4;
      if (need <= workspace_bytes) {
        float *xs = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + kTicketBytes);
        if (launch_x_group_sums(a.x, xs, a.M, a.K, stride, groupsize, a.stream) != E2H_OK) return E2H_ERR_LAUNCH;
        a.xsum = xs;
        a.xsum_stride = stride;
        // 32x32-tile kernel for whole 128-row blocks' worth of work
        // the 128 x 128-output workgroups of that kernel pay off once there are enough of them to fill the chip
        // (measured crossover on the 7B shapes: about 320 workgroups)
        const long long wgs32 = static_cast<long long>((a.M + 127) / 128) * ((a.N + 127) / 128);
        const bool use32 = options().int4_gemm32_min_rows > 0 ? a.M >= options().int4_gemm32_min_rows : wgs32 >= 320;
        if (use32 && !options().int4_no_gemm32) {
          const int rc32 = int4_gemm32(a.x, a.packed, a.sz, a.y, xs, stride, a.M, a.N, a.K, groupsize, a.stream);
          if (rc32 != E2H_OK) return rc32;
          continue;
        }
      }
    }
    int rc;
    switch (groupsize) {
      case 32: rc = dispatch_ikt<32>(inner_k_tiles, mt, sh, a); break;
      case 64: rc = dispatch_ikt<64>(inner_k_tiles, mt, sh, a); break;
      case 128: rc = dispatch_ikt<128>(inner_k_tiles, mt, sh, a); break;
      default: rc = dispatch_ikt<256>(inner_k_tiles, mt, sh, a); break;
    }
    if (rc != E2H_OK) return rc;
  }
  return E2H_OK;
}

// Scratch of the entry point that allocates nothing: split-K tickets followed by float32 partial tiles, the same layout
// e2h_int4_mm expects of a caller's workspace.  Every GPU the library runs on holds its own copy until the process ends.
constexpr size_t kStaticScratchBytes = kTicketBytes + (size_t{8} << 20);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
// device address of `scratch` on each device, resolved on first use (host threads may race to resolve it: they store
// the same value)
std::atomic<void *> g_scratch_ptr[kMaxDevices];

}  // namespace
}  // namespace e2h

extern "C" int e2h_int4_mm(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros,
                           uint16_t *y, int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles,
                           void *workspace, int64_t workspace_bytes, void *stream) {
  return e2h::int4_mm_impl(x, packed, scales_and_zeros, y, m, n, k, groupsize, inner_k_tiles, workspace, workspace_bytes, stream, false);
}

extern "C" int64_t e2h_int4_mm_static_scratch_bytes(void) { return static_cast<int64_t>(e2h::kStaticScratchBytes); }

extern "C" int e2h_int4_mm_static_scratch(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros, uint16_t *y,
                                          int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles, void *stream) {
  using namespace e2h;
  if (!x || !packed || !scales_and_zeros || !y) return E2H_ERR_NULL_POINTER;
  if (m > 64) return E2H_ERR_SCRATCH_TOO_SMALL;  // larger batches keep per-row group sums in scratch: outside the fixed budget
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return E2H_ERR_NO_DEVICE;
  void *scratch_ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!scratch_ptr) {
    // the array's name is a host-side handle, not a device address: resolve it once per device, with that device current.
    // The array starts zeroed when the code object is loaded, and every launch leaves its tickets at zero again.
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return E2H_ERR_NO_DEVICE;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    scratch_ptr = ptr;
  }
  return int4_mm_impl(x, packed, scales_and_zeros, y, m, n, k, groupsize, inner_k_tiles, scratch_ptr,
                      static_cast<int64_t>(kStaticScratchBytes), stream, true);
}

namespace e2h {
namespace {

template <int G>
int dispatch_gate(int mt, int wn, const LaunchArgs &a) {
#define E2H_GATE_CASE(MTV, WNV) \
  if (mt == MTV && wn == WNV) return launch<G, 8, MTV, 2, WNV, 2, kGate>(a);
  E2H_GATE_CASE(1, 4) E2H_GATE_CASE(2, 4) E2H_GATE_CASE(1, 2) E2H_GATE_CASE(2, 2)
  if constexpr (G == 128) {  // three column waves only where the registers suffice
    E2H_GATE_CASE(1, 3) E2H_GATE_CASE(2, 3)
  }
#undef E2H_GATE_CASE
  return E2H_ERR_BAD_SHAPE;
}

}  // namespace
}  // namespace e2h

extern "C" int e2h_int4_mm_silu_gate(const uint16_t *x, const int32_t *packed_gate, const uint16_t *sz_gate,
                                     const int32_t *packed_up, const uint16_t *sz_up, uint16_t *y, int64_t m, int64_t n,
                                     int64_t k, int groupsize, int inner_k_tiles, void *stream) {
  using namespace e2h;
  if (!x || !packed_gate || !sz_gate || !packed_up || !sz_up || !y) return E2H_ERR_NULL_POINTER;
  if (groupsize != 32 && groupsize != 64 && groupsize != 128) return E2H_ERR_BAD_GROUPSIZE;
  if (inner_k_tiles != 8) return E2H_ERR_BAD_INNER_K_TILES;
  if (m < 1 || m > 64 || n < 8 || k < 1 || (n % 8) != 0 || n > INT32_MAX || k > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if (k % groupsize != 0) return E2H_ERR_BAD_GROUPSIZE;
  if (k % 128 != 0) return E2H_ERR_BAD_INNER_K_TILES;
  if (!aligned16(x) || !aligned16(packed_gate) || !aligned16(sz_gate) || !aligned16(packed_up) || !aligned16(sz_up) ||
      (reinterpret_cast<uintptr_t>(y) & 1u))
    return E2H_ERR_MISALIGNED;
  if (n * k / 2 >= (int64_t{1} << 32) || (k / groupsize) * n * 4 >= (int64_t{1} << 32)) return E2H_ERR_BAD_SHAPE;
  LaunchArgs a;
  a.x = x; a.packed = packed_gate; a.sz = sz_gate; a.packed2 = packed_up; a.sz2 = sz_up; a.y = y;
  a.M = static_cast<int>(m); a.N = static_cast<int>(n); a.K = static_cast<int>(k);
  a.S = 1; a.ws_partial = nullptr; a.ws_ticket = nullptr; a.rope = RopeArgs{}; a.xsum = nullptr; a.xsum_stride = 0;
  a.stream = static_cast<hipStream_t>(stream);
  const int mt = a.M <= 16 ? 1 : 2;
  // column waves per workgroup: the count that leaves the fewest idle CUs in the last round of workgroups
  const int tiles16 = (a.N + 15) / 16;
  int wn = options().int4_col_waves;
  if (wn == 3 && groupsize != 128) wn = 0;
  if (wn < 2 || wn > 4) {
    wn = 4;
    double best = -1.0;
    const int slabs = (a.M + 16 * mt - 1) / (16 * mt);  // 33 .. 64 rows run as two 32-row slabs of workgroups
    for (int cand = 4; cand >= 2; --cand) {
      if (cand == 3 && groupsize != 128) continue;  // 6-wave workgroups with two tiles and several groups per chunk spill registers
      const int wgs = ((tiles16 + cand - 1) / cand) * slabs;
      const int rounds = (wgs + kCUs - 1) / kCUs;
      const double fill = static_cast<double>(wgs) / (static_cast<double>(rounds) * kCUs);
      // four-wave workgroups (one wave per SIMD) hide latency worst: they must fill the chip much better to pay off
      // (measured on 2 x 22016 x 8192 at 64 rows: 119 us with two column waves, 100 us with four)
      if (fill > best + (cand == 2 ? 0.25 : 0.05)) { best = fill; wn = cand; }
    }
  }
  switch (groupsize) {
    case 32: return dispatch_gate<32>(mt, wn, a);
    case 64: return dispatch_gate<64>(mt, wn, a);
    default: return dispatch_gate<128>(mt, wn, a);
  }
}

extern "C" int e2h_int4_mm_rope_kv(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros,
                                   const uint16_t *freqs_cis, uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache,
                                   const int64_t *input_pos, int64_t batch, int64_t n_head, int64_t n_kv_head,
                                   int64_t head_dim, int64_t cache_len, int64_t k, int groupsize, int inner_k_tiles,
                                   void *stream) {
  using namespace e2h;
  if (!x || !packed || !scales_and_zeros || !freqs_cis || !q_out || !k_cache || !v_cache || !input_pos) return E2H_ERR_NULL_POINTER;
  if (groupsize != 32 && groupsize != 64 && groupsize != 128) return E2H_ERR_BAD_GROUPSIZE;
  if (inner_k_tiles != 8) return E2H_ERR_BAD_INNER_K_TILES;
  if (batch < 1 || batch > 64 || n_head < 1 || n_kv_head < 1 || head_dim < 2 || (head_dim % 2) != 0 || cache_len < 1 || k < 1)
    return E2H_ERR_BAD_SHAPE;
  const int64_t n = (n_head + 2 * n_kv_head) * head_dim;
  if ((n % 8) != 0 || n > INT32_MAX || k > INT32_MAX || cache_len > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if (k % groupsize != 0) return E2H_ERR_BAD_GROUPSIZE;
  if (k % 128 != 0) return E2H_ERR_BAD_INNER_K_TILES;
  if (!aligned16(x) || !aligned16(packed) || !aligned16(scales_and_zeros) || (reinterpret_cast<uintptr_t>(freqs_cis) & 3u) ||
      (reinterpret_cast<uintptr_t>(q_out) & 1u) || (reinterpret_cast<uintptr_t>(k_cache) & 1u) || (reinterpret_cast<uintptr_t>(v_cache) & 1u) ||
      (reinterpret_cast<uintptr_t>(input_pos) & 7u))
    return E2H_ERR_MISALIGNED;
  if (n * k / 2 >= (int64_t{1} << 32) || (k / groupsize) * n * 4 >= (int64_t{1} << 32)) return E2H_ERR_BAD_SHAPE;
  LaunchArgs a;
  a.x = x; a.packed = packed; a.sz = scales_and_zeros; a.packed2 = nullptr; a.sz2 = nullptr; a.y = nullptr;
  a.rope = RopeArgs{freqs_cis, q_out, k_cache, v_cache, input_pos, static_cast<int>(n_head), static_cast<int>(n_kv_head),
                    static_cast<int>(cache_len), static_cast<int>(head_dim)};
  a.M = static_cast<int>(batch); a.N = static_cast<int>(n); a.K = static_cast<int>(k);
  a.S = 1; a.ws_partial = nullptr; a.ws_ticket = nullptr; a.xsum = nullptr; a.xsum_stride = 0;
  a.stream = static_cast<hipStream_t>(stream);
  const bool two = a.M > 16;
  // 32-row workgroups: two column tiles per wave once one tile per wave would need more workgroups than CUs
  // (as in e2h_int4_mm; batches of 33 .. 64 rows run two row slabs per column block)
  const int tiles16 = (a.N + 15) / 16;
  const int opt_t = options().int4_rows_per_wave / 16;
  const bool wide = two && (opt_t ? opt_t == 2 : ((tiles16 + 3) / 4) * ((a.M + 31) / 32) > kCUs);
  switch (groupsize) {
    case 32: return wide ? launch<32, 8, 2, 2, 4, 2, kRope>(a) : two ? launch<32, 8, 2, 1, 4, 2, kRope>(a) : launch<32, 8, 1, 1, 4, 2, kRope>(a);
    case 64: return wide ? launch<64, 8, 2, 2, 4, 2, kRope>(a) : two ? launch<64, 8, 2, 1, 4, 2, kRope>(a) : launch<64, 8, 1, 1, 4, 2, kRope>(a);
    default: return wide ? launch<128, 8, 2, 2, 4, 2, kRope>(a) : two ? launch<128, 8, 2, 1, 4, 2, kRope>(a) : launch<128, 8, 1, 1, 4, 2, kRope>(a);
  }
}

namespace e2h {
namespace {

// shape checks shared by the two entry points below; returns the number of K slices (>= 1) or a negative status
int partial_slices_for(int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles) {
  if (groupsize != 32 && groupsize != 64 && groupsize != 128) return E2H_ERR_BAD_GROUPSIZE;
  if (inner_k_tiles != 8) return E2H_ERR_BAD_INNER_K_TILES;
  if (m < 1 || m > 64 || n < 8 || k < 1 || (n % 8) != 0 || n > INT32_MAX || k > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if (k % groupsize != 0) return E2H_ERR_BAD_GROUPSIZE;
  if (k % 128 != 0) return E2H_ERR_BAD_INNER_K_TILES;
  if (n * k / 2 >= (int64_t{1} << 32) || (k / groupsize) * n * 4 >= (int64_t{1} << 32)) return E2H_ERR_BAD_SHAPE;
  const int mt = m <= 16 ? 1 : 2;
  const int m_chunks = static_cast<int>((m + 16 * mt - 1) / (16 * mt));
  const int tiles16 = static_cast<int>((n + 15) / 16);
  const int nchunks = static_cast<int>(k / 128);
  int s = decode_k_slices(((tiles16 + 3) / 4) * m_chunks, nchunks);
  if (options().int4_k_slices > 0) s = options().int4_k_slices;
  if (s > nchunks) s = nchunks;
  return s;
}

}  // namespace
}  // namespace e2h

extern "C" int e2h_int4_mm_partial_slices(int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles) {
  return e2h::partial_slices_for(m, n, k, groupsize, inner_k_tiles);
}

extern "C" int e2h_int4_mm_partials(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros, float *partials,
                                    int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles, int slices, void *stream) {
  using namespace e2h;
  if (!x || !packed || !scales_and_zeros || !partials) return E2H_ERR_NULL_POINTER;
  const int want = partial_slices_for(m, n, k, groupsize, inner_k_tiles);
  if (want < 0) return want;
  if (slices != want) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(packed) || !aligned16(scales_and_zeros) || (reinterpret_cast<uintptr_t>(partials) & 3u)) return E2H_ERR_MISALIGNED;
  LaunchArgs a;
  a.x = x; a.packed = packed; a.sz = scales_and_zeros; a.packed2 = nullptr; a.sz2 = nullptr; a.y = nullptr;
  a.rope = RopeArgs{}; a.xsum = nullptr; a.xsum_stride = 0;
  a.M = static_cast<int>(m); a.N = static_cast<int>(n); a.K = static_cast<int>(k);
  a.S = slices; a.ws_partial = partials; a.ws_ticket = nullptr;
  a.stream = static_cast<hipStream_t>(stream);
  const bool two = a.M > 16;
  switch (groupsize) {
    case 32: return two ? launch<32, 8, 2, 1, 4, 2, kPartial>(a) : launch<32, 8, 1, 1, 4, 2, kPartial>(a);
    case 64: return two ? launch<64, 8, 2, 1, 4, 2, kPartial>(a) : launch<64, 8, 1, 1, 4, 2, kPartial>(a);
    default: return two ? launch<128, 8, 2, 1, 4, 2, kPartial>(a) : launch<128, 8, 1, 1, 4, 2, kPartial>(a);
  }
}

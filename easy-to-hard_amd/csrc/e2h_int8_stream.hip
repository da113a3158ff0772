// int8 per-channel dequant GEMV / skinny GEMM / GEMM, streaming version (K % 128 == 0, 16-byte aligned rows).
//
// Replaces  F.linear(x, weight.to(bf16)) * scales  (reference models/quantize.py:428-429).
//
//   q int8 [N][K] row-major (checkpoint layout), scales bf16 [N], x bf16 [M][K], y bf16 [M][N].
//
// Same pipeline as the int4 kernel: a workgroup = WN column waves x WK k-groups, each wave T tiles of 16 weight
// rows and 16*MT rows of x; S workgroups may split K.  Lane L = 16*b + c of v_mfma_f32_16x16x32_bf16 owns weight row
// n0 + c; per 64-wide half chunk it loads the 16 consecutive bytes k = 64h + 16b .. +15 (one buffer_load_dwordx4):
// bytes 0..7 feed MFMA step 2h, bytes 8..15 step 2h + 1.  The matching activation fragment is 16 contiguous bytes of
// x, staged per k-group into LDS one phase at a time in fragment order.  int8 -> bf16 is exact (sign-extending byte
// convert, keep the high half).  No per-group arithmetic: the float32 accumulators run over all of K and the epilogue
// reproduces the reference's two roundings, bf16(acc) then bf16(t * scale).
#include "e2h_common.h"

namespace e2h {
namespace {

constexpr int kChunk = 128;             // k per pipeline chunk
constexpr int kSteps = 4;               // MFMA steps per chunk
constexpr int kPPR = kChunk / 8;        // 16-byte activation pieces per row per chunk
constexpr int kFragBytes = 1024 + 64;   // one fragment block in LDS (+ pad)

__device__ __forceinline__ uint32_t pack_bf16_pair_exact(float lo, float hi) {
  return (__builtin_bit_cast(uint32_t, lo) >> 16) | (__builtin_bit_cast(uint32_t, hi) & 0xFFFF0000u);
}

__device__ __forceinline__ bf16x8_t bytes_to_bf16x8(uint32_t d0, uint32_t d1) {
  u32x4_t u;
  u[0] = pack_bf16_pair_exact(static_cast<float>(static_cast<int8_t>(d0)), static_cast<float>(static_cast<int8_t>(d0 >> 8)));
  u[1] = pack_bf16_pair_exact(static_cast<float>(static_cast<int8_t>(d0 >> 16)), static_cast<float>(static_cast<int8_t>(d0 >> 24)));
  u[2] = pack_bf16_pair_exact(static_cast<float>(static_cast<int8_t>(d1)), static_cast<float>(static_cast<int8_t>(d1 >> 8)));
  u[3] = pack_bf16_pair_exact(static_cast<float>(static_cast<int8_t>(d1 >> 16)), static_cast<float>(static_cast<int8_t>(d1 >> 24)));
  return __builtin_bit_cast(bf16x8_t, u);
}

template <int MT, int T, int WN, int WK>
struct Tuning8 {
  static constexpr int NB = (MT >= 4 || T >= 2) ? 2 : 4;                       // ring of weight chunks (2 KB per tile each)
  static constexpr int kChunkLds = MT * kSteps * kFragBytes;
  static constexpr int kLdsBudget = (WK >= 4 ? 144 : 72) * 1024;
  static constexpr int CPP = (WK * 2 * 4 * kChunkLds <= kLdsBudget) ? 4 : ((WK * 2 * 2 * kChunkLds <= kLdsBudget) ? 2 : 1);
  static constexpr int XD = (NB + CPP - 1) / CPP;
};

template <int T>
struct WeightRegs8 {
  u32x4_t w[T][2];
};

// Epilogues of the decode step (one launch each, at most 64 rows, no K split over workgroups):
// kGate8: the wave's two tiles are the same 16 columns of two weight matrices (q / scales and q2 / scales2, the gate
//   and up projections of a feed-forward block); stores bf16(bf16(silu(g)) * u) with g, u the two linears' bfloat16
//   outputs -- the rounding points of F.silu(w1(x)) * w3(x) on bfloat16 tensors (reference models/model.py:343-344).
// kRope8: the product is the fused q | k | v projection of ONE new token per sequence (row m = sequence m); the
//   bfloat16 output is rotated in float32 by the angle of position input_pos[0] (interleaved pairs, reference
//   models/model.py:400-412); q goes to q_out [B, H, D], k and v into the caches [B, Hkv, S, D] at that position
//   (KVCache.update, reference models/model.py:94-104).
// kPartial8: the workgroup's float32 sums over its K slice (unscaled) go to slice blockIdx.y of a row-major [S][M][N]
// array and the launch ends there; the residual add + RMSNorm that follows adds the slices in order and applies the
// column scales with the reference's two roundings.
enum Epilogue8 { kPlain8 = 0, kGate8 = 1, kRope8 = 2, kPartial8 = 3 };

struct Rope8Args {
  const uint16_t *freqs;     // [>= S, D/2, 2] bf16 (cos, sin)
  uint16_t *q_out, *kc, *vc;
  const int64_t *input_pos;  // [1] on the device
  int H, Hkv, S, D;
};

template <int MT, int T, int WN, int WK, int EPI = kPlain8>
__global__ __launch_bounds__(64 * WN * WK) void int8_stream_mm_kernel(const uint16_t *__restrict__ x, const int8_t *__restrict__ q,
                                                                      const uint16_t *__restrict__ scales, const int8_t *__restrict__ q2,
                                                                      const uint16_t *__restrict__ scales2, uint16_t *__restrict__ y,
                                                                      float *__restrict__ ws_partial, unsigned *__restrict__ ws_ticket,
                                                                      int M, int N, int K, Rope8Args rope) {
  constexpr bool GATE = EPI == kGate8;
  static_assert(!GATE || T == 2, "gate mode pairs exactly two weight matrices");
  static_assert(EPI != kRope8 || T == 1, "the rotary epilogue handles one column tile per wave");
  constexpr int TC = GATE ? 1 : T;  // distinct column tiles per wave
  typedef Tuning8<MT, T, WN, WK> Tune;
  constexpr int NB = Tune::NB, PD = NB - 1, CPP = Tune::CPP, XD = Tune::XD;
  constexpr int U = NB > CPP * XD ? NB : CPP * XD;
  constexpr int kGroupThreads = WN * 64;
  constexpr int kPieces = 16 * MT * kPPR;
  constexpr int kPhasePieces = CPP * kPieces;
  constexpr int kPiecesPerThread = (kPhasePieces + kGroupThreads - 1) / kGroupThreads;
  constexpr int kBufBytes = MT * kSteps * kFragBytes;
  constexpr int kStageBytes = CPP * kBufBytes;
  constexpr int kSlots = T * MT * 4;
  constexpr int kXBytes = WK * 2 * kStageBytes;
  constexpr int kRedBytes = (WK - 1) * WN * kSlots * 64 * 4;
  constexpr int kLdsBytes = kXBytes > kRedBytes ? kXBytes : kRedBytes;

  __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsBytes];
  __shared__ unsigned s_ticket;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_n = wave % WN;
  const int kg = wave / WN;
  const int tid_g = tid % kGroupThreads;
  const int c = lane & 15;
  const int b = lane >> 4;
  const int nchunks = K / kChunk;
  const int S = gridDim.y;
  const int ks = blockIdx.y;
  const int C0 = static_cast<int>((static_cast<long long>(nchunks) * ks) / S);
  const int C1 = static_cast<int>((static_cast<long long>(nchunks) * (ks + 1)) / S);
  const int c0 = C0 + ((C1 - C0) * kg) / WK;
  const int c1 = C0 + ((C1 - C0) * (kg + 1)) / WK;
  const int nloc = c1 - c0;
  const int nloc_max = (C1 - C0 + WK - 1) / WK;
  const int tile16_0 = (blockIdx.x * WN + wave_n) * TC;
  const int m_base = blockIdx.z * (16 * MT);
  uint8_t *const xlds = lds + kg * (2 * kStageBytes);

  uint32_t wlane[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int n = 16 * (tile16_0 + (GATE ? 0 : t)) + c;
    n = n < N ? n : N - 1;
    wlane[t] = static_cast<uint32_t>(static_cast<size_t>(n) * K + 16 * b);
  }
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(q, static_cast<uint32_t>(static_cast<size_t>(N) * K));
  const __amdgpu_buffer_rsrc_t w2_rsrc = make_rsrc(GATE ? q2 : q, static_cast<uint32_t>(static_cast<size_t>(N) * K));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, static_cast<uint32_t>(static_cast<size_t>(M) * K * 2));

  auto load_weights = [&](WeightRegs8<T> &r, int ci) {
    const uint32_t so = static_cast<uint32_t>(ci) * kChunk;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const __amdgpu_buffer_rsrc_t wr = (GATE && t == 1) ? w2_rsrc : w_rsrc;
      r.w[t][0] = __builtin_amdgcn_raw_buffer_load_b128(wr, wlane[t], so, 2);
      r.w[t][1] = __builtin_amdgcn_raw_buffer_load_b128(wr, wlane[t], so + 64, 2);
    }
  };

  // activation staging: piece `within` (0..15) of a row's 128-wide chunk covers k = 8*within .. +7, which is the
  // fragment of lane block b = (within % 8) / 2 in MFMA step 2 * (within / 8) + within % 2
  uint32_t xsrc[kPiecesPerThread];
  int xdst[kPiecesPerThread];
  int xq[kPiecesPerThread];
#pragma unroll
  for (int i = 0; i < kPiecesPerThread; ++i) {
    const int p = tid_g + i * kGroupThreads;
    const int qc = (p / kPieces) < CPP ? (p / kPieces) : CPP - 1;
    const int pc = p % kPieces;
    int row = pc / kPPR;
    const int within = pc % kPPR;
    const int s = 2 * (within >> 3) + (within & 1), bb = (within & 7) >> 1;
    xq[i] = qc;
    xdst[i] = qc * kBufBytes + ((row >> 4) * kSteps + s) * kFragBytes + (bb * 16 + (row & 15)) * 16;
    row += m_base;
    row = row < M ? row : M - 1;
    xsrc[i] = static_cast<uint32_t>((static_cast<size_t>(row) * K + within * 8) * 2);
  }
  auto chunk_at = [&](int i) {
    const int ci = c0 + (i < nloc ? i : nloc - 1);
    return ci < C0 ? C0 : ci;
  };
  auto load_x = [&](u32x4_t (&r)[kPiecesPerThread], int phase) {
#pragma unroll
    for (int i = 0; i < kPiecesPerThread; ++i)
      if (kPhasePieces % kGroupThreads == 0 || tid_g + i * kGroupThreads < kPhasePieces)
        r[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xsrc[i], static_cast<uint32_t>(chunk_at(phase * CPP + xq[i])) * (kChunk * 2), 0);
  };
  auto store_x = [&](const u32x4_t (&r)[kPiecesPerThread], int parity) {
    uint8_t *buf = xlds + (parity & 1) * kStageBytes;
#pragma unroll
    for (int i = 0; i < kPiecesPerThread; ++i)
      if (kPhasePieces % kGroupThreads == 0 || tid_g + i * kGroupThreads < kPhasePieces)
        *reinterpret_cast<u32x4_t *>(buf + xdst[i]) = r[i];
  };

  f32x4_t acc[T][MT];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  auto compute_chunk = [&](const WeightRegs8<T> &r, int parity, int qc, uint32_t live) {
    const uint8_t *buf = xlds + (parity & 1) * kStageBytes + qc * kBufBytes + lane * 16;
    bf16x8_t xf[MT][kSteps];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int s = 0; s < kSteps; ++s) xf[mt][s] = *reinterpret_cast<const bf16x8_t *>(buf + (mt * kSteps + s) * kFragBytes);
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // live == 0 (padding iteration): zero weights contribute nothing
        const bf16x8_t w0 = bytes_to_bf16x8(r.w[t][h][0] & live, r.w[t][h][1] & live);
        const bf16x8_t w1 = bytes_to_bf16x8(r.w[t][h][2] & live, r.w[t][h][3] & live);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[mt][2 * h], w0, acc[t][mt], 0, 0, 0);
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[mt][2 * h + 1], w1, acc[t][mt], 0, 0, 0);
        }
      }
    }
  };

  WeightRegs8<T> ring[NB];
  u32x4_t xstage[XD][kPiecesPerThread];
  int rope_pos = -1;
  float rope_cs = 1.f, rope_sn = 0.f;
  if (C1 > C0) {
#pragma unroll
    for (int d = 0; d < XD; ++d) load_x(xstage[d], d);
#pragma unroll
    for (int i = 0; i < PD; ++i) load_weights(ring[i], chunk_at(i));
    if constexpr (EPI == kRope8) {
      // cos / sin depend on a position read from memory: fetch both behind the first weight loads instead of as two
      // dependent round trips at the very end
      rope_pos = static_cast<int>(rope.input_pos[0]);
      const int ncol = 16 * tile16_0 + c;
      if (ncol < N && rope_pos >= 0 && rope_pos < rope.S && ncol < (rope.H + rope.Hkv) * rope.D) {
        const uint32_t f = reinterpret_cast<const uint32_t *>(rope.freqs)[static_cast<size_t>(rope_pos) * (rope.D / 2) + ((ncol % rope.D) >> 1)];
        rope_cs = __builtin_bit_cast(float, f << 16);
        rope_sn = __builtin_bit_cast(float, f & 0xFFFF0000u);
      }
    }
    store_x(xstage[0], 0);
    lds_barrier();
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

  if constexpr (WK > 1) {
    float *red = reinterpret_cast<float *>(lds);
    if (kg > 0) {
      float *mine = red + (static_cast<size_t>(kg - 1) * WN + wave_n) * kSlots * 64 + lane;
#pragma unroll
      for (int t = 0; t < T; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int r = 0; r < 4; ++r) mine[((t * MT + mt) * 4 + r) * 64] = acc[t][mt][r];
    }
    lds_barrier();
    if (kg == 0) {
#pragma unroll
      for (int g2 = 1; g2 < WK; ++g2) {
        const float *other = red + (static_cast<size_t>(g2 - 1) * WN + wave_n) * kSlots * 64 + lane;
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][mt][r] += other[((t * MT + mt) * 4 + r) * 64];
      }
    }
  }

  if constexpr (EPI == kPartial8) {
    if (kg != 0) return;
    float *out = ws_partial + static_cast<size_t>(ks) * M * N;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const int n = 16 * (tile16_0 + t) + c;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = m_base + 16 * mt + 4 * b + r;
          if (n < N && m < M) out[static_cast<size_t>(m) * N + n] = acc[t][mt][r];
        }
    }
    return;
  }

  if (S > 1) {
    const size_t tile_floats = static_cast<size_t>(WN) * kSlots * 64;
    const size_t wg_tile = static_cast<size_t>(blockIdx.z) * gridDim.x + blockIdx.x;
    if (kg == 0) {
      float *mine = ws_partial + (wg_tile * S + ks) * tile_floats + static_cast<size_t>(wave_n) * kSlots * 64 + lane;
#pragma unroll
      for (int t = 0; t < T; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            __hip_atomic_store(mine + ((t * MT + mt) * 4 + r) * 64, acc[t][mt][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(ws_ticket + wg_tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != static_cast<unsigned>(S - 1)) return;
    if (tid == 0) __hip_atomic_store(ws_ticket + wg_tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (kg == 0) {
      const float *all = ws_partial + wg_tile * S * tile_floats + static_cast<size_t>(wave_n) * kSlots * 64 + lane;
      // the loads of four slices are issued before the first addition (one round trip to the memory side instead of
      // one per slice); the additions keep the slice order
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
              for (int r = 0; r < 4; ++r) {
                const int slot = (t * MT + mt) * 4 + r;
                acc[t][mt][r] = s0 + u == 0 ? v[u][slot] : acc[t][mt][r] + v[u][slot];
              }
        }
      }
    }
  }
  if (kg != 0) return;
  if constexpr (EPI == kRope8) {
    const int n = 16 * tile16_0 + c;
    const float scale = bf16_to_f32(scales[n < N ? n : N - 1]);
    const int D = rope.D, H = rope.H, Hkv = rope.Hkv;
    const int head = n / D, d = n % D;
    const int pos = rope_pos;
    const bool in_range = n < N && pos >= 0 && pos < rope.S;
    const bool rotated = head < H + Hkv;
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
      for (int r = 0; r < 4; ++r) {
        const int m = m_base + 16 * mt + 4 * b + r;
        const float own = bf16_round(bf16_round(acc[0][mt][r]) * scale);  // the linear's bfloat16 output
        const float other = __shfl_xor(own, 1);                           // the pair's other column lives in the neighbouring lane
        // even column: x0 * cos - x1 * sin; odd column: x1 * cos + x0 * sin (two rounded products, then the sum)
        const float rot = (c & 1) ? own * rope_cs + other * rope_sn : own * rope_cs - other * rope_sn;
        if (in_range && m < M) dst[static_cast<size_t>(m) * row_stride] = f32_to_bf16_rne(rotated ? rot : own);
      }
    return;
  }
  if constexpr (GATE) {
    const int n = 16 * tile16_0 + c;
    const float s_gate = bf16_to_f32(scales[n < N ? n : N - 1]), s_up = bf16_to_f32(scales2[n < N ? n : N - 1]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m_base + 16 * mt + 4 * b + r;
        const float gate = bf16_round(bf16_round(acc[0][mt][r]) * s_gate), up = bf16_round(bf16_round(acc[1][mt][r]) * s_up);
        const float act = bf16_round(gate / (1.0f + expf(-gate)));
        if (n < N && m < M) y[static_cast<size_t>(m) * N + n] = f32_to_bf16_rne(act * up);
      }
    return;
  }
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int n = 16 * (tile16_0 + t) + c;
    const float scale = bf16_to_f32(scales[n < N ? n : N - 1]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m_base + 16 * mt + 4 * b + r;
        if (n < N && m < M) {
          const float lin = bf16_round(acc[t][mt][r]);                              // F.linear output in bfloat16
          y[static_cast<size_t>(m) * N + n] = f32_to_bf16_rne(lin * scale);        // * self.scales
        }
      }
  }
}

struct Args8 {
  const uint16_t *x;
  const int8_t *q;
  const uint16_t *scales;
  const int8_t *q2 = nullptr;       // second weight matrix of the gated form
  const uint16_t *scales2 = nullptr;
  Rope8Args rope = {};
  uint16_t *y;
  float *ws_partial;
  unsigned *ws_ticket;
  int M, N, K, S;
  hipStream_t stream;
};

template <int MT, int T, int WN, int WK, int EPI = kPlain8>
int launch8(const Args8 &a) {
  const int tiles16 = (a.N + 15) / 16;
  constexpr int TC = EPI == kGate8 ? 1 : T;
  dim3 grid((tiles16 + WN * TC - 1) / (WN * TC), a.S, (a.M + 16 * MT - 1) / (16 * MT));
  hipLaunchKernelGGL((int8_stream_mm_kernel<MT, T, WN, WK, EPI>), grid, dim3(64 * WN * WK), 0, a.stream, a.x, a.q, a.scales, a.q2,
                     a.scales2, a.y, a.ws_partial, a.ws_ticket, a.M, a.N, a.K, a.rope);
  return launch_status();
}

constexpr size_t kTicketBytes8 = 64 * 1024;
constexpr int kCUs8 = 256;

// K slices for the 16- and 32-row decode shapes (4 column waves x 2 k-groups), as in the int4 kernel
inline int decode_k_slices8(int blocks, int nchunks) {
  int s = 1;
  while (s < 4 && blocks * s * 2 <= kCUs8 && nchunks / (2 * s * 2) >= 4) s *= 2;
  return s;
}

// rows per workgroup (in 16-row tiles) of the decode shapes, 0 where a call takes another kernel
inline int decode_row_tiles8(int M, int N) {
  const int tiles16 = (N + 15) / 16;
  if (M <= 16) return 1;
  if (M <= 32) return 2;
  if (M <= 64 && (tiles16 + 3) / 4 < kCUs8) return 2;
  return 0;
}

int partial_slices8_for(int64_t m, int64_t n, int64_t k) {
  if (m < 1 || m > 64 || n < 8 || (n % 8) != 0 || k < 128 || (k % 128) != 0 || n > INT32_MAX || k > INT32_MAX || n * k >= (int64_t{1} << 32))
    return E2H_ERR_BAD_SHAPE;
  const int mt = decode_row_tiles8(static_cast<int>(m), static_cast<int>(n));
  if (mt == 0) return E2H_ERR_BAD_SHAPE;
  const int m_chunks = static_cast<int>((m + 16 * mt - 1) / (16 * mt));
  const int tiles16 = static_cast<int>((n + 15) / 16);
  const int nchunks = static_cast<int>(k / kChunk);
  int s = decode_k_slices8(((tiles16 + 3) / 4) * m_chunks, nchunks);
  if (options().int8_k_slices > 0) s = options().int8_k_slices;
  if (s > nchunks) s = nchunks;
  return s;
}

}  // namespace

// Streaming int8 matmul; the caller has checked pointers and that K % 128 == 0 with 16-byte aligned x and q.
int int8_stream_mm(const uint16_t *x, const int8_t *q, const uint16_t *scales, uint16_t *y, int M, int N, int K, void *workspace,
                   int64_t workspace_bytes, hipStream_t stream) {
  Args8 a;
  a.q = q; a.scales = scales; a.N = N; a.K = K; a.stream = stream;
  const int tiles16 = (N + 15) / 16;
  // 33 ... 64 rows: the 64-row shape has no K split, so narrow matrices (fewer column blocks than CUs) run as
  // two 32-row slabs with the K-split shapes instead (measured 2.5x ... 3x faster at N = 4096, slower at N >= 11008)
  int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  if (M > 32 && M <= 64 && (tiles16 + 3) / 4 < kCUs8) mt = 2;
  if (options().row_tiles) mt = options().row_tiles;
  const int m_chunks = (M + 16 * mt - 1) / (16 * mt);
  const int nchunks = K / kChunk;
  const bool have_ws = workspace && workspace_bytes >= static_cast<int64_t>(kTicketBytes8) + (int64_t{1} << 20);
  int t = 1, wk = 2, s = 1;
  if (mt == 4) {
    wk = 1;
    t = (static_cast<long long>((tiles16 + 7) / 8) * m_chunks >= kCUs8) ? 2 : 1;
  } else {
    const int blocks = ((tiles16 + 3) / 4) * m_chunks;
    if (have_ws) s = decode_k_slices8(blocks, nchunks);
    // more column blocks than CUs: two column tiles per wave halve the number of workgroups and cost less than a
    // second round of them (measured: 32000 x 4096 at 32 rows 42.4 instead of 46.6 us, at 16 rows 34.6 instead of
    // 38.2; 12288 x 4096 at 64 rows, two slabs, 30.1 instead of 37.3)
    if (blocks > kCUs8) t = 2;
  }
  if (options().int8_rows_per_wave == 16 || options().int8_rows_per_wave == 32) t = options().int8_rows_per_wave / 16;
  if (options().int8_k_groups == 1 || options().int8_k_groups == 2) wk = options().int8_k_groups;
  if (options().int8_k_slices > 0) s = options().int8_k_slices;
  if (mt == 4) wk = 1;
  if (s > nchunks) s = nchunks;
  const int n_blocks = (tiles16 + 4 * t - 1) / (4 * t);
  if (s > 1) {
    const int64_t tile_floats = static_cast<int64_t>(4) * t * mt * 4 * 64;
    const int64_t need = static_cast<int64_t>(kTicketBytes8) + static_cast<int64_t>(n_blocks) * m_chunks * s * tile_floats * 4;
    if (!have_ws || need > workspace_bytes || static_cast<int64_t>(n_blocks) * m_chunks * 4 > static_cast<int64_t>(kTicketBytes8)) s = 1;
  }
  a.S = s;
  a.ws_ticket = reinterpret_cast<unsigned *>(workspace);
  a.ws_partial = workspace ? reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + kTicketBytes8) : nullptr;
  const int64_t rows_by_bytes = ((int64_t{1} << 32) - 1) / (2 * static_cast<int64_t>(K));
  const int64_t rows_by_grid = int64_t{65535} * 16 * mt;
  int64_t max_rows = rows_by_bytes < rows_by_grid ? rows_by_bytes : rows_by_grid;
  max_rows -= max_rows % (16 * mt);
  if (max_rows < 16 * mt) return E2H_ERR_BAD_SHAPE;
  for (int64_t m0 = 0; m0 < M; m0 += max_rows) {
    a.x = x + m0 * K;
    a.y = y + m0 * N;
    a.M = static_cast<int>(M - m0 < max_rows ? M - m0 : max_rows);
    int rc;
    const long long wgs32 = static_cast<long long>((a.M + 127) / 128) * ((N + 127) / 128);
    const bool use32 = options().int4_gemm32_min_rows > 0 ? a.M >= options().int4_gemm32_min_rows : wgs32 >= 320;
    if (mt == 4 && use32 && !options().int4_no_gemm32 && static_cast<int64_t>(N) * K < (int64_t{1} << 32)) {
      rc = int8_gemm32(a.x, q, scales, a.y, a.M, N, K, stream);  // many rows: 32x32-tile kernels, no K split, no scratch
      if (rc != E2H_OK) return rc;
      continue;
    }
    if (mt == 1) rc = t == 2 ? (wk == 2 ? launch8<1, 2, 4, 2>(a) : launch8<1, 2, 4, 1>(a)) : (wk == 2 ? launch8<1, 1, 4, 2>(a) : launch8<1, 1, 4, 1>(a));
    else if (mt == 2) rc = t == 2 ? (wk == 2 ? launch8<2, 2, 4, 2>(a) : launch8<2, 2, 4, 1>(a)) : (wk == 2 ? launch8<2, 1, 4, 2>(a) : launch8<2, 1, 4, 1>(a));
    else rc = t == 2 ? launch8<4, 2, 4, 1>(a) : launch8<4, 1, 4, 1>(a);
    if (rc != E2H_OK) return rc;
  }
  return E2H_OK;
}

}  // namespace e2h

extern "C" int e2h_int8_mm_silu_gate(const uint16_t *x, const int8_t *q_gate, const uint16_t *scales_gate, const int8_t *q_up,
                                     const uint16_t *scales_up, uint16_t *y, int64_t m, int64_t n, int64_t k, void *stream) {
  using namespace e2h;
  if (!x || !q_gate || !scales_gate || !q_up || !scales_up || !y) return E2H_ERR_NULL_POINTER;
  if (m < 1 || m > 64 || n < 1 || k < 128 || (k % 128) != 0 || n > INT32_MAX || k > INT32_MAX || n * k >= (int64_t{1} << 32)) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(q_gate) || !aligned16(q_up) || (reinterpret_cast<uintptr_t>(scales_gate) & 1u) ||
      (reinterpret_cast<uintptr_t>(scales_up) & 1u) || (reinterpret_cast<uintptr_t>(y) & 1u))
    return E2H_ERR_MISALIGNED;
  Args8 a;
  a.x = x; a.q = q_gate; a.scales = scales_gate; a.q2 = q_up; a.scales2 = scales_up; a.y = y;
  a.ws_partial = nullptr; a.ws_ticket = nullptr;
  a.M = static_cast<int>(m); a.N = static_cast<int>(n); a.K = static_cast<int>(k); a.S = 1;
  a.stream = static_cast<hipStream_t>(stream);
  return a.M <= 16 ? launch8<1, 2, 4, 2, kGate8>(a) : launch8<2, 2, 4, 2, kGate8>(a);
}

extern "C" int e2h_int8_mm_rope_kv(const uint16_t *x, const int8_t *q, const uint16_t *scales, const uint16_t *freqs_cis, uint16_t *q_out,
                                   uint16_t *k_cache, uint16_t *v_cache, const int64_t *input_pos, int64_t batch, int64_t n_head,
                                   int64_t n_kv_head, int64_t head_dim, int64_t cache_len, int64_t k, void *stream) {
  using namespace e2h;
  if (!x || !q || !scales || !freqs_cis || !q_out || !k_cache || !v_cache || !input_pos) return E2H_ERR_NULL_POINTER;
  if (batch < 1 || batch > 64 || n_head < 1 || n_kv_head < 1 || head_dim < 2 || (head_dim % 2) != 0 || cache_len < 1 || k < 128 || (k % 128) != 0)
    return E2H_ERR_BAD_SHAPE;
  const int64_t n = (n_head + 2 * n_kv_head) * head_dim;
  if (n > INT32_MAX || k > INT32_MAX || cache_len > INT32_MAX || n * k >= (int64_t{1} << 32)) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(q) || (reinterpret_cast<uintptr_t>(scales) & 1u) || (reinterpret_cast<uintptr_t>(freqs_cis) & 3u) ||
      (reinterpret_cast<uintptr_t>(q_out) & 1u) || (reinterpret_cast<uintptr_t>(k_cache) & 1u) || (reinterpret_cast<uintptr_t>(v_cache) & 1u) ||
      (reinterpret_cast<uintptr_t>(input_pos) & 7u))
    return E2H_ERR_MISALIGNED;
  Args8 a;
  a.x = x; a.q = q; a.scales = scales; a.y = nullptr;
  a.rope = Rope8Args{freqs_cis, q_out, k_cache, v_cache, input_pos, static_cast<int>(n_head), static_cast<int>(n_kv_head),
                     static_cast<int>(cache_len), static_cast<int>(head_dim)};
  a.ws_partial = nullptr; a.ws_ticket = nullptr;
  a.M = static_cast<int>(batch); a.N = static_cast<int>(n); a.K = static_cast<int>(k); a.S = 1;
  a.stream = static_cast<hipStream_t>(stream);
  return a.M <= 16 ? launch8<1, 1, 4, 2, kRope8>(a) : launch8<2, 1, 4, 2, kRope8>(a);
}

extern "C" int e2h_int8_mm_partial_slices(int64_t m, int64_t n, int64_t k) { return e2h::partial_slices8_for(m, n, k); }

extern "C" int e2h_int8_mm_partials(const uint16_t *x, const int8_t *q, float *partials, int64_t m, int64_t n, int64_t k, int slices,
                                    void *stream) {
  using namespace e2h;
  if (!x || !q || !partials) return E2H_ERR_NULL_POINTER;
  const int want = partial_slices8_for(m, n, k);
  if (want < 0) return want;
  if (slices != want) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(q) || (reinterpret_cast<uintptr_t>(partials) & 3u)) return E2H_ERR_MISALIGNED;
  Args8 a;
  a.x = x; a.q = q; a.scales = nullptr; a.q2 = nullptr; a.scales2 = nullptr; a.y = nullptr;
  a.rope = Rope8Args{};
  a.ws_partial = partials; a.ws_ticket = nullptr;
  a.M = static_cast<int>(m); a.N = static_cast<int>(n); a.K = static_cast<int>(k); a.S = slices;
  a.stream = static_cast<hipStream_t>(stream);
  return decode_row_tiles8(a.M, a.N) == 1 ? launch8<1, 1, 4, 2, kPartial8>(a) : launch8<2, 1, 4, 2, kPartial8>(a);
}

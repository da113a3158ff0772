// int4 group-wise dequant GEMV for decode batches (M <= 64) on activations handed over in matrix-core operand order.
//
// Replaces torch.ops.aten._weight_int4pack_mm as called by linear_forward_int4 (reference models/quantize.py:445-453)
// for the one-token-per-sequence steps of the decode loop (reference inference_generate.py:123-157), where every
// quantized linear is a stream over its weights with a few rows of activations.  The activations arrive "staged"
// (layout in e2h_staged.h), written by e2h_int4_stage_x or directly by the kernel that produces them.
//
// Arithmetic per output: y[m,n] = sum_g s[g,n] * P[m,n,g] + sum_g (z[g,n] - 136 s[g,n]) * X[m,g] with
// P = sum_k x[m,k] (128 + q[n,k]) over the group (exact products, float32 accumulation in the matrix cores) and X the
// group sum of x taken from the staged buffer.  The second sum is a small float32 matrix product over the groups
// (v_mfma_f32_16x16x4_f32, four groups per instruction).
//
// Decomposition: a workgroup is eight waves that split K (each wave a contiguous run of at most C 128-wide chunks of
// the workgroup's K slice) and all work on the same T tiles of 16 weight rows.  No wave shares anything with another
// until the end: weights, qparams and activation operands go straight from memory into registers; there is no barrier
// and no LDS traffic before the last chunk is done.  The code is straight-line over the C chunks with every load at a
// fixed place in the instruction stream (weights DW chunks ahead, activation operands DX chunks ahead, pinned with
// scheduling barriers: left alone, the compiler's scheduler sinks each load to its first use).  The eight partial
// tiles meet once in LDS; wave w adds and finishes the (column tile, row tile) units w, w + 8, .. in k order, a fixed
// order, so results are deterministic.  S workgroups may split K further (partial epilogue only): their float32 sums
// go to slice s of a [S][M][N] array for the consumer to add in slice order.
//
// Measured on MI355X at 32 rows, 7B shapes (the kernel this replaces in brackets): 12288 x 4096 10.5 us (13.5),
// 4096 x 4096 6.0 (8.9), 4096 x 11008 10.5 (13.6), gated 2 x 11008 x 4096 15.9 (19.5).  Timed by omission on
// 12288 x 4096: launch + first round trip + meeting + stores 4.0 us, arithmetic 0.5, the weight stream 3.2 (25 MB, the
// HBM rate), the activation operands 2.9 (every CU reads all 256 KB of them from its L2).
#include "e2h_common.h"
#include "e2h_int4_unpack.h"
#include "e2h_staged.h"

namespace e2h {
namespace {

constexpr int kWaves = 8;
constexpr int kNt = 2;  // "nt" cache policy: weights are streamed once
constexpr int kCUs = 256;

enum StagedEpilogue { kStPlain = 0, kStGate = 1, kStRope = 2, kStPartial = 3, kStArgmax = 4 };

struct StagedRope {
  const uint16_t *freqs;     // [>= S, D/2, 2] bf16 (cos, sin)
  uint16_t *q_out, *kc, *vc;
  const int64_t *input_pos;  // [1] on the device
  int H, Hkv, S, D;
};

struct StagedArgs {
  const uint8_t *frag;  // staged activations
  const float *sums;
  const uint32_t *wp, *sz, *wp2, *sz2;
  uint16_t *y;          // bf16 [M][N] (plain, gate; may be null for gate when only the staged result is wanted)
  float *partials;      // f32 [S][M][N] (partial)
  unsigned long long *cand;  // [column blocks][M] (arg-max): per row the best (value key << 32 | ~column) of the block's columns
  StagedOut out;        // gate: the result in staged form for the next linear (frag null: not wanted)
  int M, Mpad, N, K;
  int slabs, col_blocks;
  StagedRope rope;
};

// G group size; MT row tiles of 16 per workgroup; T weight tiles of 16 rows per workgroup (GATE: T/2 of each matrix);
// C chunks a wave has at most; DW / DX prefetch distance of weights / activation operands in chunks.
template <int G, int MT, int T, int C, int DW, int DX, int EPI>
__global__ __launch_bounds__(64 * kWaves) void int4_staged_mm_kernel(const StagedArgs a) {
  constexpr bool GATE = EPI == kStGate;
  static_assert(!GATE || T % 2 == 0, "gate mode pairs the tiles of two matrices");
  constexpr int TC = GATE ? T / 2 : T;     // distinct column tiles per workgroup
  constexpr int NGRP = 128 / G;            // groups per 128-wide chunk
  constexpr int SPG = G / 32;              // MFMA steps per group
  constexpr int R = (C * NGRP + 3) / 4;    // float32 MFMAs of the zero-point term per (tile, row tile)
  constexpr int kUnits = TC * MT;          // (column tile, row tile) pairs, each finished by one wave
  constexpr int kUnitsPerWave = (kUnits + kWaves - 1) / kWaves;
  constexpr int kAccFloats = T * MT * 4 * 64;

  __shared__ __attribute__((aligned(16))) float red[kWaves * kAccFloats];
  __shared__ unsigned long long unit_best[EPI == kStArgmax ? kUnits : 1][16];  // arg-max: per unit and row of its tile

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int kg = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave = k part
  const int c = lane & 15, b = lane >> 4;
  const int N = a.N, K = a.K, M = a.M;
  const int n_tiles8 = N >> 3;
  const int KT = K >> 7;  // packed k-blocks (inner_k_tiles = 8) = chunks
  const int S = gridDim.y, ks = blockIdx.y;
  const int C0 = static_cast<int>((static_cast<unsigned>(KT) * static_cast<unsigned>(ks)) / static_cast<unsigned>(S));
  const int C1 = static_cast<int>((static_cast<unsigned>(KT) * static_cast<unsigned>(ks + 1)) / static_cast<unsigned>(S));
  const int c0 = C0 + ((C1 - C0) * kg) / kWaves;
  const int c1 = C0 + ((C1 - C0) * (kg + 1)) / kWaves;
  const int nloc = c1 - c0;  // <= C (the host picks C)
  // Column block and row slab.  With two row slabs (33 .. 64 rows) the slabs of a column block sit 8 workgroups apart:
  // workgroup i runs on XCD i % 8, so the second slab finds the weights in the same L2.
  int col_block = blockIdx.x, slab = 0;
  if (a.slabs > 1) {
    slab = (blockIdx.x >> 3) % a.slabs;
    col_block = (blockIdx.x / (8 * a.slabs)) * 8 + (blockIdx.x & 7);
    if (col_block >= a.col_blocks) return;  // padding of the folded grid; uniform, before any barrier
  }
  const int tile16_0 = col_block * TC;
  const int m_base = slab * (16 * MT);
  const uint32_t row_block = static_cast<uint32_t>(a.Mpad) * 64u;  // bytes of one k segment of all rows

  uint32_t wlane[T], szlane[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int tcol = tile16_0 + (GATE ? t % TC : t);
    int nt8 = 2 * tcol + (c >> 3);
    nt8 = nt8 < n_tiles8 ? nt8 : n_tiles8 - 1;
    wlane[t] = static_cast<uint32_t>((static_cast<size_t>(nt8) * KT * 32 + ((c & 7) * 4 + b)) * 16);
    int ncol = 16 * tcol + c;
    ncol = ncol < N ? ncol : N - 1;
    szlane[t] = static_cast<uint32_t>(ncol) * 4u;
  }
  const uint32_t xlane = static_cast<uint32_t>((m_base + c) * 64 + 16 * b);  // lane (b, m = c) of row tile 0
  const uint32_t w_bytes = static_cast<uint32_t>(static_cast<size_t>(N) * K / 2);
  const uint32_t sz_bytes = static_cast<uint32_t>(static_cast<size_t>(K / G) * N * 4);
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(a.wp, w_bytes);
  const __amdgpu_buffer_rsrc_t sz_rsrc = make_rsrc(a.sz, sz_bytes);
  const __amdgpu_buffer_rsrc_t w2_rsrc = make_rsrc(GATE ? a.wp2 : a.wp, w_bytes);
  const __amdgpu_buffer_rsrc_t sz2_rsrc = make_rsrc(GATE ? a.sz2 : a.sz, sz_bytes);
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(a.frag, static_cast<uint32_t>(static_cast<size_t>(K / 32) * row_block));
  const __amdgpu_buffer_rsrc_t xs_rsrc = make_rsrc(a.sums, static_cast<uint32_t>(static_cast<size_t>(KT) * a.Mpad * 32));

  struct WRegs {
    u32x4_t w[T];
    uint32_t sz[T][NGRP];
  };
  struct XRegs {
    u32x4_t x[MT][4];
  };
  auto chunk_at = [&](int i) {
    const int ci = c0 + (i < nloc ? i : nloc - 1);
    return ci < C0 ? C0 : ci;  // a wave without chunks re-reads the slice's first chunk (its results are scaled by zero)
  };
  auto load_x = [&](XRegs &r, int ci) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int s = 0; s < 4; ++s)
        r.x[mt][s] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xlane + mt * 1024, static_cast<uint32_t>(ci * 4 + s) * row_block, 0);
  };
  auto load_w = [&](WRegs &r, int ci) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const bool second = GATE && t >= TC;
      r.w[t] = __builtin_amdgcn_raw_buffer_load_b128(second ? w2_rsrc : w_rsrc, wlane[t], static_cast<uint32_t>(ci) * 512u, kNt);
#pragma unroll
      for (int g = 0; g < NGRP; ++g)
        r.sz[t][g] = __builtin_amdgcn_raw_buffer_load_b32(second ? sz2_rsrc : sz_rsrc, szlane[t], static_cast<uint32_t>(ci * NGRP + g) * static_cast<uint32_t>(N) * 4u, 0);
    }
  };

  f32x4_t acc[T][MT];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const UnpackConsts uc = unpack_consts();

  auto compute_chunk = [&](const WRegs &r, const XRegs &rx, uint32_t live) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
      for (int g = 0; g < NGRP; ++g) {
        f32x4_t part[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) part[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < SPG; ++s) {
          const bf16x8_t wf = unpack_word(r.w[t][g * SPG + s], uc);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            part[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, rx.x[mt][g * SPG + s]), wf, part[mt], 0, 0, 0);
        }
        const float scale = __builtin_bit_cast(float, (r.sz[t][g] & live) << 16);  // live == 0: the chunk adds nothing
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[t][mt][q] = __builtin_fmaf(scale, part[mt][q], acc[t][mt][q]);
      }
    }
  };

  // RoPE epilogue: the rotation's cos / sin depend on a position read from memory; both are fetched now, behind the
  // first weight loads, for the units this wave will finish
  int rope_pos = -1;
  float rope_cs[kUnitsPerWave], rope_sn[kUnitsPerWave];
#pragma unroll
  for (int u = 0; u < kUnitsPerWave; ++u) {
    rope_cs[u] = 1.f;
    rope_sn[u] = 0.f;
  }

  if (C1 > C0) {
    // ---- the zero-point term: four groups per float32 MFMA, lane (b, .) owns group 4 r + b of the wave's run -----------
    // Its operands are requested first and used right after the first chunks have been requested: loads return in issue
    // order, so waiting for them does not wait for the chunks.
    const int ngroups = nloc * NGRP;
    u32x4_t xs_raw[R][MT][NGRP == 1 ? 2 : 1];
    uint32_t zsz[R][T];
    bool zlive[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int gi = 4 * r + b;  // group of this lane within the wave's run
      zlive[r] = gi < ngroups;
      const int gcl = zlive[r] ? gi : 0;
      int chunk = c0 + gcl / NGRP;
      chunk = chunk < C1 ? chunk : C1 - 1;
      const int sub = gcl % NGRP;
      // chunk and sub differ between lanes: everything goes into the vector offset
      const uint32_t so = static_cast<uint32_t>(chunk) * static_cast<uint32_t>(a.Mpad) * 32u;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        // the 128 / NGRP values of the group: 8 / NGRP sums of 16
        const uint32_t off = so + static_cast<uint32_t>((m_base + 16 * mt + c) * 32 + sub * (32 / NGRP));
        if constexpr (NGRP == 1) {
          xs_raw[r][mt][0] = __builtin_amdgcn_raw_buffer_load_b128(xs_rsrc, off, 0, 0);
          xs_raw[r][mt][1] = __builtin_amdgcn_raw_buffer_load_b128(xs_rsrc, off + 16, 0, 0);
        } else if constexpr (NGRP == 2) {
          xs_raw[r][mt][0] = __builtin_amdgcn_raw_buffer_load_b128(xs_rsrc, off, 0, 0);
        } else {
          const u32x2_t lo = __builtin_amdgcn_raw_buffer_load_b64(xs_rsrc, off, 0, 0);
          xs_raw[r][mt][0] = u32x4_t{lo[0], lo[1], 0u, 0u};
        }
      }
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const bool second = GATE && t >= TC;
        zsz[r][t] = __builtin_amdgcn_raw_buffer_load_b32(second ? sz2_rsrc : sz_rsrc,
                                                         szlane[t] + static_cast<uint32_t>(chunk * NGRP + sub) * static_cast<uint32_t>(N) * 4u, 0, 0);
      }
    }
    WRegs wr[C];
    XRegs xr[C];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < (DW > DX ? DW : DX); ++i) {
      if (i < DW && i < C) load_w(wr[i], chunk_at(i));
      if (i < DX && i < C) load_x(xr[i], chunk_at(i));
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (EPI == kStRope) {
      rope_pos = static_cast<int>(a.rope.input_pos[0]);
#pragma unroll
      for (int u = 0; u < kUnitsPerWave; ++u) {
        const int unit = kg + u * kWaves;
        const int ncol = 16 * (tile16_0 + unit / MT) + c;
        if (unit < kUnits && ncol < N && rope_pos >= 0 && rope_pos < a.rope.S && ncol < (a.rope.H + a.rope.Hkv) * a.rope.D) {
          const uint32_t f = reinterpret_cast<const uint32_t *>(a.rope.freqs)[static_cast<size_t>(rope_pos) * (a.rope.D / 2) + ((ncol % a.rope.D) >> 1)];
          rope_cs[u] = __builtin_bit_cast(float, f << 16);
          rope_sn[u] = __builtin_bit_cast(float, f & 0xFFFF0000u);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float xsum[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const f32x4_t lo = __builtin_bit_cast(f32x4_t, xs_raw[r][mt][0]);
        float v;
        if constexpr (NGRP == 1) {
          const f32x4_t hi = __builtin_bit_cast(f32x4_t, xs_raw[r][mt][1]);
          v = ((lo[0] + lo[1]) + (lo[2] + lo[3])) + ((hi[0] + hi[1]) + (hi[2] + hi[3]));
        } else if constexpr (NGRP == 2) {
          v = (lo[0] + lo[1]) + (lo[2] + lo[3]);
        } else {
          v = lo[0] + lo[1];
        }
        xsum[mt] = zlive[r] ? v : 0.f;
      }
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const float scale = __builtin_bit_cast(float, zsz[r][t] << 16);
        const float zero = __builtin_bit_cast(float, zsz[r][t] & 0xFFFF0000u);
        const float zc = zlive[r] ? __builtin_fmaf(-136.0f, scale, zero) : 0.f;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(xsum[mt], zc, acc[t][mt], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // straight-line over the C chunks a wave can have: every load sits at a fixed place in the instruction stream, so
    // the waits for a chunk's operands never include younger prefetches
#pragma unroll
    for (int i = 0; i < C; ++i) {
      if (i + DW < C) load_w(wr[i + DW], chunk_at(i + DW));
      if (i + DX < C) load_x(xr[i + DX], chunk_at(i + DX));
      __builtin_amdgcn_sched_barrier(0);
      compute_chunk(wr[i], xr[i], i < nloc ? 0xFFFFFFFFu : 0u);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- the eight K parts meet in LDS; wave w finishes units w, w + 8, .. --------------------------------------------
  {
    float *mine = red + kg * kAccFloats + lane;
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int q = 0; q < 4; ++q) mine[((t * MT + mt) * 4 + q) * 64] = acc[t][mt][q];
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < kUnitsPerWave; ++u) {
    const int unit = kg + u * kWaves;
    if (unit >= kUnits) break;  // uniform per wave
    const int tc = unit / MT, mt = unit % MT;
    float v[GATE ? 2 : 1][4];
#pragma unroll
    for (int h = 0; h < (GATE ? 2 : 1); ++h) {
      const int t = tc + h * TC;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float *src = red + ((t * MT + mt) * 4 + q) * 64 + lane;
        float s = src[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) s += src[w * kAccFloats];
        v[h][q] = s;
      }
    }
    const int n = 16 * (tile16_0 + tc) + c;
    if constexpr (EPI == kStPartial) {
      float *out = a.partials + static_cast<size_t>(ks) * M * N;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = m_base + 16 * mt + 4 * b + q;
        if (n < N && m < M) out[static_cast<size_t>(m) * N + n] = v[0][q];
      }
    } else if constexpr (EPI == kStGate) {
      // bf16(bf16(silu(bf16 gate)) * bf16 up): the rounding points of F.silu(w1(x)) * w3(x) on bfloat16 tensors
      // (reference models/model.py:359-360)
      const bool tile_live = 16 * (tile16_0 + tc) < N;  // whole tiles: N % 16 == 0 on this path
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = m_base + 16 * mt + 4 * b + q;
        const float gate = bf16_round(v[0][q]), up = bf16_round(v[1][q]);
        const float act = bf16_round(gate / (1.0f + expf(-gate)));
        const uint16_t o = f32_to_bf16_rne(act * up);
        if (a.y && n < N && m < M) a.y[static_cast<size_t>(m) * N + n] = o;
        // staged form for the next linear: whole 16-lane groups store (rows past M hold values nobody reads)
        if (a.out.frag && tile_live && m < a.out.mpad) staged_store_run16(a.out, m, n, o);
      }
    } else if constexpr (EPI == kStRope) {
      // the product is the fused q | k | v projection, rounded to bfloat16; the interleaved pairs of the q and k heads
      // are rotated in float32 (reference models/model.py:400-412); q goes to q_out [B, H, D], k and v into the caches
      // [B, Hkv, S, D] at the position (KVCache.update, reference models/model.py:121-129)
      const StagedRope &rp = a.rope;
      const int Dh = rp.D, H = rp.H, Hkv = rp.Hkv;
      const int pos = rope_pos;
      const int head = n / Dh, d = n % Dh;
      const bool in_range = n < N && pos >= 0 && pos < rp.S;
      const bool rotated = head < H + Hkv;
      const float cs = rope_cs[u], sn = rope_sn[u];
      uint16_t *dst;
      size_t row_stride;
      if (head < H) {
        dst = rp.q_out + static_cast<size_t>(head) * Dh + d;
        row_stride = static_cast<size_t>(H) * Dh;
      } else {
        const int hk = rotated ? head - H : head - H - Hkv;
        dst = (rotated ? rp.kc : rp.vc) + (static_cast<size_t>(hk) * rp.S + pos) * Dh + d;
        row_stride = static_cast<size_t>(Hkv) * rp.S * Dh;
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = m_base + 16 * mt + 4 * b + q;
        const float own = bf16_round(v[0][q]);
        const float other = __shfl_xor(own, 1);  // the pair's other column lives in the neighbouring lane
        const float r = (c & 1) ? own * cs + other * sn : own * cs - other * sn;
        if (in_range && m < M) dst[static_cast<size_t>(m) * row_stride] = f32_to_bf16_rne(rotated ? r : own);
      }
    } else if constexpr (EPI == kStArgmax) {
      // greedy token straight from the LM head: the logit is rounded to bfloat16 as the plain epilogue would store it and
      // offered as (order-preserving key << 32 | ~column), so that the maximum is the largest value and, among equals,
      // the lowest column; a NaN counts as the largest value (torch.argmax over the float32 view of bfloat16 logits,
      // reference inference_generate.py:110-120 with sampling switched off).  First over the tile's 16 columns ...
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t u = static_cast<uint32_t>(f32_to_bf16_rne(v[0][q])) << 16;
        const uint32_t key = (u & 0x7FFFFFFFu) > 0x7F800000u ? 0xFFFFFFFFu : ((u & 0x80000000u) ? ~u : (u | 0x80000000u));
        unsigned long long best = n < N ? ((static_cast<unsigned long long>(key) << 32) | static_cast<uint32_t>(~static_cast<uint32_t>(n))) : 0ull;
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
          const unsigned long long other = __shfl_xor(best, off);
          best = other > best ? other : best;
        }
        if (c == 0) unit_best[unit][4 * b + q] = best;
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = m_base + 16 * mt + 4 * b + q;
        if (n < N && m < M) a.y[static_cast<size_t>(m) * N + n] = f32_to_bf16_rne(v[0][q]);
      }
    }
  }
  if constexpr (EPI == kStArgmax) {
    // ... then over the workgroup's column tiles: one candidate per row and column block for the reduction kernel
    __syncthreads();
    if (tid < 16 * MT) {
      const int mt = tid >> 4, m = m_base + tid;
      unsigned long long best = 0ull;
#pragma unroll
      for (int tc = 0; tc < TC; ++tc) best = unit_best[tc * MT + mt][tid & 15] > best ? unit_best[tc * MT + mt][tid & 15] : best;
      if (m < M) a.cand[static_cast<size_t>(col_block) * M + m] = best;
    }
  }
}

// arg-max: the candidates of all column blocks of a row -> the row's token (one wave per row)
__global__ __launch_bounds__(64) void argmax_candidates_kernel(const unsigned long long *__restrict__ cand, int blocks, int M, int64_t *__restrict__ out) {
  const int m = blockIdx.x;
  unsigned long long best = 0ull;
  for (int i = threadIdx.x; i < blocks; i += 64) {
    const unsigned long long v = cand[static_cast<size_t>(i) * M + m];
    best = v > best ? v : best;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const unsigned long long other = __shfl_xor(best, off);
    best = other > best ? other : best;
  }
  if (threadIdx.x == 0) out[m] = static_cast<int64_t>(~static_cast<uint32_t>(best & 0xFFFFFFFFull));
}

// ---- staging pass: row-major activations -> operand order + sums of 16 ------------------------------------------------
// One thread per 16-byte piece (8 values); rows M .. Mpad-1 are written as zeros.
__global__ __launch_bounds__(256) void int4_stage_x_kernel(const uint16_t *__restrict__ x, StagedOut out, int M, int K) {
  const int pieces_per_row = K >> 3;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int m = idx / pieces_per_row, pc = idx % pieces_per_row;
  if (m >= out.mpad) return;  // pieces_per_row is even: both lanes of a pair leave or stay
  u32x4_t raw = {0u, 0u, 0u, 0u};
  if (m < M) raw = *reinterpret_cast<const u32x4_t *>(x + static_cast<size_t>(m) * K + pc * 8);
  staged_store_piece(out, m, pc, raw);
}

// ---- launch geometry ---------------------------------------------------------------------------------------------------
struct Geometry {
  int t, c, dw, dx;  // kernel instantiation
  int slices;        // workgroups along K
};

// instantiated (T, C, DW, DX) per epilogue; registers: about 8 T (sums) + DW * 5 T (weights) + DX * 32 (operands) + 50
struct Inst {
  int t, c, dw, dx;
};
constexpr Inst kPlainInsts[] = {{3, 4, 2, 2}, {4, 4, 2, 2}, {8, 4, 1, 1}, {6, 4, 2, 1}, {2, 2, 2, 2}, {4, 2, 2, 2}, {6, 2, 2, 2}, {4, 1, 1, 1}, {4, 3, 3, 1}, {4, 8, 2, 1}, {8, 8, 1, 1}, {2, 1, 1, 1}};
constexpr Inst kArgmaxInsts[] = {{8, 4, 1, 1}, {4, 4, 2, 2}, {8, 8, 1, 1}, {4, 8, 2, 1}, {4, 1, 1, 1}, {2, 1, 1, 1}};  // LM heads: few K shapes
constexpr Inst kGateInsts[] = {{6, 4, 2, 1}, {4, 4, 2, 2}, {8, 4, 1, 1}, {6, 8, 1, 1}, {8, 8, 1, 1}};

// instantiations that do not fit the 256 vector registers of a wave (they would run, slowly, out of scratch memory):
// smaller groups carry more (scale, zero) pairs per chunk and more rounds of the zero-point term
inline bool fits_registers(int groupsize, const Inst &in) {
  if (groupsize == 32) return !((in.t >= 3 && in.c == 4) || in.t >= 6);
  if (groupsize == 64) return !(in.t == 8 || (in.t == 4 && in.c == 4));
  return true;
}

template <int NI>
bool pick(const Inst (&insts)[NI], bool gate, int groupsize, int tiles16, int kt, int slabs, int max_slices, Geometry *best) {
  long best_cost = -1;
  const int want_t = options().staged_tiles, want_s = options().staged_slices;  // experiments: force a geometry
  for (int s = 1; s <= max_slices; s *= 2) {
    if (want_s && s != want_s) continue;
    if (s > kt) break;
    const int per_slice = (kt + s - 1) / s;  // the longest slice
    const int c_need = (per_slice + kWaves - 1) / kWaves;
    for (const Inst &in : insts) {
      if (in.c != c_need || !fits_registers(groupsize, in)) continue;
      if (want_t && !gate && in.t != want_t) continue;
      const int tc = gate ? in.t / 2 : in.t;
      const long wgs = static_cast<long>((tiles16 + tc - 1) / tc) * s * slabs;
      const long rounds = (wgs + kCUs - 1) / kCUs;
      // per workgroup: a fixed part, the weight tiles, the activation operands of its chunks (about two tiles' worth each);
      // per slice: what the consumer pays to add it
      const long cost = rounds * (4 + static_cast<long>(in.t) * in.c + 2L * in.c) * 2 + 2L * s;
      if (best_cost < 0 || cost < best_cost) {
        best_cost = cost;
        *best = Geometry{in.t, in.c, in.dw, in.dx, s};
      }
    }
  }
  return best_cost >= 0;
}

template <int G, int MT, int T, int C, int DW, int DX, int EPI>
int launch_staged(const StagedArgs &a, int slices, hipStream_t stream) {
  const unsigned gx = a.slabs > 1 ? static_cast<unsigned>((a.col_blocks + 7) / 8 * 8 * a.slabs) : static_cast<unsigned>(a.col_blocks);
  hipLaunchKernelGGL((int4_staged_mm_kernel<G, MT, T, C, DW, DX, EPI>), dim3(gx, slices, 1), dim3(64 * kWaves), 0, stream, a);
  return launch_status();
}

template <int G, int MT, int EPI>
int dispatch_inst(const StagedArgs &a, const Geometry &g, hipStream_t stream) {
#define E2H_ST_CASE(TV, CV, DWV, DXV) \
  if (g.t == TV && g.c == CV && g.dw == DWV && g.dx == DXV) return launch_staged<G, MT, TV, CV, DWV, DXV, EPI>(a, g.slices, stream);
  if constexpr (EPI == kStGate) {
    E2H_ST_CASE(6, 4, 2, 1) E2H_ST_CASE(4, 4, 2, 2) E2H_ST_CASE(8, 4, 1, 1) E2H_ST_CASE(6, 8, 1, 1) E2H_ST_CASE(8, 8, 1, 1)
  } else if constexpr (EPI == kStArgmax) {
    E2H_ST_CASE(8, 4, 1, 1) E2H_ST_CASE(4, 4, 2, 2) E2H_ST_CASE(8, 8, 1, 1) E2H_ST_CASE(4, 8, 2, 1) E2H_ST_CASE(4, 1, 1, 1) E2H_ST_CASE(2, 1, 1, 1)
  } else {
    E2H_ST_CASE(3, 4, 2, 2) E2H_ST_CASE(4, 4, 2, 2) E2H_ST_CASE(8, 4, 1, 1) E2H_ST_CASE(6, 4, 2, 1) E2H_ST_CASE(2, 2, 2, 2)
    E2H_ST_CASE(4, 2, 2, 2) E2H_ST_CASE(6, 2, 2, 2) E2H_ST_CASE(4, 1, 1, 1) E2H_ST_CASE(2, 1, 1, 1) E2H_ST_CASE(4, 3, 3, 1) E2H_ST_CASE(4, 8, 2, 1) E2H_ST_CASE(8, 8, 1, 1)
  }
#undef E2H_ST_CASE
  return E2H_ERR_BAD_SHAPE;
}

template <int EPI>
int dispatch_staged(const StagedArgs &a, int groupsize, const Geometry &g, hipStream_t stream) {
  const bool one = a.M <= 16;
  switch (groupsize) {
    case 32: return one ? dispatch_inst<32, 1, EPI>(a, g, stream) : dispatch_inst<32, 2, EPI>(a, g, stream);
    case 64: return one ? dispatch_inst<64, 1, EPI>(a, g, stream) : dispatch_inst<64, 2, EPI>(a, g, stream);
    default: return one ? dispatch_inst<128, 1, EPI>(a, g, stream) : dispatch_inst<128, 2, EPI>(a, g, stream);
  }
}

int check_shape(int64_t m, int64_t n, int64_t k, int groupsize) {
  if (groupsize != 32 && groupsize != 64 && groupsize != 128) return E2H_ERR_BAD_GROUPSIZE;
  if (m < 1 || m > 64 || n < 16 || (n % 16) != 0 || k < 128 || n > INT32_MAX || k > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if ((k % 128) != 0) return E2H_ERR_BAD_INNER_K_TILES;
  if (n * k / 2 >= (int64_t{1} << 32) || (k / groupsize) * n * 4 >= (int64_t{1} << 32)) return E2H_ERR_BAD_SHAPE;
  return E2H_OK;
}

// fills the shape part of the arguments and picks the geometry; false if no instantiation covers the shape
bool plan(StagedArgs *a, Geometry *g, const void *staged, int64_t m, int64_t n, int64_t k, int groupsize, int epi) {
  a->M = static_cast<int>(m);
  a->Mpad = staged_mpad(m);
  a->N = static_cast<int>(n);
  a->K = static_cast<int>(k);
  a->frag = static_cast<const uint8_t *>(staged);
  a->sums = reinterpret_cast<const float *>(a->frag + static_cast<size_t>(a->Mpad) * k * 2);
  const int mt = a->M <= 16 ? 1 : 2;
  a->slabs = (a->M + 16 * mt - 1) / (16 * mt);
  const int tiles16 = static_cast<int>(n / 16);
  const int kt = static_cast<int>(k / 128);
  bool ok;
  if (epi == kStGate) ok = pick(kGateInsts, true, groupsize, tiles16, kt, a->slabs, 1, g);
  else if (epi == kStArgmax) ok = pick(kArgmaxInsts, false, groupsize, tiles16, kt, a->slabs, 1, g);
  else ok = pick(kPlainInsts, false, groupsize, tiles16, kt, a->slabs, epi == kStPartial ? 8 : 1, g);
  if (!ok) return false;
  const int tc = epi == kStGate ? g->t / 2 : g->t;
  a->col_blocks = (tiles16 + tc - 1) / tc;
  return true;
}

}  // namespace
}  // namespace e2h

using namespace e2h;

extern "C" int64_t e2h_int4_staged_bytes(int64_t m, int64_t k) {
  if (m < 1 || m > 64 || k < 128 || (k % 128) != 0) return E2H_ERR_BAD_SHAPE;
  return staged_bytes(m, k);
}

extern "C" int e2h_int4_stage_x(const uint16_t *x, void *staged, int64_t m, int64_t k, void *stream) {
  if (!x || !staged) return E2H_ERR_NULL_POINTER;
  if (m < 1 || m > 64 || k < 128 || (k % 128) != 0 || k > (1 << 24)) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(staged)) return E2H_ERR_MISALIGNED;
  const StagedOut out = staged_out(staged, m, k);
  const int64_t threads = static_cast<int64_t>(out.mpad) * (k / 8);
  hipLaunchKernelGGL(int4_stage_x_kernel, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream), x,
                     out, static_cast<int>(m), static_cast<int>(k));
  return launch_status();
}

extern "C" int e2h_int4_mm_staged_supported(int64_t m, int64_t n, int64_t k, int groupsize, int epilogue) {
  if (check_shape(m, n, k, groupsize) != E2H_OK || epilogue < 0 || epilogue > 4) return 0;
  StagedArgs a = {};
  Geometry g;
  return plan(&a, &g, nullptr, m, n, k, groupsize, epilogue) ? 1 : 0;
}

extern "C" int e2h_int4_mm_staged(const void *staged, const int32_t *packed, const uint16_t *scales_and_zeros, uint16_t *y, int64_t m,
                                  int64_t n, int64_t k, int groupsize, void *stream) {
  if (!staged || !packed || !scales_and_zeros || !y) return E2H_ERR_NULL_POINTER;
  const int rc = check_shape(m, n, k, groupsize);
  if (rc != E2H_OK) return rc;
  if (!aligned16(staged) || !aligned16(packed) || !aligned16(scales_and_zeros) || (reinterpret_cast<uintptr_t>(y) & 1u)) return E2H_ERR_MISALIGNED;
  StagedArgs a = {};
  Geometry g;
  if (!plan(&a, &g, staged, m, n, k, groupsize, kStPlain)) return E2H_ERR_BAD_SHAPE;
  a.wp = reinterpret_cast<const uint32_t *>(packed);
  a.sz = reinterpret_cast<const uint32_t *>(scales_and_zeros);
  a.y = y;
  return dispatch_staged<kStPlain>(a, groupsize, g, static_cast<hipStream_t>(stream));
}

extern "C" int64_t e2h_int4_mm_staged_argmax_scratch_bytes(int64_t m, int64_t n, int64_t k, int groupsize) {
  const int rc = check_shape(m, n, k, groupsize);
  if (rc != E2H_OK) return rc;
  StagedArgs a = {};
  Geometry g;
  if (!plan(&a, &g, nullptr, m, n, k, groupsize, kStArgmax)) return E2H_ERR_BAD_SHAPE;
  return static_cast<int64_t>(a.col_blocks) * m * 8;
}

extern "C" int e2h_int4_mm_staged_argmax(const void *staged, const int32_t *packed, const uint16_t *scales_and_zeros, void *scratch,
                                         int64_t *tokens, int64_t m, int64_t n, int64_t k, int groupsize, void *stream) {
  if (!staged || !packed || !scales_and_zeros || !scratch || !tokens) return E2H_ERR_NULL_POINTER;
  const int rc = check_shape(m, n, k, groupsize);
  if (rc != E2H_OK) return rc;
  if (!aligned16(staged) || !aligned16(packed) || !aligned16(scales_and_zeros) || (reinterpret_cast<uintptr_t>(scratch) & 7u) ||
      (reinterpret_cast<uintptr_t>(tokens) & 7u))
    return E2H_ERR_MISALIGNED;
  StagedArgs a = {};
  Geometry g;
  if (!plan(&a, &g, staged, m, n, k, groupsize, kStArgmax)) return E2H_ERR_BAD_SHAPE;
  a.wp = reinterpret_cast<const uint32_t *>(packed);
  a.sz = reinterpret_cast<const uint32_t *>(scales_and_zeros);
  a.cand = static_cast<unsigned long long *>(scratch);
  const int rc2 = dispatch_staged<kStArgmax>(a, groupsize, g, static_cast<hipStream_t>(stream));
  if (rc2 != E2H_OK) return rc2;
  hipLaunchKernelGGL(argmax_candidates_kernel, dim3(static_cast<unsigned>(m)), dim3(64), 0, static_cast<hipStream_t>(stream), a.cand,
                     a.col_blocks, a.M, tokens);
  return launch_status();
}

extern "C" int e2h_int4_mm_staged_partial_slices(int64_t m, int64_t n, int64_t k, int groupsize) {
  const int rc = check_shape(m, n, k, groupsize);
  if (rc != E2H_OK) return rc;
  if (m > 32 && !options().staged_no_rows64) {  // one pass over the weights for all rows
    const int s64 = rows64_partial_slices(m, n, k, groupsize);
    if (s64 > 0) return s64;
  }
  StagedArgs a = {};
  Geometry g;
  if (!plan(&a, &g, nullptr, m, n, k, groupsize, kStPartial)) return E2H_ERR_BAD_SHAPE;
  return g.slices;
}

extern "C" int e2h_int4_mm_staged_partials(const void *staged, const int32_t *packed, const uint16_t *scales_and_zeros, float *partials,
                                           int64_t m, int64_t n, int64_t k, int groupsize, int slices, void *stream) {
  if (!staged || !packed || !scales_and_zeros || !partials) return E2H_ERR_NULL_POINTER;
  const int rc = check_shape(m, n, k, groupsize);
  if (rc != E2H_OK) return rc;
  if (!aligned16(staged) || !aligned16(packed) || !aligned16(scales_and_zeros) || (reinterpret_cast<uintptr_t>(partials) & 3u)) return E2H_ERR_MISALIGNED;
  if (m > 32 && !options().staged_no_rows64 && rows64_partial_slices(m, n, k, groupsize) > 0)
    return rows64_partials(staged, packed, scales_and_zeros, partials, m, n, k, groupsize, slices, static_cast<hipStream_t>(stream));
  StagedArgs a = {};
  Geometry g;
  if (!plan(&a, &g, staged, m, n, k, groupsize, kStPartial)) return E2H_ERR_BAD_SHAPE;
  if (slices != g.slices) return E2H_ERR_BAD_SHAPE;
  a.wp = reinterpret_cast<const uint32_t *>(packed);
  a.sz = reinterpret_cast<const uint32_t *>(scales_and_zeros);
  a.partials = partials;
  return dispatch_staged<kStPartial>(a, groupsize, g, static_cast<hipStream_t>(stream));
}

extern "C" int e2h_int4_mm_staged_silu_gate(const void *staged, const int32_t *packed_gate, const uint16_t *sz_gate, const int32_t *packed_up,
                                            const uint16_t *sz_up, uint16_t *y, void *staged_out_buf, int64_t m, int64_t n, int64_t k,
                                            int groupsize, void *stream) {
  if (!staged || !packed_gate || !sz_gate || !packed_up || !sz_up || (!y && !staged_out_buf)) return E2H_ERR_NULL_POINTER;
  const int rc = check_shape(m, n, k, groupsize);
  if (rc != E2H_OK) return rc;
  if (staged_out_buf && (n % 128) != 0) return E2H_ERR_BAD_SHAPE;  // the result is the next linear's K
  if (!aligned16(staged) || !aligned16(packed_gate) || !aligned16(sz_gate) || !aligned16(packed_up) || !aligned16(sz_up) ||
      (reinterpret_cast<uintptr_t>(y) & 1u) || !aligned16(staged_out_buf))
    return E2H_ERR_MISALIGNED;
  StagedArgs a = {};
  Geometry g;
  if (!plan(&a, &g, staged, m, n, k, groupsize, kStGate)) return E2H_ERR_BAD_SHAPE;
  a.wp = reinterpret_cast<const uint32_t *>(packed_gate);
  a.sz = reinterpret_cast<const uint32_t *>(sz_gate);
  a.wp2 = reinterpret_cast<const uint32_t *>(packed_up);
  a.sz2 = reinterpret_cast<const uint32_t *>(sz_up);
  a.y = y;
  a.out = staged_out(staged_out_buf, m, n);
  return dispatch_staged<kStGate>(a, groupsize, g, static_cast<hipStream_t>(stream));
}

extern "C" int e2h_int4_mm_staged_rope_kv(const void *staged, const int32_t *packed, const uint16_t *scales_and_zeros, const uint16_t *freqs_cis,
                                          uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache, const int64_t *input_pos, int64_t batch,
                                          int64_t n_head, int64_t n_kv_head, int64_t head_dim, int64_t cache_len, int64_t k, int groupsize,
                                          void *stream) {
  if (!staged || !packed || !scales_and_zeros || !freqs_cis || !q_out || !k_cache || !v_cache || !input_pos) return E2H_ERR_NULL_POINTER;
  if (n_head < 1 || n_kv_head < 1 || head_dim < 2 || (head_dim % 2) != 0 || cache_len < 1 || cache_len > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  const int64_t n = (n_head + 2 * n_kv_head) * head_dim;
  const int rc = check_shape(batch, n, k, groupsize);
  if (rc != E2H_OK) return rc;
  if (!aligned16(staged) || !aligned16(packed) || !aligned16(scales_and_zeros) || (reinterpret_cast<uintptr_t>(freqs_cis) & 3u) ||
      (reinterpret_cast<uintptr_t>(q_out) & 1u) || (reinterpret_cast<uintptr_t>(k_cache) & 1u) || (reinterpret_cast<uintptr_t>(v_cache) & 1u) ||
      (reinterpret_cast<uintptr_t>(input_pos) & 7u))
    return E2H_ERR_MISALIGNED;
  StagedArgs a = {};
  Geometry g;
  if (!plan(&a, &g, staged, batch, n, k, groupsize, kStRope)) return E2H_ERR_BAD_SHAPE;
  a.wp = reinterpret_cast<const uint32_t *>(packed);
  a.sz = reinterpret_cast<const uint32_t *>(scales_and_zeros);
  a.rope = StagedRope{freqs_cis, q_out, k_cache, v_cache, input_pos, static_cast<int>(n_head), static_cast<int>(n_kv_head),
                      static_cast<int>(cache_len), static_cast<int>(head_dim)};
  return dispatch_staged<kStRope>(a, groupsize, g, static_cast<hipStream_t>(stream));
}

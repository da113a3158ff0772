// int4 group-wise dequant matmul for decode batches of 33 .. 64 rows on staged activations, K-slice sums out.
//
// Same contract, arithmetic and data layouts as the partial-sum entry point of e2h_int4_staged.hip (torch.ops.aten.
// _weight_int4pack_mm as called by linear_forward_int4, reference models/quantize.py:445-453; the slices are added by
// the consumer in slice order), for the row counts at which that kernel's decomposition stops paying: there every
// workgroup covers 32 rows, reads the activation operands of all of its K slice for a handful of weight tiles, and a
// second slab of workgroups passes over the weights again.  At 64 rows and K = 8192 that is 1 MB of operands per
// 0.16 - 0.7 MB of weights and CU.  Here
//   * a workgroup covers all (up to) 64 rows: one pass over the weights;
//   * its eight waves split N (T tiles of 16 weight rows each), not K, and share the activation operands of a
//     128-wide chunk through LDS, so a CU reads them once per 8 T tiles instead of once per wave;
//   * S workgroups split K, so a CU reads 1 / S of the operands (the price: S float32 slices for the consumer to add);
//   * the chunk loop is a rolling pipeline: operands reach LDS by 16-byte buffer loads that write LDS directly (lane L
//     of an instruction lands at base + 16 L), four stages, loads three chunks ahead, one barrier per chunk; weights
//     and (scale, zero) pairs go straight into a register ring of the same depth.
// Arithmetic per output as in e2h_int4_staged.hip: y = sum_g s * P_g + sum_g (z - 136 s) * X_g with exact products
// P_g = sum_k x (128 + q) in v_mfma_f32_16x16x32_bf16 and the group sums X_g continued from the staged sums of 16; the
// second sum is a float32 matrix product over groups (v_mfma_f32_16x16x4_f32, four groups per instruction: lane group
// b takes group 4 r + b, picked up chunk by chunk as its chunk comes by).
//
// Measured at 64 rows, group size 64: 8192 x 22016 48.8 us (two 32-row slabs: 68.2), 8192 x 8192 24.1 (22.1).  The kernel
// is bound by its vector work (per tile and chunk 16 MFMAs and about 60 vector instructions at four row tiles), not by
// memory: eight stages instead of four, or a register cap for two workgroups per CU, are slower.
//
// LDS stage (18 KB): [segment 0..3][row tile 0..3] blocks of 1 KB = 16 rows x 64 bytes of the staged fragment array
// (contiguous in memory); inside a block the 16-byte quarter q of row r sits at r * 64 + ((q ^ (r >> 2)) & 3) * 16, so
// the operand read of 16 rows at one quarter touches 16 different bank groups; then the chunk's sums [64 rows][8].
#include "e2h_common.h"
#include "e2h_int4_unpack.h"
#include "e2h_staged.h"

namespace e2h {
namespace {

constexpr int kWaves64 = 8;
constexpr int kRing = 4;                     // LDS stages and register sets; loads run kRing - 1 chunks ahead
constexpr int kStageFrag = 16 * 1024;        // 4 segments x 4 row tiles x 1 KB
constexpr int kStageBytes = kStageFrag + 2048;
constexpr int kNt64 = 2;                     // "nt" cache policy: weights are streamed once
constexpr int kCUs64 = 256;

struct Rows64Args {
  const uint8_t *frag;
  const float *sums;
  const uint32_t *wp, *sz;
  float *partials;  // f32 [S][M][N]
  int M, Mpad, N, K;
};

// G group size, T tiles of 16 weight rows per wave
template <int G, int T>
__global__ __launch_bounds__(64 * kWaves64) void int4_rows64_partials_kernel(const Rows64Args a) {
  constexpr int NGRP = 128 / G;      // groups per chunk
  constexpr int SPG = G / 32;        // 32-wide segments (MFMA steps) per group
  constexpr int RC = 4 / NGRP;       // chunks per round of the zero-point term (four groups)
  constexpr int MT = 4;              // row tiles of 16
  constexpr int kOps = 3 + T * (2 + NGRP);  // memory instructions a wave issues per chunk
  typedef __attribute__((address_space(3))) void lds_void;
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kRing * kStageBytes];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, b = lane >> 4;
  const int N = a.N, K = a.K, M = a.M;
  const int n_tiles8 = N >> 3;
  const int KT = K >> 7;
  const int S = gridDim.y, ks = blockIdx.y;
  const int C0 = static_cast<int>((static_cast<unsigned>(KT) * static_cast<unsigned>(ks)) / static_cast<unsigned>(S));
  const int C1 = static_cast<int>((static_cast<unsigned>(KT) * static_cast<unsigned>(ks + 1)) / static_cast<unsigned>(S));
  const int L = C1 - C0;  // >= 1: the host never asks for more slices than chunks
  const int tile16_0 = (blockIdx.x * kWaves64 + wave) * T;
  const uint32_t row_block = static_cast<uint32_t>(a.Mpad) * 64u;  // bytes of one k segment of all rows

  uint32_t wlane[T], szlane[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int tcol = tile16_0 + t;
    int nt8 = 2 * tcol + (c >> 3);
    nt8 = nt8 < n_tiles8 ? nt8 : n_tiles8 - 1;
    wlane[t] = static_cast<uint32_t>((static_cast<size_t>(nt8) * KT * 32 + ((c & 7) * 4 + b)) * 16);
    int ncol = 16 * tcol + c;
    ncol = ncol < N ? ncol : N - 1;
    szlane[t] = static_cast<uint32_t>(ncol) * 4u;
  }
  const uint32_t frag_bytes = static_cast<uint32_t>(static_cast<size_t>(K / 32) * row_block);
  const uint32_t sums_bytes = static_cast<uint32_t>(static_cast<size_t>(KT) * a.Mpad * 32);
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(a.wp, static_cast<uint32_t>(static_cast<size_t>(N) * K / 2));
  const __amdgpu_buffer_rsrc_t sz_rsrc = make_rsrc(a.sz, static_cast<uint32_t>(static_cast<size_t>(K / G) * N * 4));
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(a.frag, frag_bytes);
  const __amdgpu_buffer_rsrc_t xs_rsrc = make_rsrc(a.sums, sums_bytes);

  // ---- what this lane brings into LDS per chunk: the 16-byte piece that belongs at position `lane` of blocks `wave` and
  // `wave + 8` (block = 4 * segment + row tile: row lane / 4 of the tile, quarter (lane % 4) ^ (row / 4) -- reads past the
  // rows of a batch of 33 .. 48 land in the next segment or past the buffer (zeros): rows nobody uses), and dword
  // 64 * wave + lane of the chunk's sums
  uint32_t xl[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int blk = wave + 8 * j, seg = blk >> 2, mt = blk & 3;
    const int r = lane >> 2, q = (lane & 3) ^ ((lane >> 4) & 3);
    xl[j] = static_cast<uint32_t>(seg) * row_block + static_cast<uint32_t>((16 * mt + r) * 64 + q * 16);
  }
  const uint32_t sl = static_cast<uint32_t>((wave * 64 + lane) * 4);

  struct WRegs {
    u32x4_t w[T];
    uint32_t sz[T][NGRP];
    uint32_t zsz[T];  // the (scale, zero) pair of this lane's group of the zero-point term, if the group is in this chunk
  };
  WRegs ring[kRing];
  auto chunk_at = [&](int i) { return C0 + (i < L ? i : L - 1); };  // past the slice: re-read its last chunk, used with weight zero
  // all loads of chunk i of the slice: operands and sums into LDS stage `slot`, weights and qparams into ring[slot]
  auto issue = [&](int i, int slot) {
    const int ci = chunk_at(i);
    const uint32_t stage = static_cast<uint32_t>(slot) * kStageBytes;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (lds_void *)(lds + stage + (wave + 8 * j) * 1024), 16, xl[j],
                                               static_cast<uint32_t>(ci) * 4u * row_block, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(xs_rsrc, (lds_void *)(lds + stage + kStageFrag + wave * 256), 4, sl,
                                             static_cast<uint32_t>(ci) * static_cast<uint32_t>(a.Mpad) * 32u, 0, 0);
    WRegs &r = ring[slot];
#pragma unroll
    for (int t = 0; t < T; ++t) {
      r.w[t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wlane[t], static_cast<uint32_t>(ci) * 512u, kNt64);
#pragma unroll
      for (int g = 0; g < NGRP; ++g)
        r.sz[t][g] = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, szlane[t], static_cast<uint32_t>(ci * NGRP + g) * static_cast<uint32_t>(N) * 4u, 0);
      // lane group b owns group b % NGRP of the chunk in which its turn comes (lane-dependent: in the vector offset)
      r.zsz[t] = __builtin_amdgcn_raw_buffer_load_b32(
          sz_rsrc, szlane[t] + static_cast<uint32_t>(ci * NGRP + (b % NGRP)) * static_cast<uint32_t>(N) * 4u, 0, 0);
    }
  };

  f32x4_t acc[T][MT];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const UnpackConsts uc = unpack_consts();
  // operand read of lane (b, c): row c of a tile, quarter b
  const uint32_t frag_lane = static_cast<uint32_t>(c * 64 + ((b ^ ((c >> 2) & 3)) << 4));
  float xz[MT], zc[T];  // this lane's operands of the zero-point term for the round in progress
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xz[mt] = 0.f;
#pragma unroll
  for (int t = 0; t < T; ++t) zc[t] = 0.f;

  // chunk i of the slice, in ring slot u = i % kRing (compile-time)
  auto compute = [&](int i, int u) {
    const WRegs &r = ring[u];
    const uint8_t *stage = lds + u * kStageBytes;
    const bool live = i < L;
    const uint32_t live_mask = live ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int g = 0; g < NGRP; ++g) {
      u32x4_t xf[SPG][MT];
#pragma unroll
      for (int sg = 0; sg < SPG; ++sg)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          xf[sg][mt] = *reinterpret_cast<const u32x4_t *>(stage + ((g * SPG + sg) * 4 + mt) * 1024 + frag_lane);
#pragma unroll
      for (int t = 0; t < T; ++t) {
        f32x4_t part[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) part[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sg = 0; sg < SPG; ++sg) {
          const bf16x8_t wf = unpack_word(r.w[t][g * SPG + sg], uc);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            part[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, xf[sg][mt]), wf, part[mt], 0, 0, 0);
        }
        const float scale = __builtin_bit_cast(float, (r.sz[t][g] & live_mask) << 16);  // past the slice: the chunk adds nothing
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[t][mt][q] = __builtin_fmaf(scale, part[mt][q], acc[t][mt][q]);
      }
    }
    // ---- zero-point term: the lane groups whose group lies in this chunk pick up their operands
    const bool mine = (b / NGRP) == (u % RC);
    {
      const uint8_t *sums = stage + kStageFrag;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const uint8_t *p = sums + (16 * mt + c) * 32 + (b % NGRP) * (32 / NGRP);
        float v;
        if constexpr (NGRP == 1) {
          const f32x4_t lo = *reinterpret_cast<const f32x4_t *>(p), hi = *reinterpret_cast<const f32x4_t *>(p + 16);
          v = ((lo[0] + lo[1]) + (lo[2] + lo[3])) + ((hi[0] + hi[1]) + (hi[2] + hi[3]));
        } else if constexpr (NGRP == 2) {
          const f32x4_t lo = *reinterpret_cast<const f32x4_t *>(p);
          v = (lo[0] + lo[1]) + (lo[2] + lo[3]);
        } else {
          const float lo0 = *reinterpret_cast<const float *>(p), lo1 = *reinterpret_cast<const float *>(p + 4);
          v = lo0 + lo1;
        }
        xz[mt] = mine ? (live ? v : 0.f) : xz[mt];
      }
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const float scale = __builtin_bit_cast(float, r.zsz[t] << 16), zero = __builtin_bit_cast(float, r.zsz[t] & 0xFFFF0000u);
        zc[t] = mine ? (live ? __builtin_fmaf(-136.0f, scale, zero) : 0.f) : zc[t];
      }
    }
    if ((u % RC) == RC - 1) {
#pragma unroll
      for (int t = 0; t < T; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(xz[mt], zc[t], acc[t][mt], 0, 0, 0);
    }
  };

  // ---- pipeline: chunks 0 .. 2 on their way, then per chunk: arithmetic, the loads three chunks ahead (into the stage
  // and the registers of the chunk before this one, which every wave left at the previous barrier), wait until the
  // next chunk has landed (loads complete in order: the two younger chunks' may still be out), barrier
#pragma unroll
  for (int i = 0; i < kRing - 1; ++i) issue(i, i);
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((kRing - 2) * kOps) : "memory");
  for (int i0 = 0; i0 < L; i0 += kRing) {
#pragma unroll
    for (int u = 0; u < kRing; ++u) {
      compute(i0 + u, u);
      __builtin_amdgcn_sched_barrier(0);
      issue(i0 + u + kRing - 1, (u + kRing - 1) % kRing);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((kRing - 2) * kOps) : "memory");
    }
  }
  // the loads issued past the slice still write LDS: they must land before the workgroup gives its LDS away
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- store: lane (b, c) holds column c of a tile, rows 4 b .. 4 b + 3 of each row tile
  float *out = a.partials + static_cast<size_t>(ks) * M * N;
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int n = 16 * (tile16_0 + t) + c;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = 16 * mt + 4 * b + q;
        if (n < N && m < M) out[static_cast<size_t>(m) * N + n] = acc[t][mt][q];
      }
  }
}

struct Geometry64 {
  int t, slices;
};

// T in {1, 2} tiles per wave, S in {1, 2, 4, 8} slices: the fewest rounds of workgroups over the CUs, then the least
// work per workgroup (per chunk T KB of weights per wave against 18 KB of operands per workgroup), then the fewest slices
bool pick64(int groupsize, int tiles16, int kt, Geometry64 *best) {
  long best_cost = -1;
  for (int t = 1; t <= 1; ++t)  // (two tiles per wave: the register ring of that depth does not fit)
    for (int s = 1; s <= 8; s *= 2) {
      if (s > kt) break;
      if (options().staged_slices && s != options().staged_slices) continue;  // experiments: force the number of slices
      const long col_blocks = (tiles16 + kWaves64 * t - 1) / (kWaves64 * t);
      const long rounds = (col_blocks * s + kCUs64 - 1) / kCUs64;
      const long chunks = (kt + s - 1) / s;
      const long cost = rounds * (8 + chunks * (t + 2)) + 4L * s;
      if (best_cost < 0 || cost < best_cost) {
        best_cost = cost;
        *best = Geometry64{t, s};
      }
    }
  return best_cost >= 0;
}

template <int G>
int launch64(const Rows64Args &a, const Geometry64 &g, hipStream_t stream) {
  const int tiles16 = a.N / 16;
  const unsigned gx = static_cast<unsigned>((tiles16 + kWaves64 * g.t - 1) / (kWaves64 * g.t));
  if (g.t != 1) return E2H_ERR_BAD_SHAPE;
  hipLaunchKernelGGL((int4_rows64_partials_kernel<G, 1>), dim3(gx, g.slices, 1), dim3(64 * kWaves64), 0, stream, a);
  return launch_status();
}

}  // namespace

int rows64_partial_slices(int64_t m, int64_t n, int64_t k, int groupsize) {
  if (m <= 32 || m > 64 || (groupsize != 32 && groupsize != 64 && groupsize != 128)) return 0;
  Geometry64 g;
  if (!pick64(groupsize, static_cast<int>(n / 16), static_cast<int>(k / 128), &g)) return 0;
  return g.slices;
}

int rows64_partials(const void *staged, const int32_t *packed, const uint16_t *sz, float *partials, int64_t m, int64_t n, int64_t k,
                    int groupsize, int slices, hipStream_t stream) {
  Geometry64 g;
  if (!pick64(groupsize, static_cast<int>(n / 16), static_cast<int>(k / 128), &g) || g.slices != slices) return E2H_ERR_BAD_SHAPE;
  Rows64Args a;
  a.M = static_cast<int>(m);
  a.Mpad = staged_mpad(m);
  a.N = static_cast<int>(n);
  a.K = static_cast<int>(k);
  a.frag = static_cast<const uint8_t *>(staged);
  a.sums = reinterpret_cast<const float *>(a.frag + static_cast<size_t>(a.Mpad) * k * 2);
  a.wp = reinterpret_cast<const uint32_t *>(packed);
  a.sz = reinterpret_cast<const uint32_t *>(sz);
  a.partials = partials;
  switch (groupsize) {
    case 32: return launch64<32>(a, g, stream);
    case 64: return launch64<64>(a, g, stream);
    default: return launch64<128>(a, g, stream);
  }
}

}  // namespace e2h

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
//   with the same k order (dwords j, j+4, j+8, j+12 of the 64-byte activation segment) and the weights
//   are never re-packed.
//   The scale and zero are applied to the float32 accumulators once per group:
//     y[m,n] += s * sum_k x[m,k]*(128+q[n,k]) + (z - 136*s) * sum_k x[m,k]
//   (the group sums of x come from one extra MFMA against an all-ones fragment, which lands them in the
//   accumulator layout).  bf16*bf16 products are exact in float32, so this is more accurate than a
//   dequantize-to-bf16 kernel.
//
// Work decomposition: a workgroup of 4 waves owns 16*T output columns (T tiles of 16 rows of the weight)
// and 16*MT rows of x; the 4 waves split K (interleaved chunks) and their partial accumulators are
// summed in a fixed order through LDS, so the result is deterministic.
#include "e2h_common.h"

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
};

template <int N> struct WordVec;
template <> struct WordVec<1> { typedef uint32_t type; };
template <> struct WordVec<2> { typedef u32x2_t type; };
template <> struct WordVec<4> { typedef u32x4_t type; };

constexpr int kWaves = 4;

template <int G, int IKT, int MT, int T>
struct ChunkRegs {
  typedef Int4Geom<G, IKT> Geo;
  uint32_t w[T][Geo::STEPS];
  u32x4_t xf[MT][Geo::STEPS];
  uint32_t sz[T][Geo::NGRP];
};

__device__ __forceinline__ bf16x8_t unpack_word(uint32_t w) {
  constexpr uint32_t kMask = 0x000F000Fu, kMagic = 0x43004300u;  // bf16 128.0 | q  == 128 + q
  u32x4_t u;
  u[0] = (w & kMask) | kMagic;
  u[1] = ((w >> 4) & kMask) | kMagic;
  u[2] = ((w >> 8) & kMask) | kMagic;
  u[3] = ((w >> 12) & kMask) | kMagic;
  return __builtin_bit_cast(bf16x8_t, u);
}

template <int G, int IKT, int MT, int T>
__global__ __launch_bounds__(kWaves * 64, 2) void int4_skinny_mm_kernel(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ wp, const uint32_t *__restrict__ sz,
    uint16_t *__restrict__ y, int M, int N, int K) {
  typedef Int4Geom<G, IKT> Geo;
  typedef typename WordVec<Geo::WORDS>::type wvec_t;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = lane & 15;  // column of the MFMA tile (weight row within the 16-row tile) / x row
  const int b = lane >> 4;  // k-block of the MFMA
  const int n_tiles8 = N >> 3;
  const int KT = K / Geo::KBLK;
  const int nchunks = K / Geo::CHUNK;
  const int tile16_0 = blockIdx.x * T;
  const int m_base = blockIdx.y * (16 * MT);

  const uint32_t *wlane[T];
  const uint32_t *szlane[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int nt8 = 2 * (tile16_0 + t) + (c >> 3);
    nt8 = nt8 < n_tiles8 ? nt8 : n_tiles8 - 1;
    wlane[t] = wp + (static_cast<size_t>(nt8) * KT * 32 + ((c & 7) * 4 + b)) * Geo::WORDS;
    int ncol = 16 * (tile16_0 + t) + c;
    ncol = ncol < N ? ncol : N - 1;
    szlane[t] = sz + ncol;
  }
  const uint16_t *xlane[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int row = m_base + 16 * mt + c;
    row = row < M ? row : M - 1;
    xlane[mt] = x + static_cast<size_t>(row) * K + 2 * b;
  }

  f32x4_t acc[T][MT];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  auto load_chunk = [&](ChunkRegs<G, IKT, MT, T> &r, int ci) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
      for (int blk = 0; blk < Geo::NBLK; ++blk) {
        const size_t kb = static_cast<size_t>(ci) * Geo::NBLK + blk;
        wvec_t v = *reinterpret_cast<const wvec_t *>(wlane[t] + kb * (32 * Geo::WORDS));
        if constexpr (Geo::WORDS == 1) {
          r.w[t][blk] = v;
        } else {
#pragma unroll
          for (int p = 0; p < Geo::WORDS; ++p) r.w[t][blk * Geo::WORDS + p] = v[p];
        }
      }
#pragma unroll
      for (int g = 0; g < Geo::NGRP; ++g)
        r.sz[t][g] = szlane[t][(static_cast<size_t>(ci) * Geo::NGRP + g) * N];
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const uint16_t *xp = xlane[mt] + static_cast<size_t>(ci) * Geo::CHUNK;
#pragma unroll
      for (int s = 0; s < Geo::STEPS; ++s) {
#pragma unroll
        for (int i = 0; i < 4; ++i) r.xf[mt][s][i] = *reinterpret_cast<const uint32_t *>(xp + 32 * s + 8 * i);
      }
    }
  };

  const bf16x8_t ones = __builtin_bit_cast(bf16x8_t, u32x4_t{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});

  auto compute_chunk = [&](const ChunkRegs<G, IKT, MT, T> &r) {
    // group sums of x, already in accumulator layout (every column holds the same sum)
    f32x4_t xs[MT][Geo::NGRP];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int g = 0; g < Geo::NGRP; ++g) {
        f32x4_t s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < Geo::SPG; ++s)
          s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, r.xf[mt][g * Geo::SPG + s]), ones, s4, 0, 0, 0);
        xs[mt][g] = s4;
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
          const bf16x8_t wf = unpack_word(r.w[t][g * Geo::SPG + s]);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            part[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, r.xf[mt][g * Geo::SPG + s]), wf, part[mt], 0, 0, 0);
        }
        const uint32_t szw = r.sz[t][g];
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

  ChunkRegs<G, IKT, MT, T> bufA, bufB;
  int ci = wave;
  if (ci < nchunks) load_chunk(bufA, ci);
  while (ci < nchunks) {
    const int c1 = ci + kWaves;
    if (c1 < nchunks) load_chunk(bufB, c1);
    compute_chunk(bufA);
    if (c1 >= nchunks) break;
    const int c2 = c1 + kWaves;
    if (c2 < nchunks) load_chunk(bufA, c2);
    compute_chunk(bufB);
    ci = c2;
  }

  // cross-wave reduction in a fixed order, then bf16 store
  __shared__ float red[kWaves][T * MT * 4][64];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int q = 0; q < 4; ++q) red[wave][(t * MT + mt) * 4 + q][lane] = acc[t][mt][q];
  __syncthreads();
#pragma unroll
  for (int it = 0; it < T * MT; ++it) {
    const int e = it * (kWaves * 64) + threadIdx.x;
    const int L = e & 63;
    const int slot = e >> 6;
    const int q = slot & 3;
    const int mt = (slot >> 2) % MT;
    const int t = (slot >> 2) / MT;
    float s = red[0][slot][L];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) s += red[w][slot][L];
    const int n = 16 * (tile16_0 + t) + (L & 15);
    const int m = m_base + 16 * mt + 4 * (L >> 4) + q;
    if (n < N && m < M) y[static_cast<size_t>(m) * N + n] = f32_to_bf16_rne(s);
  }
}

template <int G, int IKT, int MT, int T>
int launch(const uint16_t *x, const int32_t *packed, const uint16_t *sz, uint16_t *y, int M, int N, int K,
           hipStream_t stream) {
  const int tiles16 = (N + 15) / 16;
  dim3 grid((tiles16 + T - 1) / T, (M + 16 * MT - 1) / (16 * MT));
  hipLaunchKernelGGL((int4_skinny_mm_kernel<G, IKT, MT, T>), grid, dim3(kWaves * 64), 0, stream, x,
                     reinterpret_cast<const uint32_t *>(packed), reinterpret_cast<const uint32_t *>(sz), y, M, N, K);
  return launch_status();
}

template <int G, int IKT>
int dispatch_mt_t(int mt, int t, const uint16_t *x, const int32_t *packed, const uint16_t *sz, uint16_t *y,
                  int M, int N, int K, hipStream_t stream) {
  if constexpr (IKT == 8 && G <= 128) {
#define E2H_CASE(MTV, TV) \
  if (mt == MTV && t == TV) return launch<G, IKT, MTV, TV>(x, packed, sz, y, M, N, K, stream);
    E2H_CASE(1, 1) E2H_CASE(1, 2) E2H_CASE(1, 4)
    E2H_CASE(2, 1) E2H_CASE(2, 2) E2H_CASE(2, 4)
    E2H_CASE(4, 1) E2H_CASE(4, 2)
#undef E2H_CASE
    return launch<G, IKT, 4, 2>(x, packed, sz, y, M, N, K, stream);
  } else {
    // rarely used geometries: one column tile per workgroup keeps the register footprint small
    if (mt == 1) return launch<G, IKT, 1, 1>(x, packed, sz, y, M, N, K, stream);
    if (mt == 2) return launch<G, IKT, 2, 1>(x, packed, sz, y, M, N, K, stream);
    return launch<G, IKT, 4, 1>(x, packed, sz, y, M, N, K, stream);
  }
}

template <int G>
int dispatch_ikt(int ikt, int mt, int t, const uint16_t *x, const int32_t *packed, const uint16_t *sz,
                 uint16_t *y, int M, int N, int K, hipStream_t stream) {
  switch (ikt) {
    case 2: return dispatch_mt_t<G, 2>(mt, t, x, packed, sz, y, M, N, K, stream);
    case 4: return dispatch_mt_t<G, 4>(mt, t, x, packed, sz, y, M, N, K, stream);
    default: return dispatch_mt_t<G, 8>(mt, t, x, packed, sz, y, M, N, K, stream);
  }
}

}  // namespace
}  // namespace e2h

extern "C" int e2h_int4_mm(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros,
                           uint16_t *y, int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles,
                           void *stream) {
  using namespace e2h;
  if (!x || !packed || !scales_and_zeros || !y) return E2H_ERR_NULL_POINTER;
  if (groupsize != 32 && groupsize != 64 && groupsize != 128 && groupsize != 256) return E2H_ERR_BAD_GROUPSIZE;
  if (inner_k_tiles != 2 && inner_k_tiles != 4 && inner_k_tiles != 8) return E2H_ERR_BAD_INNER_K_TILES;
  if (m < 1 || n < 8 || k < 1 || (n % 8) != 0 || m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if (k % groupsize != 0) return E2H_ERR_BAD_GROUPSIZE;
  if (k % (16 * inner_k_tiles) != 0) return E2H_ERR_BAD_INNER_K_TILES;
  if (!aligned16(x) || !aligned16(packed) || !aligned16(scales_and_zeros) || (reinterpret_cast<uintptr_t>(y) & 1u))
    return E2H_ERR_MISALIGNED;
  const int M = static_cast<int>(m), N = static_cast<int>(n), K = static_cast<int>(k);
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  // columns per workgroup: enough workgroups to cover the chip a few times over, otherwise as many
  // weight tiles per activation fragment as possible
  int t = options().int4_rows_per_wave / 16;
  if (t != 1 && t != 2 && t != 4) {
    const int tiles16 = (N + 15) / 16;
    t = 1;
    if (tiles16 >= 2 * 1024) t = 2;
    if (tiles16 >= 4 * 1024 && mt <= 2) t = 4;
  }
  if (mt == 4 && t == 4) t = 2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (groupsize) {
    case 32: return dispatch_ikt<32>(inner_k_tiles, mt, t, x, packed, scales_and_zeros, y, M, N, K, s);
    case 64: return dispatch_ikt<64>(inner_k_tiles, mt, t, x, packed, scales_and_zeros, y, M, N, K, s);
    case 128: return dispatch_ikt<128>(inner_k_tiles, mt, t, x, packed, scales_and_zeros, y, M, N, K, s);
    default: return dispatch_ikt<256>(inner_k_tiles, mt, t, x, packed, scales_and_zeros, y, M, N, K, s);
  }
}

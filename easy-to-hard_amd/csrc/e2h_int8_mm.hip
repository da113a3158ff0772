// int8 per-channel dequant GEMV / skinny GEMM for gfx950.
//
// Replaces  F.linear(x, weight.to(bf16)) * scales  (reference models/quantize.py:428-429).
//
//   q      int8 [N][K] row-major (checkpoint layout),  scales bf16 [N],  x bf16 [M][K],  y bf16 [M][N].
//
// Mapping to v_mfma_f32_16x16x32_bf16 (A = activations, B = weights): lane L = 16*b + c owns weight row
// n0 + c and, per 64-wide k chunk, the 16 consecutive bytes k = 64*chunk + 16*b .. +15 (one 128-bit load).
// Bytes 0..7 feed the first MFMA, bytes 8..15 the second; the activation fragment of lane (b, m) is the
// matching 16 contiguous bytes of x, so neither operand needs a shuffle.  int8 -> bf16 is exact
// (|q| <= 128 fits the 8-bit significand): sign-extending byte convert to float32, then keep the high half.
//
// A workgroup of 4 waves owns 16*T weight rows and 16*MT rows of x; the waves split K in interleaved
// chunks and are summed through LDS in a fixed order.  Epilogue as the reference: round the float32 sum
// to bfloat16 (F.linear's output), multiply by the bfloat16 scale, round again.
#include "e2h_common.h"

namespace e2h {
namespace {

constexpr int kWaves = 4;
constexpr int kChunk = 64;

__device__ __forceinline__ uint32_t pack_bf16_pair_exact(float lo, float hi) {
  // both values are exactly representable in bfloat16: truncation == rounding
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

template <int MT, int T>
struct ChunkRegs8 {
  u32x4_t w[T];
  u32x4_t xf[MT][2];
};

// GUARD: element-wise bounds-checked loads (any K, any alignment).  Otherwise K % 64 == 0 and 16-byte
// aligned rows are required.
template <int MT, int T, bool GUARD>
__global__ __launch_bounds__(kWaves * 64, 2) void int8_generic_mm_kernel(const uint16_t *__restrict__ x, const int8_t *__restrict__ q,
                                                                        const uint16_t *__restrict__ scales, uint16_t *__restrict__ y,
                                                                        int M, int N, int K) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = lane & 15;
  const int b = lane >> 4;
  const int nchunks = (K + kChunk - 1) / kChunk;
  const int n_base = blockIdx.x * (16 * T);
  const int m_base = blockIdx.y * (16 * MT);

  const int8_t *wlane[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int n = n_base + 16 * t + c;
    n = n < N ? n : N - 1;
    wlane[t] = q + static_cast<size_t>(n) * K + 16 * b;
  }
  const uint16_t *xlane[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int row = m_base + 16 * mt + c;
    row = row < M ? row : M - 1;
    xlane[mt] = x + static_cast<size_t>(row) * K + 16 * b;
  }

  f32x4_t acc[T][MT];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  auto load_chunk = [&](ChunkRegs8<MT, T> &r, int ci) {
    const int k0 = ci * kChunk;
    if constexpr (!GUARD) {
#pragma unroll
      for (int t = 0; t < T; ++t) r.w[t] = *reinterpret_cast<const u32x4_t *>(wlane[t] + k0);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        r.xf[mt][0] = *reinterpret_cast<const u32x4_t *>(xlane[mt] + k0);
        r.xf[mt][1] = *reinterpret_cast<const u32x4_t *>(xlane[mt] + k0 + 8);
      }
    } else {
      const int kl = k0 + 16 * b;  // first k of this lane
#pragma unroll
      for (int t = 0; t < T; ++t) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          uint32_t v = 0;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int k = kl + 4 * d + e;
            const uint32_t byte = k < K ? static_cast<uint8_t>(wlane[t][k0 + 4 * d + e]) : 0u;
            v |= byte << (8 * e);
          }
          r.w[t][d] = v;
        }
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            uint32_t v = 0;
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const int k = kl + 8 * s + 2 * d + e;
              const uint32_t h = k < K ? xlane[mt][k0 + 8 * s + 2 * d + e] : 0u;
              v |= h << (16 * e);
            }
            r.xf[mt][s][d] = v;
          }
        }
      }
    }
  };

  auto compute_chunk = [&](const ChunkRegs8<MT, T> &r) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const bf16x8_t w0 = bytes_to_bf16x8(r.w[t][0], r.w[t][1]);
      const bf16x8_t w1 = bytes_to_bf16x8(r.w[t][2], r.w[t][3]);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, r.xf[mt][0]), w0, acc[t][mt], 0, 0, 0);
        acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, r.xf[mt][1]), w1, acc[t][mt], 0, 0, 0);
      }
    }
  };

  ChunkRegs8<MT, T> bufA, bufB;
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

  __shared__ float red[kWaves][T * MT * 4][64];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][(t * MT + mt) * 4 + r][lane] = acc[t][mt][r];
  __syncthreads();
#pragma unroll
  for (int it = 0; it < T * MT; ++it) {
    const int e = it * (kWaves * 64) + threadIdx.x;
    const int L = e & 63;
    const int slot = e >> 6;
    const int r = slot & 3;
    const int mt = (slot >> 2) % MT;
    const int t = (slot >> 2) / MT;
    float s = red[0][slot][L];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) s += red[w][slot][L];
    const int n = n_base + 16 * t + (L & 15);
    const int m = m_base + 16 * mt + 4 * (L >> 4) + r;
    if (n < N && m < M) {
      const float lin = bf16_round(s);                        // F.linear output in bfloat16
      y[static_cast<size_t>(m) * N + n] = f32_to_bf16_rne(lin * bf16_to_f32(scales[n]));  // * self.scales
    }
  }
}

template <int MT, int T>
int launch(bool guard, const uint16_t *x, const int8_t *q, const uint16_t *scales, uint16_t *y, int M, int N, int K,
           hipStream_t stream) {
  dim3 grid((N + 16 * T - 1) / (16 * T), (M + 16 * MT - 1) / (16 * MT));
  if (guard)
    hipLaunchKernelGGL((int8_generic_mm_kernel<MT, T, true>), grid, dim3(kWaves * 64), 0, stream, x, q, scales, y, M, N, K);
  else
    hipLaunchKernelGGL((int8_generic_mm_kernel<MT, T, false>), grid, dim3(kWaves * 64), 0, stream, x, q, scales, y, M, N, K);
  return launch_status();
}

}  // namespace
}  // namespace e2h

extern "C" int e2h_int8_mm(const uint16_t *x, const int8_t *q, const uint16_t *scales, uint16_t *y, int64_t m, int64_t n,
                           int64_t k, void *workspace, int64_t workspace_bytes, void *stream) {
  using namespace e2h;
  if (!x || !q || !scales || !y) return E2H_ERR_NULL_POINTER;
  if (m < 1 || n < 1 || k < 1 || m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(x) & 1u) || (reinterpret_cast<uintptr_t>(y) & 1u) || (reinterpret_cast<uintptr_t>(scales) & 1u))
    return E2H_ERR_MISALIGNED;
  const int M = static_cast<int>(m), N = static_cast<int>(n), K = static_cast<int>(k);
  if (workspace && !aligned16(workspace)) return E2H_ERR_MISALIGNED;
  // streaming kernel: K in whole 128-wide chunks, 16-byte aligned rows, weight matrix below 4 GB
  if ((K % 128) == 0 && aligned16(x) && aligned16(q) && n * k < (int64_t{1} << 32) && !options().int8_force_generic)
    return int8_stream_mm(x, q, scales, y, M, N, K, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
  const bool guard = (K % kChunk) != 0 || !aligned16(x) || !aligned16(q);
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  int t = options().int8_rows_per_wave / 16;
  if (t != 1 && t != 2 && t != 4) {
    const int tiles16 = (N + 15) / 16;
    t = 1;
    if (tiles16 >= 2 * 1024) t = 2;
    if (tiles16 >= 4 * 1024) t = 4;
  }
  if (mt == 4 && t == 4) t = 2;  // 64 rows x 64 columns per wave does not fit the register file
  hipStream_t s = static_cast<hipStream_t>(stream);
#define E2H_CASE(MTV, TV) \
  if (mt == MTV && t == TV) return launch<MTV, TV>(guard, x, q, scales, y, M, N, K, s);
  E2H_CASE(1, 1) E2H_CASE(1, 2) E2H_CASE(1, 4)
  E2H_CASE(2, 1) E2H_CASE(2, 2) E2H_CASE(2, 4)
  E2H_CASE(4, 1) E2H_CASE(4, 2)
#undef E2H_CASE
  return E2H_ERR_BAD_SHAPE;
}

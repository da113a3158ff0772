// Quantization, packing and dequantization kernels (one pass over a weight matrix each; HBM-bound,
// run once per checkpoint or once per on-the-fly conversion).
//
// Bit-exactness contract: the int8 path is IEEE float32 (true division, round-half-even); the int4
// path reproduces torch's bfloat16 elementwise semantics, i.e. every op of the reference is computed
// in float32 and rounded to bfloat16 before the next op.  This file must be compiled without fast-math
// and without FMA contraction.
#include "e2h_common.h"

namespace e2h {
namespace {

// ------------------------------------------------------------------------------------------------
// int8 per-channel (reference models/quantize.py:39-71)
// ------------------------------------------------------------------------------------------------

template <bool BF16>
__device__ __forceinline__ float load_w(const void *w, size_t i) {
  if constexpr (BF16) {
    return bf16_to_f32(static_cast<const uint16_t *>(w)[i]);
  } else {
    return static_cast<const float *>(w)[i];
  }
}

template <bool BF16>
__global__ __launch_bounds__(256) void int8_quantize_rows_kernel(const void *__restrict__ w, int8_t *__restrict__ q,
                                                                 float *__restrict__ scales_f32,
                                                                 uint16_t *__restrict__ scales_bf16, int64_t K) {
  const int64_t row = blockIdx.x;
  const size_t base = static_cast<size_t>(row) * K;
  // max(-min(min_val, 0), max(max_val, 0)) == max |x| over the row  (:49-58)
  float amax = 0.f;
  for (int64_t k = threadIdx.x; k < K; k += blockDim.x) amax = fmaxf(amax, fabsf(load_w<BF16>(w, base + k)));
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  __shared__ float wave_max[4];
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
  float scale = amax / 127.5f;             // :59  float(quant_max - quant_min) / 2
  scale = fmaxf(scale, 1.1920928955078125e-07f);  // :61  clamp(min=float32 eps)
  if (threadIdx.x == 0) {
    if (scales_f32) scales_f32[row] = scale;
    if (scales_bf16) scales_bf16[row] = f32_to_bf16_rne(scale);
  }
  for (int64_t k = threadIdx.x; k < K; k += blockDim.x) {
    float v = load_w<BF16>(w, base + k) / scale;  // :66  true division
    v = rintf(v);                                  // :67  half to even
    v = fminf(fmaxf(v, -128.f), 127.f);            // :69
    q[base + k] = static_cast<int8_t>(static_cast<int>(v));
  }
}

// ------------------------------------------------------------------------------------------------
// int4 group-wise (reference models/quantize.py:74-92, :118-144), bfloat16 arithmetic
// ------------------------------------------------------------------------------------------------

struct GroupQParams {
  float scale, zero;  // bfloat16-exact values
};

__device__ __forceinline__ GroupQParams qparams_from_minmax(float mn, float mx) {
  float r = bf16_round(mx - mn);                  // :88  max_val - min_val
  r = fmaxf(r, bf16_to_f32(0x3586));              // :88  .clamp(min=1e-6); bfloat16(1e-6) = 0x3586
  const float scale = bf16_round(r / 15.0f);      // :88  / max_int
  const float half = bf16_round(scale * 8.0f);    // :89  scales * 2**(n_bit-1)
  const float zero = bf16_round(mn + half);       // :89
  return {scale, zero};
}

__device__ __forceinline__ int quantize_one(float w, float scale, float min_val) {
  float t = bf16_round(w - min_val);  // :136 .sub(min_val)
  t = bf16_round(t / scale);          // :137 .div(scales)
  t = rintf(t);                       // :138 .round()
  t = fminf(fmaxf(t, 0.f), 15.f);     // :139 .clamp_(0, 15)
  return static_cast<int>(t);
}

__device__ __forceinline__ float requant_min(float scale, float zero) {
  return bf16_round(zero - bf16_round(scale * 8.0f));  // :132
}

enum : int { kModeQParams = 0, kModeCodes = 1, kModeFromQParams = 2 };

// One lane handles 8 consecutive k (one 16-byte load); a group is G/8 adjacent lanes of a wave.
// MODE kModeQParams:     writes scales/zeros [N][K/G].
// MODE kModeCodes:       writes codes [N][K] int32 and scales_and_zeros [K/G][N][2].
// MODE kModeFromQParams: reads scales/zeros [N][K/G], writes codes.
template <int G, int MODE>
__global__ __launch_bounds__(256) void int4_group_kernel(const uint16_t *__restrict__ w, uint16_t *__restrict__ scales,
                                                         uint16_t *__restrict__ zeros, int32_t *__restrict__ codes,
                                                         uint16_t *__restrict__ sz, int64_t N, int64_t K) {
  constexpr int LPG = G / 8;
  const int64_t total8 = N * K / 8;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const bool live = idx < total8;
  const int64_t e0 = (live ? idx : total8 - 1) * 8;
  const int64_t n = e0 / K;
  const int64_t k = e0 - n * K;
  const int64_t groups_per_row = K / G;
  const int64_t g = k / G;

  const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(w + e0);
  float v[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __builtin_bit_cast(float, raw[i] << 16);
    v[2 * i + 1] = __builtin_bit_cast(float, raw[i] & 0xFFFF0000u);
  }
  float scale, zero;
  if constexpr (MODE == kModeFromQParams) {
    scale = bf16_to_f32(scales[n * groups_per_row + g]);
    zero = bf16_to_f32(zeros[n * groups_per_row + g]);
  } else {
    float mn = v[0], mx = v[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) {
      mn = fminf(mn, v[i]);
      mx = fmaxf(mx, v[i]);
    }
#pragma unroll
    for (int off = 1; off < LPG; off <<= 1) {
      mn = fminf(mn, __shfl_xor(mn, off));
      mx = fmaxf(mx, __shfl_xor(mx, off));
    }
    const GroupQParams qp = qparams_from_minmax(mn, mx);
    scale = qp.scale;
    zero = qp.zero;
  }
  if (!live) return;
  if constexpr (MODE == kModeQParams) {
    if ((k % G) == 0) {
      scales[n * groups_per_row + g] = f32_to_bf16_rne(scale);
      zeros[n * groups_per_row + g] = f32_to_bf16_rne(zero);
    }
  } else {
    const float min_val = requant_min(scale, zero);
    int32_t out[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = quantize_one(v[i], scale, min_val);
    int4 *dst = reinterpret_cast<int4 *>(codes + e0);
    dst[0] = make_int4(out[0], out[1], out[2], out[3]);
    dst[1] = make_int4(out[4], out[5], out[6], out[7]);
    if constexpr (MODE == kModeCodes) {
      if ((k % G) == 0) {
        const uint32_t pair = static_cast<uint32_t>(f32_to_bf16_rne(scale)) | (static_cast<uint32_t>(f32_to_bf16_rne(zero)) << 16);
        reinterpret_cast<uint32_t *>(sz)[g * N + n] = pair;  // [K/G][N][2]
      }
    }
  }
}

// Generic group size (any g >= 2 dividing K): one thread per group, serial over the group.
template <int MODE>
__global__ __launch_bounds__(256) void int4_group_generic_kernel(const uint16_t *__restrict__ w, uint16_t *__restrict__ scales,
                                                                 uint16_t *__restrict__ zeros, int32_t *__restrict__ codes,
                                                                 uint16_t *__restrict__ sz, int64_t N, int64_t K, int G) {
  const int64_t groups_per_row = K / G;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid >= N * groups_per_row) return;
  const int64_t n = gid / groups_per_row, g = gid - n * groups_per_row;
  const uint16_t *src = w + n * K + g * G;
  float scale, zero;
  if constexpr (MODE == kModeFromQParams) {
    scale = bf16_to_f32(scales[gid]);
    zero = bf16_to_f32(zeros[gid]);
  } else {
    float mn = bf16_to_f32(src[0]), mx = mn;
    for (int i = 1; i < G; ++i) {
      const float v = bf16_to_f32(src[i]);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
    const GroupQParams qp = qparams_from_minmax(mn, mx);
    scale = qp.scale;
    zero = qp.zero;
  }
  if constexpr (MODE == kModeQParams) {
    scales[gid] = f32_to_bf16_rne(scale);
    zeros[gid] = f32_to_bf16_rne(zero);
  } else {
    const float min_val = requant_min(scale, zero);
    for (int i = 0; i < G; ++i) codes[n * K + g * G + i] = quantize_one(bf16_to_f32(src[i]), scale, min_val);
    if constexpr (MODE == kModeCodes) {
      const uint32_t pair = static_cast<uint32_t>(f32_to_bf16_rne(scale)) | (static_cast<uint32_t>(f32_to_bf16_rne(zero)) << 16);
      reinterpret_cast<uint32_t *>(sz)[g * N + n] = pair;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// tile packing (torch.ops.aten._convert_weight_to_int4pack, PyTorch 2.2.0 CUDA nibble order)
// ------------------------------------------------------------------------------------------------

// k offsets (relative to the 32-wide span of a packed word) of nibbles 0..7 for j = t % 4
__device__ __forceinline__ int nibble_k(int i, int j) {
  // nibble i holds v[s], s = {0,2,4,6,1,3,5,7}[i]; v[s] sits at 16*(s>>2) + 8*((s>>1)&1) + (s&1) + 2j
  const int s = (i < 4) ? 2 * i : 2 * (i - 4) + 1;
  return 16 * (s >> 2) + 8 * ((s >> 1) & 1) + (s & 1) + 2 * j;
}

// word index -> (row n, first k of its 32-wide span, j)
struct WordCoord {
  int64_t n, k0;
  int j;
};

__device__ __forceinline__ WordCoord word_coord(int64_t widx, int64_t K, int ikt) {
  const int words = ikt / 2;
  const int64_t kt = K / (16 * ikt);
  const int p = static_cast<int>(widx % words);
  int64_t r = widx / words;
  const int t = static_cast<int>(r % 32);
  r /= 32;
  const int64_t k_outer = r % kt;
  const int64_t n_tile = r / kt;
  return {n_tile * 8 + (t >> 2), (k_outer * ikt + 2 * p) * 16, t & 3};
}

__global__ __launch_bounds__(256) void int4_pack_kernel(const int32_t *__restrict__ codes, uint32_t *__restrict__ packed,
                                                        int64_t N, int64_t K, int ikt) {
  const int64_t widx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (widx >= N * K / 8) return;
  const WordCoord wc = word_coord(widx, K, ikt);
  const int32_t *row = codes + wc.n * K + wc.k0;
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) word |= (static_cast<uint32_t>(row[nibble_k(i, wc.j)]) & 15u) << (4 * i);
  packed[widx] = word;
}

__global__ __launch_bounds__(256) void int4_unpack_kernel(const uint32_t *__restrict__ packed, int32_t *__restrict__ codes,
                                                          int64_t N, int64_t K, int ikt) {
  const int64_t widx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (widx >= N * K / 8) return;
  const WordCoord wc = word_coord(widx, K, ikt);
  int32_t *row = codes + wc.n * K + wc.k0;
  const uint32_t word = packed[widx];
#pragma unroll
  for (int i = 0; i < 8; ++i) row[nibble_k(i, wc.j)] = static_cast<int32_t>((word >> (4 * i)) & 15u);
}

// group_dequantize_tensor_from_qparams (:154-171) on the packed weight: bf16(bf16((q-8)*s) + z)
__global__ __launch_bounds__(256) void int4_dequantize_kernel(const uint32_t *__restrict__ packed, const uint16_t *__restrict__ sz,
                                                              uint16_t *__restrict__ w_out, int64_t N, int64_t K, int G, int ikt) {
  const int64_t widx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (widx >= N * K / 8) return;
  const WordCoord wc = word_coord(widx, K, ikt);
  const uint32_t word = packed[widx];
  const int64_t g = wc.k0 / G;  // a 32-wide span never straddles a group (G >= 32)
  const float scale = bf16_to_f32(sz[(g * N + wc.n) * 2]);
  const float zero = bf16_to_f32(sz[(g * N + wc.n) * 2 + 1]);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float qv = static_cast<float>(static_cast<int>((word >> (4 * i)) & 15u) - 8);
    const float t = bf16_round(qv * scale);
    w_out[wc.n * K + wc.k0 + nibble_k(i, wc.j)] = f32_to_bf16_rne(t + zero);
  }
}


// group_dequantize_tensor_from_qparams (:154-171) on plain int32 codes [N][K] with qparams [N][K/G]
__global__ __launch_bounds__(256) void int4_dequantize_codes_kernel(const int32_t *__restrict__ codes, const uint16_t *__restrict__ scales,
                                                                    const uint16_t *__restrict__ zeros, uint16_t *__restrict__ w_out,
                                                                    int64_t N, int64_t K, int G) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= N * K) return;
  const int64_t n = idx / K, k = idx - n * K;
  const int64_t gi = n * (K / G) + k / G;
  const float t = bf16_round(static_cast<float>(codes[idx] - 8) * bf16_to_f32(scales[gi]));  // :169 .sub(8).mul(scales)
  w_out[idx] = f32_to_bf16_rne(t + bf16_to_f32(zeros[gi]));                                   // :169 .add(zeros)
}

// Fused quantize + pack: a workgroup owns one 8-row tile x 256 k.  Lane layout as int4_group_kernel
// (8 consecutive k per lane); codes go through LDS as bytes and leave as packed words, so the int32
// code matrix (4 bytes per weight) never touches HBM.
template <int G>
__global__ __launch_bounds__(256) void int4_quantize_pack_kernel(const uint16_t *__restrict__ w, uint32_t *__restrict__ packed,
                                                                 uint16_t *__restrict__ sz, int64_t N, int64_t K, int ikt) {
  constexpr int LPG = G / 8;
  constexpr int SPAN = 256;
  __shared__ uint8_t lds_codes[8][SPAN + 16];
  const int64_t spans = K / SPAN;
  const int64_t n_tile = blockIdx.x / spans;
  const int64_t span = blockIdx.x - n_tile * spans;
  const int r = threadIdx.x >> 5;        // row within the tile
  const int kl = (threadIdx.x & 31) * 8;  // k within the span
  const int64_t n = n_tile * 8 + r;
  const int64_t k = span * SPAN + kl;

  const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(w + n * K + k);
  float v[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __builtin_bit_cast(float, raw[i] << 16);
    v[2 * i + 1] = __builtin_bit_cast(float, raw[i] & 0xFFFF0000u);
  }
  float mn = v[0], mx = v[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    mn = fminf(mn, v[i]);
    mx = fmaxf(mx, v[i]);
  }
#pragma unroll
  for (int off = 1; off < LPG; off <<= 1) {
    mn = fminf(mn, __shfl_xor(mn, off));
    mx = fmaxf(mx, __shfl_xor(mx, off));
  }
  const GroupQParams qp = qparams_from_minmax(mn, mx);
  const float min_val = requant_min(qp.scale, qp.zero);
  uint32_t lo = 0, hi = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    lo |= static_cast<uint32_t>(quantize_one(v[i], qp.scale, min_val)) << (8 * i);
    hi |= static_cast<uint32_t>(quantize_one(v[4 + i], qp.scale, min_val)) << (8 * i);
  }
  *reinterpret_cast<uint32_t *>(&lds_codes[r][kl]) = lo;
  *reinterpret_cast<uint32_t *>(&lds_codes[r][kl + 4]) = hi;
  if ((k % G) == 0) {
    const uint32_t pair = static_cast<uint32_t>(f32_to_bf16_rne(qp.scale)) | (static_cast<uint32_t>(f32_to_bf16_rne(qp.zero)) << 16);
    reinterpret_cast<uint32_t *>(sz)[(k / G) * N + n] = pair;
  }
  __syncthreads();

  // 8 rows x 256 k = 256 packed words, contiguous in the packed tensor for this (n_tile, span)
  const int words = ikt / 2;
  const int kblk = 16 * ikt;
  const int64_t kt = K / kblk;
  const int widx_local = threadIdx.x;            // [k_outer_local][t][p]
  const int p = widx_local % words;
  const int t = (widx_local / words) % 32;
  const int ko_local = widx_local / (words * 32);
  const int row = t >> 2, j = t & 3;
  const int k0 = ko_local * kblk + 2 * p * 16;
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) word |= static_cast<uint32_t>(lds_codes[row][k0 + nibble_k(i, j)]) << (4 * i);
  const int64_t k_outer = span * (SPAN / kblk) + ko_local;
  packed[((n_tile * kt + k_outer) * 32 + t) * words + p] = word;
}

inline unsigned blocks_for(int64_t items, int per_block) { return static_cast<unsigned>((items + per_block - 1) / per_block); }

int check_int4_quant_args(const void *w, int64_t n, int64_t k, int g) {
  if (!w) return E2H_ERR_NULL_POINTER;
  if (n < 1 || k < 1 || n * k > (int64_t{1} << 40)) return E2H_ERR_BAD_SHAPE;
  if (g < 2 || k % g != 0) return E2H_ERR_BAD_GROUPSIZE;
  return E2H_OK;
}

bool fast_group(int g) { return g == 32 || g == 64 || g == 128 || g == 256; }

template <int MODE>
int launch_group_kernel(const uint16_t *w, uint16_t *scales, uint16_t *zeros, int32_t *codes, uint16_t *sz, int64_t n,
                        int64_t k, int g, hipStream_t s) {
  if (fast_group(g) && aligned16(w) && (MODE == kModeQParams || aligned16(codes))) {
    const unsigned blocks = blocks_for(n * k / 8, 256);
    switch (g) {
      case 32: hipLaunchKernelGGL((int4_group_kernel<32, MODE>), dim3(blocks), dim3(256), 0, s, w, scales, zeros, codes, sz, n, k); break;
      case 64: hipLaunchKernelGGL((int4_group_kernel<64, MODE>), dim3(blocks), dim3(256), 0, s, w, scales, zeros, codes, sz, n, k); break;
      case 128: hipLaunchKernelGGL((int4_group_kernel<128, MODE>), dim3(blocks), dim3(256), 0, s, w, scales, zeros, codes, sz, n, k); break;
      default: hipLaunchKernelGGL((int4_group_kernel<256, MODE>), dim3(blocks), dim3(256), 0, s, w, scales, zeros, codes, sz, n, k); break;
    }
  } else {
    const unsigned blocks = blocks_for(n * (k / g), 256);
    hipLaunchKernelGGL((int4_group_generic_kernel<MODE>), dim3(blocks), dim3(256), 0, s, w, scales, zeros, codes, sz, n, k, g);
  }
  return launch_status();
}

}  // namespace
}  // namespace e2h

using namespace e2h;

extern "C" int e2h_int8_quantize_per_channel(const void *w, int w_is_bf16, int8_t *q, float *scales_f32,
                                             uint16_t *scales_bf16, int64_t n, int64_t k, void *stream) {
  if (!w || !q) return E2H_ERR_NULL_POINTER;
  if (n < 1 || k < 1 || n > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (w_is_bf16)
    hipLaunchKernelGGL((int8_quantize_rows_kernel<true>), dim3(static_cast<unsigned>(n)), dim3(256), 0, s, w, q, scales_f32, scales_bf16, k);
  else
    hipLaunchKernelGGL((int8_quantize_rows_kernel<false>), dim3(static_cast<unsigned>(n)), dim3(256), 0, s, w, q, scales_f32, scales_bf16, k);
  return launch_status();
}

extern "C" int e2h_int4_group_qparams(const uint16_t *w, uint16_t *scales, uint16_t *zeros, int64_t n, int64_t k,
                                      int groupsize, void *stream) {
  if (int rc = check_int4_quant_args(w, n, k, groupsize)) return rc;
  if (!scales || !zeros) return E2H_ERR_NULL_POINTER;
  return launch_group_kernel<kModeQParams>(w, scales, zeros, nullptr, nullptr, n, k, groupsize, static_cast<hipStream_t>(stream));
}

extern "C" int e2h_int4_quantize_from_qparams(const uint16_t *w, const uint16_t *scales, const uint16_t *zeros,
                                              int32_t *codes, int64_t n, int64_t k, int groupsize, void *stream) {
  if (int rc = check_int4_quant_args(w, n, k, groupsize)) return rc;
  if (!scales || !zeros || !codes) return E2H_ERR_NULL_POINTER;
  return launch_group_kernel<kModeFromQParams>(w, const_cast<uint16_t *>(scales), const_cast<uint16_t *>(zeros), codes, nullptr, n, k,
                                               groupsize, static_cast<hipStream_t>(stream));
}

extern "C" int e2h_int4_group_quantize(const uint16_t *w, int32_t *codes, uint16_t *scales_and_zeros, int64_t n,
                                       int64_t k, int groupsize, void *stream) {
  if (int rc = check_int4_quant_args(w, n, k, groupsize)) return rc;
  if (!codes || !scales_and_zeros) return E2H_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(scales_and_zeros) & 3u) return E2H_ERR_MISALIGNED;
  return launch_group_kernel<kModeCodes>(w, nullptr, nullptr, codes, scales_and_zeros, n, k, groupsize, static_cast<hipStream_t>(stream));
}

static int check_pack_args(const void *a, const void *b, int64_t n, int64_t k, int ikt) {
  if (!a || !b) return E2H_ERR_NULL_POINTER;
  if (ikt != 2 && ikt != 4 && ikt != 8) return E2H_ERR_BAD_INNER_K_TILES;
  if (n < 8 || k < 1 || (n % 8) != 0 || n * k > (int64_t{1} << 40)) return E2H_ERR_BAD_SHAPE;
  if (k % (16 * ikt) != 0) return E2H_ERR_BAD_INNER_K_TILES;
  return E2H_OK;
}

extern "C" int e2h_int4_pack(const int32_t *codes, int32_t *packed, int64_t n, int64_t k, int inner_k_tiles, void *stream) {
  if (int rc = check_pack_args(codes, packed, n, k, inner_k_tiles)) return rc;
  hipLaunchKernelGGL(int4_pack_kernel, dim3(blocks_for(n * k / 8, 256)), dim3(256), 0, static_cast<hipStream_t>(stream), codes,
                     reinterpret_cast<uint32_t *>(packed), n, k, inner_k_tiles);
  return launch_status();
}

extern "C" int e2h_int4_unpack(const int32_t *packed, int32_t *codes, int64_t n, int64_t k, int inner_k_tiles, void *stream) {
  if (int rc = check_pack_args(packed, codes, n, k, inner_k_tiles)) return rc;
  hipLaunchKernelGGL(int4_unpack_kernel, dim3(blocks_for(n * k / 8, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const uint32_t *>(packed), codes, n, k, inner_k_tiles);
  return launch_status();
}

extern "C" int e2h_int4_dequantize(const int32_t *packed, const uint16_t *scales_and_zeros, uint16_t *w_out, int64_t n,
                                   int64_t k, int groupsize, int inner_k_tiles, void *stream) {
  if (int rc = check_pack_args(packed, w_out, n, k, inner_k_tiles)) return rc;
  if (!scales_and_zeros) return E2H_ERR_NULL_POINTER;
  if (!fast_group(groupsize) || k % groupsize != 0) return E2H_ERR_BAD_GROUPSIZE;
  hipLaunchKernelGGL(int4_dequantize_kernel, dim3(blocks_for(n * k / 8, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const uint32_t *>(packed), scales_and_zeros, w_out, n, k, groupsize, inner_k_tiles);
  return launch_status();
}

extern "C" int e2h_int4_dequantize_codes(const int32_t *codes, const uint16_t *scales, const uint16_t *zeros, uint16_t *w_out,
                                         int64_t n, int64_t k, int groupsize, void *stream) {
  if (!codes || !scales || !zeros || !w_out) return E2H_ERR_NULL_POINTER;
  if (n < 1 || k < 1 || n * k > (int64_t{1} << 40)) return E2H_ERR_BAD_SHAPE;
  if (groupsize < 2 || k % groupsize != 0) return E2H_ERR_BAD_GROUPSIZE;
  hipLaunchKernelGGL(int4_dequantize_codes_kernel, dim3(blocks_for(n * k, 256)), dim3(256), 0, static_cast<hipStream_t>(stream), codes,
                     scales, zeros, w_out, n, k, groupsize);
  return launch_status();
}

extern "C" int e2h_int4_quantize_pack(const uint16_t *w, int32_t *packed, uint16_t *scales_and_zeros, int64_t n, int64_t k,
                                      int groupsize, int inner_k_tiles, void *stream) {
  if (int rc = check_pack_args(w, packed, n, k, inner_k_tiles)) return rc;
  if (!scales_and_zeros) return E2H_ERR_NULL_POINTER;
  if (!fast_group(groupsize) || k % groupsize != 0) return E2H_ERR_BAD_GROUPSIZE;
  if (!aligned16(w) || (reinterpret_cast<uintptr_t>(scales_and_zeros) & 3u) || (reinterpret_cast<uintptr_t>(packed) & 3u))
    return E2H_ERR_MISALIGNED;
  if (k % 256 != 0) return E2H_ERR_BAD_SHAPE;  // callers fall back to quantize + pack
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned blocks = static_cast<unsigned>((n / 8) * (k / 256));
  uint32_t *out = reinterpret_cast<uint32_t *>(packed);
  switch (groupsize) {
    case 32: hipLaunchKernelGGL((int4_quantize_pack_kernel<32>), dim3(blocks), dim3(256), 0, s, w, out, scales_and_zeros, n, k, inner_k_tiles); break;
    case 64: hipLaunchKernelGGL((int4_quantize_pack_kernel<64>), dim3(blocks), dim3(256), 0, s, w, out, scales_and_zeros, n, k, inner_k_tiles); break;
    case 128: hipLaunchKernelGGL((int4_quantize_pack_kernel<128>), dim3(blocks), dim3(256), 0, s, w, out, scales_and_zeros, n, k, inner_k_tiles); break;
    default: hipLaunchKernelGGL((int4_quantize_pack_kernel<256>), dim3(blocks), dim3(256), 0, s, w, out, scales_and_zeros, n, k, inner_k_tiles); break;
  }
  return launch_status();
}

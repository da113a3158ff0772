// Next-token sampling for one decode step (HBM / L2-bound, one workgroup per sequence).
//
// Replaces  sample() -> logits_to_probs() -> multinomial_sample_one_no_sync()
// (reference inference_generate.py:53-85) on the logits of the last position:
//
//   l      = float(logits) / max(temperature, 1e-5)
//   pivot  = k-th largest l of the row                  (top_k given)
//   l      = l < pivot ? -inf : l
//   probs  = softmax(l)                                   (float32, written out: the reference returns them)
//   idx    = argmax(probs / q)                            q ~ Exp(1), drawn by the caller (the reference draws it with
//                                                         torch.empty_like(probs).exponential_(1))
//
// The pivot is found exactly with a 4-pass radix select over order-preserving 32-bit keys (256-bin histograms in
// LDS), so ties at the pivot keep every tied logit, as torch.where(logits < pivot) does.  The row (vocab * 2 bytes)
// is re-read from L2 for every pass; nothing but probs and the index is written.
#include "e2h_common.h"

#include <cfloat>

namespace e2h {
namespace {

constexpr int kSampleThreads = 1024;

__device__ __forceinline__ uint32_t order_key(float f) {  // larger float <=> larger key
  const uint32_t u = __builtin_bit_cast(uint32_t, f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float block_reduce_max(float v, float *scratch) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = scratch[0];
  for (int w = 1; w < kSampleThreads / 64; ++w) r = fmaxf(r, scratch[w]);
  __syncthreads();
  return r;
}

__device__ __forceinline__ float block_reduce_sum(float v, float *scratch) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = 0.f;
  for (int w = 0; w < kSampleThreads / 64; ++w) r += scratch[w];  // fixed order: deterministic
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(kSampleThreads) void sample_top_k_kernel(const uint16_t *__restrict__ logits, int64_t row_stride,
                                                                      const float *__restrict__ q, float *__restrict__ probs,
                                                                      int32_t *__restrict__ idx_out, int vocab, float inv_t_div,
                                                                      int top_k) {
  __shared__ unsigned hist[256];
  __shared__ float scratch[kSampleThreads / 64];
  __shared__ unsigned s_prefix, s_remaining;
  __shared__ float s_best[kSampleThreads / 64];
  __shared__ int s_best_i[kSampleThreads / 64];

  const int row = blockIdx.x;
  const uint16_t *lrow = logits + static_cast<int64_t>(row) * row_stride;
  auto value = [&](int i) { return bf16_to_f32(lrow[i]) / inv_t_div; };  // true division, as logits / max(temperature, 1e-5)

  // ---- pivot: k-th largest value, by radix select on the keys -------------------------------------
  float pivot = -INFINITY;
  if (top_k > 0 && top_k < vocab) {
    unsigned prefix = 0, remaining = static_cast<unsigned>(top_k);
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      const unsigned mask = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8));
      for (int i = threadIdx.x; i < 256; i += kSampleThreads) hist[i] = 0;
      __syncthreads();
      for (int i = threadIdx.x; i < vocab; i += kSampleThreads) {
        const uint32_t key = order_key(value(i));
        if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
      }
      __syncthreads();
      if (threadIdx.x == 0) {
        unsigned rem = remaining;
        int bin = 255;
        for (; bin > 0; --bin) {  // walk down from the largest digit until the k-th element's bin
          if (hist[bin] >= rem) break;
          rem -= hist[bin];
        }
        s_prefix = prefix | (static_cast<unsigned>(bin) << shift);
        s_remaining = rem;
      }
      __syncthreads();
      prefix = s_prefix;
      remaining = s_remaining;
    }
    const uint32_t u = (prefix & 0x80000000u) ? (prefix & 0x7FFFFFFFu) : ~prefix;
    pivot = __builtin_bit_cast(float, u);
  }

  // ---- masked softmax -----------------------------------------------------------------------------
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < vocab; i += kSampleThreads) {
    const float v = value(i);
    if (!(v < pivot)) mx = fmaxf(mx, v);
  }
  mx = block_reduce_max(mx, scratch);
  float sum = 0.f;
  for (int i = threadIdx.x; i < vocab; i += kSampleThreads) {
    const float v = value(i);
    if (!(v < pivot)) sum += expf(v - mx);
  }
  sum = block_reduce_sum(sum, scratch);

  // ---- probs out, exponential race ------------------------------------------------------------------
  float best = -INFINITY;
  int best_i = 0x7FFFFFFF;
  float *prow = probs + static_cast<int64_t>(row) * vocab;
  const float *qrow = q + static_cast<int64_t>(row) * vocab;
  for (int i = threadIdx.x; i < vocab; i += kSampleThreads) {
    const float v = value(i);
    const float p = (v < pivot) ? 0.f : expf(v - mx) / sum;
    prow[i] = p;
    const float score = p / qrow[i];
    if (score > best || (score == best && i < best_i)) {
      best = score;
      best_i = i;
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ob = __shfl_xor(best, off);
    const int oi = __shfl_xor(best_i, off);
    if (ob > best || (ob == best && oi < best_i)) {
      best = ob;
      best_i = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    s_best[threadIdx.x >> 6] = best;
    s_best_i[threadIdx.x >> 6] = best_i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kSampleThreads / 64; ++w)
      if (s_best[w] > best || (s_best[w] == best && s_best_i[w] < best_i)) {
        best = s_best[w];
        best_i = s_best_i[w];
      }
    idx_out[row] = best_i == 0x7FFFFFFF ? 0 : best_i;
  }
}

// Greedy choice: argmax(float(logits)) per row (reference inference_generate.py: the temperature-0 / greedy path of the
// harness, torch.argmax over the last position's logits).  Ties go to the lowest index and a NaN counts as the
// largest value, as in ATen's arg-max reduction.  One workgroup per row, 16-byte loads where the row allows them.
__device__ __forceinline__ uint32_t argmax_key(uint32_t bf16_bits) {  // larger value <=> larger key, NaN above +inf
  const uint32_t u = bf16_bits << 16;
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0xFFFFFFFFu;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(kSampleThreads) void argmax_rows_kernel(const uint16_t *__restrict__ logits, int64_t row_stride,
                                                                     int64_t *__restrict__ out, int vocab) {
  __shared__ unsigned long long s_best[kSampleThreads / 64];
  const uint16_t *row = logits + static_cast<size_t>(blockIdx.x) * row_stride;
  // candidate = (key << 32) | ~index: the maximum is the largest key and, among equals, the smallest index
  unsigned long long best = 0ull;
  auto offer = [&](uint32_t bits, int i) {
    const unsigned long long cand = (static_cast<unsigned long long>(argmax_key(bits)) << 32) | static_cast<uint32_t>(~static_cast<uint32_t>(i));
    best = cand > best ? cand : best;
  };
  if ((reinterpret_cast<uintptr_t>(row) & 15u) == 0) {
    const int pieces = vocab / 8;
    for (int p = threadIdx.x; p < pieces; p += kSampleThreads) {
      const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(row + p * 8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        offer(raw[j] & 0xFFFFu, p * 8 + 2 * j);
        offer(raw[j] >> 16, p * 8 + 2 * j + 1);
      }
    }
    for (int i = pieces * 8 + threadIdx.x; i < vocab; i += kSampleThreads) offer(row[i], i);
  } else {
    for (int i = threadIdx.x; i < vocab; i += kSampleThreads) offer(row[i], i);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const unsigned long long other = __shfl_xor(best, off);
    best = other > best ? other : best;
  }
  if ((threadIdx.x & 63) == 0) s_best[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kSampleThreads / 64; ++w) best = s_best[w] > best ? s_best[w] : best;
    out[blockIdx.x] = static_cast<int64_t>(~static_cast<uint32_t>(best & 0xFFFFFFFFull));
  }
}

}  // namespace
}  // namespace e2h

extern "C" int e2h_argmax_rows(const uint16_t *logits, int64_t row_stride, int64_t *idx, int64_t rows, int64_t vocab, void *stream) {
  using namespace e2h;
  if (!logits || !idx) return E2H_ERR_NULL_POINTER;
  if (rows < 1 || vocab < 1 || rows > INT32_MAX || vocab > INT32_MAX || row_stride < vocab) return E2H_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(logits) & 1u) || (reinterpret_cast<uintptr_t>(idx) & 7u)) return E2H_ERR_MISALIGNED;
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(static_cast<unsigned>(rows)), dim3(kSampleThreads), 0, static_cast<hipStream_t>(stream), logits,
                     row_stride, idx, static_cast<int>(vocab));
  return launch_status();
}

extern "C" int e2h_sample_top_k(const uint16_t *logits, int64_t row_stride, const float *q, float *probs, int32_t *idx,
                                int64_t rows, int64_t vocab, float temperature, int top_k, void *stream) {
  using namespace e2h;
  if (!logits || !q || !probs || !idx) return E2H_ERR_NULL_POINTER;
  if (rows < 1 || vocab < 1 || rows > INT32_MAX || vocab > INT32_MAX || row_stride < vocab || top_k < 0) return E2H_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(logits) & 1u) || (reinterpret_cast<uintptr_t>(q) & 3u) || (reinterpret_cast<uintptr_t>(probs) & 3u) ||
      (reinterpret_cast<uintptr_t>(idx) & 3u))
    return E2H_ERR_MISALIGNED;
  const float t = temperature > 1e-5f ? temperature : 1e-5f;
  hipLaunchKernelGGL(sample_top_k_kernel, dim3(static_cast<unsigned>(rows)), dim3(kSampleThreads), 0, static_cast<hipStream_t>(stream), logits,
                     row_stride, q, probs, idx, static_cast<int>(vocab), t, top_k);
  return launch_status();
}

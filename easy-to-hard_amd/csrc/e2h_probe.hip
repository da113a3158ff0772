// Streaming-read probe: what a launch that does nothing but read `bytes` of HBM costs on this machine.
//
// No reference counterpart: it is the yardstick the decode-batch matmuls are measured against (their weights are
// read exactly once, so no launch that has to read them can be faster than this one launched the same way).
// 256 workgroups of 8 waves; every wave walks its share with 16-byte streaming loads, eight in flight (8 KB per wave,
// 64 KB per CU); the values are folded into one word per lane that is stored only if it equals a value it cannot
// take, so that the loads are not optimised away and the launch writes nothing.
// Optionally every workgroup also reads one shared region in full (its eight waves an eighth each, requests interleaved
// with the streaming ones): the access pattern of a decode-batch matmul's activations, which every CU needs whole.
#include "e2h_common.h"

namespace e2h {
namespace {

constexpr int kProbeWgs = 256, kProbeThreads = 512, kProbeDepth = 8;

template <bool kShared>
__global__ __launch_bounds__(kProbeThreads) void stream_read_probe_kernel(const uint8_t *__restrict__ src, uint32_t pieces,
                                                                          const uint8_t *__restrict__ shared, uint32_t shared_pieces,
                                                                          uint32_t *__restrict__ sink) {
  // piece = 16 bytes; lane-contiguous: a wave-wide load covers 1 KB of consecutive memory
  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(src, pieces * 16u);
  const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(shared, shared_pieces * 16u);
  const uint32_t stride = kProbeWgs * kProbeThreads;
  uint32_t p = blockIdx.x * kProbeThreads + threadIdx.x;
  uint32_t q = threadIdx.x;  // the shared region: every workgroup all of it
  uint32_t acc = 0u;
  while (p < pieces || (kShared && q < shared_pieces)) {
    u32x4_t v[kProbeDepth], w[kProbeDepth];
#pragma unroll
    for (int i = 0; i < kProbeDepth; ++i) {
      // out-of-range requests of a buffer load return zero without touching memory
      v[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (p + i * stride) * 16u, 0, 2);
      if constexpr (kShared) w[i] = __builtin_amdgcn_raw_buffer_load_b128(srsrc, (q + i * kProbeThreads) * 16u, 0, 0);
      else w[i] = u32x4_t{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < kProbeDepth; ++i) acc ^= v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3] ^ w[i][0] ^ w[i][3];
    p = p + kProbeDepth * stride < p ? pieces : p + kProbeDepth * stride;
    q += kProbeDepth * kProbeThreads;
  }
  if (acc == 0x9E3779B9u && sink) sink[threadIdx.x] = acc;  // practically never: keeps the loads alive
}

}  // namespace
}  // namespace e2h

extern "C" int e2h_stream_read_probe(const void *src, int64_t bytes, const void *shared, int64_t shared_bytes, uint32_t *sink, void *stream) {
  using namespace e2h;
  if (bytes < 0 || bytes >= (int64_t{1} << 31) || (bytes % 16) != 0) return E2H_ERR_BAD_SHAPE;
  if (shared_bytes < 0 || shared_bytes >= (int64_t{1} << 31) || (shared_bytes % 16) != 0) return E2H_ERR_BAD_SHAPE;
  if ((bytes > 0 && !src) || (shared_bytes > 0 && !shared)) return E2H_ERR_NULL_POINTER;
  if (!aligned16(src) || !aligned16(shared)) return E2H_ERR_MISALIGNED;
  const auto kernel = shared_bytes > 0 ? stream_read_probe_kernel<true> : stream_read_probe_kernel<false>;
  hipLaunchKernelGGL(kernel, dim3(kProbeWgs), dim3(kProbeThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint8_t *>(src), static_cast<uint32_t>(bytes / 16), static_cast<const uint8_t *>(shared),
                     static_cast<uint32_t>(shared_bytes / 16), sink);
  return launch_status();
}

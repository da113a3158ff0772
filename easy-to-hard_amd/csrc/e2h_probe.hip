// Streaming-read probe: what a launch that does nothing but read `bytes` of HBM costs on this machine.
//
// No reference counterpart: it is the yardstick the decode-batch matmuls are measured against (their weights are
// read exactly once, so no launch that has to read them can be faster than this one launched the same way).
// 256 workgroups of 8 waves; every wave walks its share with 16-byte streaming loads, eight in flight (8 KB per wave,
// 64 KB per CU); the values are folded into one word per lane that is stored only if it equals a value it cannot
// take, so that the loads are not optimised away and the launch writes nothing.
#include "e2h_common.h"

namespace e2h {
namespace {

constexpr int kProbeWgs = 256, kProbeThreads = 512, kProbeDepth = 8;

__global__ __launch_bounds__(kProbeThreads) void stream_read_probe_kernel(const uint8_t *__restrict__ src, uint32_t pieces, uint32_t *__restrict__ sink) {
  // piece = 16 bytes; lane-contiguous: a wave-wide load covers 1 KB of consecutive memory
  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(src, pieces * 16u);
  const uint32_t stride = kProbeWgs * kProbeThreads;
  uint32_t p = blockIdx.x * kProbeThreads + threadIdx.x;
  uint32_t acc = 0u;
  for (; p + (kProbeDepth - 1) * stride < pieces; p += kProbeDepth * stride) {
    u32x4_t v[kProbeDepth];
#pragma unroll
    for (int i = 0; i < kProbeDepth; ++i) v[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (p + i * stride) * 16u, 0, 2);
#pragma unroll
    for (int i = 0; i < kProbeDepth; ++i) acc ^= v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3];
  }
  for (; p < pieces; p += stride) {
    const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, p * 16u, 0, 2);
    acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (acc == 0x9E3779B9u && sink) sink[threadIdx.x] = acc;  // practically never: keeps the loads alive
}

}  // namespace
}  // namespace e2h

extern "C" int e2h_stream_read_probe(const void *src, int64_t bytes, uint32_t *sink, void *stream) {
  using namespace e2h;
  if (bytes < 0 || bytes >= (int64_t{1} << 32) || (bytes % 16) != 0) return E2H_ERR_BAD_SHAPE;
  if (bytes > 0 && !src) return E2H_ERR_NULL_POINTER;
  if (!aligned16(src)) return E2H_ERR_MISALIGNED;
  hipLaunchKernelGGL(stream_read_probe_kernel, dim3(kProbeWgs), dim3(kProbeThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint8_t *>(src), static_cast<uint32_t>(bytes / 16), sink);
  return launch_status();
}

"""The reference's CPU execution path for a weight-only quantized linear, restated with torch CPU ops.

TEST AND CPU-BASELINE INFRASTRUCTURE ONLY (same rule as quant_oracle.py): used as the timed CPU baseline of the
benchmark and as a cross-check in tests, never by the shipped package.

  int8:  F.linear(x, weight.to(x.dtype)) * scales                       reference models/quantize.py:428-429
  int4:  W = ((q - 8) * scale + zero) in bfloat16 (:154-171), then F.linear(x, W); this is what
         "dequantize + F.linear" means for a machine without the aten int4 kernels (:445-453).
"""

import torch
import torch.nn.functional as F


def int8_linear_cpu(x, q, scales):
    """x bf16 [M, K], q int8 [N, K], scales bf16 [N] -> bf16 [M, N]."""
    return F.linear(x, q.to(dtype=x.dtype)) * scales


def int4_dequantize_cpu(codes, scales_and_zeros, groupsize):
    """codes int32 [N, K], scales_and_zeros bf16 [K/g, N, 2] -> bf16 [N, K] (bf16 arithmetic per op)."""
    n, k = codes.shape
    sz = scales_and_zeros.transpose(0, 1)  # [N, K/g, 2]
    scales = sz[..., 0].reshape(-1, 1)
    zeros = sz[..., 1].reshape(-1, 1)
    return codes.reshape(-1, groupsize).sub(8).mul(scales).add(zeros).reshape(n, k)


def int4_linear_cpu(x, codes, scales_and_zeros, groupsize):
    """x bf16 [M, K] -> bf16 [M, N]: dequantize the whole weight, then F.linear."""
    return F.linear(x, int4_dequantize_cpu(codes, scales_and_zeros, groupsize))

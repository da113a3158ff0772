"""Pins oracle.int8_quantize_per_channel / int8_linear_* against independent evidence (CPU only)."""

import numpy as np
import pytest
import torch

from oracle import quant_oracle as qo
from tests.helpers import randn_bf16, weight_with_edge_rows


def _inputs():
    w = weight_with_edge_rows(64, 512, 128).float()
    w[7, 3] = 1e-30  # tiny value next to zeros
    return w


def test_scales_match_library_observer():
    # torch.ao's per-channel symmetric observer is a library routine with the same divisor (quant_max -
    # quant_min) / 2 and the same eps clamp; it knows nothing about this repository's oracle.
    from torch.ao.quantization.observer import PerChannelMinMaxObserver

    w = _inputs()
    obs = PerChannelMinMaxObserver(ch_axis=0, dtype=torch.qint8, qscheme=torch.per_channel_symmetric,
                                   quant_min=-128, quant_max=127)
    obs(w)
    scale_lib, zp_lib = obs.calculate_qparams()
    _, scales, zps = qo.int8_quantize_per_channel(w.numpy())
    np.testing.assert_array_equal(scales, scale_lib.numpy().astype(np.float32))
    assert np.all(zps == 0) and torch.all(zp_lib == 0)


def test_codes_match_torch_cpu_op_chain():
    # the reference's op sequence executed by torch's CPU kernels (independent division / rounding code)
    w = _inputs()
    mn, mx = torch.aminmax(w, dim=1)
    amax = torch.max(-torch.min(mn, torch.zeros_like(mn)), torch.max(mx, torch.zeros_like(mx)))
    scales_t = torch.clamp(amax / (float(127 - (-128)) / 2), min=torch.finfo(torch.float32).eps)
    q_t = torch.clamp(torch.round(w / scales_t.unsqueeze(-1)), -128, 127).to(torch.int8)
    q, scales, _ = qo.int8_quantize_per_channel(w.numpy())
    np.testing.assert_array_equal(scales, scales_t.numpy())
    np.testing.assert_array_equal(q, q_t.numpy())


def test_scalar_brute_force_and_invariants():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((6, 33)).astype(np.float32)
    x[2] = 0
    q, scales, _ = qo.int8_quantize_per_channel(x)
    for i in range(x.shape[0]):
        amax = max(abs(float(v)) for v in x[i])
        s = np.float32(max(np.float32(np.float32(amax) / np.float32(127.5)), np.float32(2.0**-23)))
        assert scales[i] == s
        for j in range(x.shape[1]):
            v = np.float32(x[i, j]) / s
            r = float(np.round(np.float64(v)))  # numpy rounds half to even
            assert q[i, j] == int(min(max(r, -128), 127))
    # reconstruction within half a step (the +127.5 -> 127 clamp costs at most one more half step)
    err = np.abs(q.astype(np.float64) * scales[:, None] - x)
    assert np.all(err <= 0.5 * scales[:, None] * (1 + 1e-6) + (q == 127) * 0.5 * scales[:, None])
    assert q.min() >= -128 and q.max() <= 127
    # the extreme element of every non-zero row maps to +-127/128
    nz = np.abs(x).max(axis=1) > 0
    assert np.all(np.abs(q[nz].astype(np.int32)).max(axis=1) >= 127)
    # the all-zero row: eps scale, zero codes
    assert scales[2] == np.float32(2.0**-23) and np.all(q[2] == 0)


def test_half_even_rounding_and_negative_extreme():
    # row max 127.5 -> scale exactly 1: 0.5 -> 0, 1.5 -> 2, 2.5 -> 2, -127.5 -> -128, +127.5 -> 128 -> clamp 127
    x = np.array([[127.5, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5],
                  [-127.5, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, -126.5]], dtype=np.float32)
    q, scales, _ = qo.int8_quantize_per_channel(x)
    assert np.all(scales == 1.0)
    np.testing.assert_array_equal(q[0], [127, 0, 2, 2, 0, -2, -2, 126])
    np.testing.assert_array_equal(q[1], [-128, 0, 2, 2, 0, -2, -2, -126])


def test_linear_oracles_against_float64_and_library_kernel():
    n, k, m = 48, 256, 5
    w = randn_bf16((n, k), std=0.02).float()
    q, scales, _ = qo.int8_quantize_per_channel(w.numpy())
    s_bf16 = qo.bf16_round(scales)
    x = randn_bf16((m, k))
    xf = x.float().numpy()
    y = qo.int8_linear_fp32(xf, q, s_bf16)
    # brute force
    ref = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            ref[i, j] = float(np.dot(xf[i].astype(np.float64), q[j].astype(np.float64))) * float(s_bf16[j])
    np.testing.assert_allclose(y, ref, rtol=1e-6, atol=1e-7)
    # library kernel of the same contract (bf16 output -> loose tolerance)
    y_lib = torch.ops.aten._weight_int8pack_mm(x, torch.from_numpy(q), torch.from_numpy(s_bf16).to(torch.bfloat16))
    assert qo.normwise_rel_err(y_lib.float().numpy(), y) < 1e-2
    # the reference-rounding variant differs from the exact form by at most ~2 bf16 ulps
    y_rr = qo.int8_linear_reference_rounding(xf, q, s_bf16)
    assert qo.is_bf16_exact(y_rr)
    assert qo.normwise_rel_err(y_rr, y) < 2 ** -7

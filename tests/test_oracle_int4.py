"""Pins the int4 group-wise oracle (qparams, codes, dequant, scales_and_zeros layout) on the CPU."""

import struct

import numpy as np
import pytest
import torch

from oracle import quant_oracle as qo
from tests.helpers import bf16_to_np, randn_bf16, weight_with_edge_rows

GROUPS = [32, 64, 128, 256]


def _torch_chain(w, g):
    """The reference's op sequence (models/quantize.py:82-92, :127-141) run by torch's CPU bfloat16 kernels."""
    tq = w.reshape(-1, g)
    mx = tq.amax(dim=1, keepdim=True)
    mn = tq.amin(dim=1, keepdim=True)
    scales = (mx - mn).clamp(min=1e-6) / 15
    zeros = mn + scales * 8
    assert scales.dtype == torch.bfloat16 and zeros.dtype == torch.bfloat16
    min_val = zeros - scales * 8
    codes = tq.sub(min_val).div(scales).round().clamp_(0, 15).to(torch.int32).reshape_as(w)
    return scales.reshape(w.shape[0], -1), zeros.reshape(w.shape[0], -1), codes


@pytest.mark.parametrize("g", GROUPS)
def test_against_torch_cpu_bf16_kernels(g):
    w = weight_with_edge_rows(32, 1024, g)
    s_t, z_t, c_t = _torch_chain(w, g)
    wf = bf16_to_np(w)
    s, z = qo.int4_group_qparams(wf, 4, g)
    np.testing.assert_array_equal(s, bf16_to_np(s_t))
    np.testing.assert_array_equal(z, bf16_to_np(z_t))
    codes = qo.int4_quantize_from_qparams(wf, s, z, 4, g)
    np.testing.assert_array_equal(codes, c_t.numpy())
    codes2, sz = qo.int4_group_quantize(wf, 4, g)
    np.testing.assert_array_equal(codes2, codes)
    assert sz.shape == (1024 // g, 32, 2)
    # large-magnitude and tiny-magnitude weights go through the same roundings
    for std in (5.0, 1e-4):
        w2 = randn_bf16((8, 512), std=std, seed=99)
        s_t, z_t, c_t = _torch_chain(w2, g)
        c2, sz2 = qo.int4_group_quantize(bf16_to_np(w2), 4, g)
        np.testing.assert_array_equal(c2, c_t.numpy())
        np.testing.assert_array_equal(sz2[:, :, 0].T, bf16_to_np(s_t))
        np.testing.assert_array_equal(sz2[:, :, 1].T, bf16_to_np(z_t))


def _bf16_py(x):
    """Round a Python float (via float32) to bfloat16 with pure integer arithmetic."""
    u = struct.unpack("<I", struct.pack("<f", x))[0]
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFFFFFF
    return struct.unpack("<f", struct.pack("<I", (u >> 16) << 16))[0]


def _f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


def test_scalar_brute_force():
    g = 32
    w = bf16_to_np(weight_with_edge_rows(8, 64, g, seed=5))
    s, z = qo.int4_group_qparams(w, 4, g)
    codes = qo.int4_quantize_from_qparams(w, s, z, 4, g)
    for n in range(8):
        for gi in range(64 // g):
            grp = [float(v) for v in w[n, gi * g:(gi + 1) * g]]
            mx, mn = max(grp), min(grp)
            r = _bf16_py(_f32(mx - mn))
            r = max(r, _bf16_py(1e-6))
            scale = _bf16_py(_f32(r / 15.0))
            zero = _bf16_py(_f32(mn + _bf16_py(_f32(scale * 8.0))))
            assert s[n, gi] == np.float32(scale) and z[n, gi] == np.float32(zero)
            min_val = _bf16_py(_f32(zero - _bf16_py(_f32(scale * 8.0))))
            for i, v in enumerate(grp):
                t = _bf16_py(_f32(v - min_val))
                t = _bf16_py(float(np.float32(t) / np.float32(scale)))
                qv = int(min(max(round(t), 0), 15))  # Python round() is half-to-even
                assert codes[n, gi * g + i] == qv


@pytest.mark.parametrize("g", GROUPS)
def test_invariants(g):
    w = bf16_to_np(randn_bf16((64, 1024), std=0.02, seed=3))
    codes, sz = qo.int4_group_quantize(w, 4, g)
    assert codes.dtype == np.int32 and codes.min() >= 0 and codes.max() <= 15
    grouped_w = w.reshape(-1, g)
    grouped_c = codes.reshape(-1, g)
    # the group maximum quantizes to 15 and the minimum to 0 (up to one step from bf16 rounding of qparams)
    assert np.all(grouped_c[np.arange(len(grouped_w)), grouped_w.argmax(1)] >= 14)
    assert np.all(grouped_c[np.arange(len(grouped_w)), grouped_w.argmin(1)] <= 1)
    assert np.mean(grouped_c.max(1) == 15) > 0.95 and np.mean(grouped_c.min(1) == 0) > 0.95
    # reconstruction error <= scale/2 plus the bf16 roundings of scale / zero (relative 2^-8 each)
    deq = qo.int4_dequantize_fp32(codes, sz, g)
    scale_full = np.repeat(sz[:, :, 0].T, g, axis=1)
    slack = 2.0 ** -7 * (np.abs(w) + 16 * scale_full)
    assert np.all(np.abs(deq - w) <= 0.5 * scale_full + slack)
    # a dropped "+ 8*scale" / wrong sign in the zero point would shift every code by 8
    assert 6.5 < grouped_c.mean() < 8.5


def test_constant_and_zero_groups_closed_form():
    g = 32
    w = np.zeros((8, 64), dtype=np.float32)
    w[1] = 0.5
    s, z = qo.int4_group_qparams(w, 4, g)
    s_const = qo.bf16_round(qo.bf16_round(np.float32(1e-6)) / np.float32(15))
    assert np.all(s == s_const)
    assert qo.bf16_bits(s_const) == 0x338F and qo.bf16_bits(qo.bf16_round(np.float32(1e-6))) == 0x3586
    np.testing.assert_array_equal(z[0], qo.bf16_round(qo.bf16_round(s_const * 8)))
    np.testing.assert_array_equal(z[1], qo.bf16_round(np.float32(0.5) + qo.bf16_round(s_const * 8)))
    codes = qo.int4_quantize_from_qparams(w, s, z, 4, g)
    # zero group: zero = 8s, min' = zero - 8s = 0, so (0 - 0)/s = 0; constant 0.5: 0.5 +- 8s rounds back to 0.5,
    # min' = 0.5 and the code is 0 again.  Dequantized: (0 - 8)*s + zero = 0 resp. 0.5 - 8s (within 5.4e-7).
    assert np.all(codes[0] == 0)
    assert np.all(codes[1] == 0)
    sz = qo.pack_scales_and_zeros(s, z)
    deq = qo.int4_dequantize_fp32(codes, sz, g)
    assert np.all(deq[0] == 0) and np.all(np.abs(deq[1] - 0.5) < 1e-6)


def test_scales_and_zeros_layout_and_dequant():
    g = 64
    w = bf16_to_np(randn_bf16((16, 256), std=0.02, seed=11))
    s, z = qo.int4_group_qparams(w, 4, g)
    sz = qo.pack_scales_and_zeros(s, z)
    assert sz.shape == (4, 16, 2) and sz.flags["C_CONTIGUOUS"]
    for gi in range(4):
        for n in range(16):
            assert sz[gi, n, 0] == s[n, gi] and sz[gi, n, 1] == z[n, gi]
    s2, z2 = qo.unpack_scales_and_zeros(sz)
    np.testing.assert_array_equal(s2, s)
    np.testing.assert_array_equal(z2, z)
    # the torch restatement of the same shuffle (reference :95-109)
    ts, tz = torch.from_numpy(s), torch.from_numpy(z)
    t = torch.cat([ts.reshape(16, 4, 1), tz.reshape(16, 4, 1)], 2).transpose(0, 1).contiguous()
    np.testing.assert_array_equal(sz, t.numpy())
    codes = qo.int4_quantize_from_qparams(w, s, z, 4, g)
    deq_bf16 = qo.int4_dequantize_from_qparams(codes, s, z, 4, g)
    deq_f32 = qo.int4_dequantize_fp32(codes, sz, g)
    assert qo.is_bf16_exact(deq_bf16)
    for n in (0, 7, 15):
        for k in (0, 63, 64, 255):
            exact = (int(codes[n, k]) - 8) * float(s[n, k // g]) + float(z[n, k // g])
            assert abs(float(deq_f32[n, k]) - exact) <= 1e-7 * max(1.0, abs(exact))
            t1 = _bf16_py(_f32((int(codes[n, k]) - 8) * float(s[n, k // g])))
            assert float(deq_bf16[n, k]) == _bf16_py(_f32(t1 + float(z[n, k // g])))
    # torch's own promotion rules for int32 * bf16 + bf16 (reference :168-170)
    tc = torch.from_numpy(codes).reshape(-1, g)
    td = tc.sub(8).mul(torch.from_numpy(s).to(torch.bfloat16).reshape(-1, 1)).add(torch.from_numpy(z).to(torch.bfloat16).reshape(-1, 1))
    assert td.dtype == torch.bfloat16
    np.testing.assert_array_equal(deq_bf16, td.reshape(16, 256).float().numpy())


def test_check_linear_int4_k():
    assert qo.check_linear_int4_k(4096, 128, 8)
    assert qo.check_linear_int4_k(11008, 128, 8)
    assert qo.check_linear_int4_k(11008, 256, 8) and not qo.check_linear_int4_k(11008, 512, 8)
    assert not qo.check_linear_int4_k(4000, 128, 8)
    assert qo.check_linear_int4_k(32, 32, 2)

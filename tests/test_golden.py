"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU part: the oracle still reproduces them (guards against drift of the checker itself).
GPU part: the HIP path reproduces them through the C ABI -- bit-exact for codes, scales, zeros and packed words,
max|y - y_ref| / max|y_ref| <= 1e-2 for the matmuls -- without using the oracle's quantizers at run time."""

import os

import numpy as np
import pytest
import torch

from oracle import quant_oracle as qo

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
GROUPS = (32, 64, 128, 256)
IKTS = (2, 4, 8)
TOL = 1e-2


def _load(name):
    return np.load(os.path.join(HERE, name), allow_pickle=False)


def _bf16(bits, device=None):
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16)
    return t.to(device) if device else t


def test_fixture_files_are_small_and_complete():
    for name in ("int8_per_channel.npz", "int4_groupwise.npz"):
        path = os.path.join(HERE, name)
        assert os.path.getsize(path) < 256 * 1024
    f4 = _load("int4_groupwise.npz")
    for g in GROUPS:
        assert f4[f"codes_g{g}"].max() <= 15
        for ikt in IKTS:
            assert f"packed_g{g}_ikt{ikt}" in f4.files


def test_oracle_reproduces_int8_fixture():
    f = _load("int8_per_channel.npz")
    q, scales, _ = qo.int8_quantize_per_channel(f["w"])
    assert np.array_equal(q, f["q"]) and np.array_equal(scales, f["scales_f32"])
    assert np.array_equal(qo.bf16_bits(qo.bf16_round(scales)), f["scales_bf16_bits"])
    # rows built for the edge cases: all-zero row -> scale eps and codes 0; tiny constant row clamps the scale
    assert np.all(f["q"][0] == 0) and f["scales_f32"][0] == np.float32(np.finfo(np.float32).eps)
    assert f["q"].min() == -128 and f["q"].max() == 127


@pytest.mark.parametrize("g", GROUPS)
def test_oracle_reproduces_int4_fixture(g):
    f = _load("int4_groupwise.npz")
    w = qo.bf16_from_bits(f[f"w_bits_g{g}"])
    codes, sz = qo.int4_group_quantize(w, 4, g)
    assert np.array_equal(codes, f[f"codes_g{g}"]) and np.array_equal(qo.bf16_bits(sz), f[f"sz_bits_g{g}"])
    for ikt in IKTS:
        packed = f[f"packed_g{g}_ikt{ikt}"]
        assert np.array_equal(qo.int4_tile_pack(codes, ikt), packed)
        assert np.array_equal(qo.int4_tile_unpack(packed, ikt), codes)


# ---- GPU: the product path against the same files -------------------------------------------------

DEV = "cuda:0"


@pytest.mark.gpu
@pytest.mark.parametrize("as_bf16", [False, True])
def test_gpu_int8_quantize_and_mm_match_fixture(as_bf16):
    from easy_to_hard_amd import ops

    f = _load("int8_per_channel.npz")
    w = torch.from_numpy(f["w"])
    if as_bf16:
        # the bf16 input route must equal quantizing the widened values
        w = w.to(torch.bfloat16)
        q_ref, s_ref, _ = qo.int8_quantize_per_channel(w.float().numpy())
    else:
        q_ref, s_ref = f["q"], f["scales_f32"]
    q, scales = ops.int8_quantize_per_channel(w.to(DEV))
    assert np.array_equal(q.cpu().numpy(), q_ref) and np.array_equal(scales.cpu().numpy(), s_ref)
    if not as_bf16:
        x = _bf16(f["x_bits"], DEV)
        y = ops.int8_mm_direct(x, torch.from_numpy(f["q"]).to(DEV), _bf16(f["scales_bf16_bits"], DEV))
        assert qo.normwise_rel_err(y.float().cpu().numpy(), f["y_fp32"]) <= TOL
        # the two-rounding form of the reference differs from the kernel by at most one bf16 step
        y_rr = qo.bf16_from_bits(f["y_reference_rounding_bits"])
        assert np.max(np.abs(y.float().cpu().numpy() - y_rr)) <= np.max(np.abs(y_rr)) * 2.0 ** -6


@pytest.mark.gpu
@pytest.mark.parametrize("g", GROUPS)
def test_gpu_int4_quantize_pack_mm_match_fixture(g):
    from easy_to_hard_amd import ops

    f = _load("int4_groupwise.npz")
    w = _bf16(f[f"w_bits_g{g}"], DEV)
    codes, sz = ops.int4_group_quantize(w, g)
    assert np.array_equal(codes.cpu().numpy(), f[f"codes_g{g}"].astype(np.int32))
    assert np.array_equal(sz.cpu().view(torch.int16).numpy().view(np.uint16), f[f"sz_bits_g{g}"])
    x = _bf16(f["x_bits"], DEV)
    for ikt in IKTS:
        want = torch.from_numpy(f[f"packed_g{g}_ikt{ikt}"])
        packed = ops.int4_pack(codes, ikt)
        assert torch.equal(packed.cpu(), want)
        fused, sz2 = ops.int4_quantize_pack(w, g, ikt)
        assert torch.equal(fused.cpu(), want) and torch.equal(sz2, sz)
        assert torch.equal(ops.int4_unpack(packed).cpu(), codes.cpu())
        deq = ops.int4_dequantize(packed, sz, g)
        assert np.array_equal(deq.cpu().view(torch.int16).numpy().view(np.uint16), f[f"dequant_bits_g{g}"])
        y = ops.int4_mm_direct(x, packed, g, sz)
        assert qo.normwise_rel_err(y.float().cpu().numpy(), f[f"y_fp32_g{g}"]) <= TOL

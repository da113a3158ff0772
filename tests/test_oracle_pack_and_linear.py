"""Self-consistency of the tile-pack restatement and pins of the int4 linear oracle (CPU only).

The nibble order is the published algorithm of PyTorch 2.2's CUDA `_convert_weight_to_int4pack`; no file
in the reference pins it (parity unpinned against that kernel), so these tests establish that the
vectorised packer equals the literal scalar loop, that unpack inverts it, and a hand-computed word."""

import numpy as np
import pytest
import torch

from oracle import quant_oracle as qo
from tests.helpers import bf16_to_np, randn_bf16


@pytest.mark.parametrize("ikt", [2, 4, 8])
def test_vectorised_pack_equals_scalar_loop_and_roundtrips(ikt):
    rng = np.random.default_rng(ikt)
    for n, k in [(8, 16 * ikt), (16, 32 * ikt), (24, 256)]:
        codes = rng.integers(0, 16, size=(n, k), dtype=np.int32)
        packed = qo.int4_tile_pack(codes, ikt)
        assert packed.shape == (n // 8, k // (16 * ikt), 32, ikt // 2) and packed.dtype == np.int32
        np.testing.assert_array_equal(packed, qo.int4_tile_pack_scalar(codes, ikt))
        np.testing.assert_array_equal(qo.int4_tile_unpack(packed, ikt), codes)


def test_hand_computed_word():
    # codes[n, k] = k % 16 on row 3 only; lane t = 4*3 + 2 (row 3, j = 2), ikt = 2, single k block:
    # v = codes at k = 4,5,12,13,20,21,28,29 -> 4,5,12,13,4,5,12,13
    codes = np.zeros((8, 32), dtype=np.int32)
    codes[3] = np.arange(32) % 16
    packed = qo.int4_tile_pack(codes, 2).view(np.uint32)
    v = [4, 5, 12, 13, 4, 5, 12, 13]
    expect = v[0] | v[2] << 4 | v[4] << 8 | v[6] << 12 | v[1] << 16 | v[3] << 20 | v[5] << 24 | v[7] << 28
    assert packed[0, 0, 14, 0] == expect
    # (word >> 4i) & 0x000F000F yields consecutive-k pairs: the property the matmul kernels rely on
    for i, (lo, hi) in enumerate([(4, 5), (12, 13), (4, 5), (12, 13)]):
        pair = (int(packed[0, 0, 14, 0]) >> (4 * i)) & 0x000F000F
        assert pair & 0xFFFF == lo and pair >> 16 == hi
    assert np.count_nonzero(packed[0, 0, :12]) == 0 and np.count_nonzero(packed[0, 0, 16:]) == 0


def test_every_position_is_stored_exactly_once():
    # a one-hot code matrix lands in exactly one nibble
    ikt, n, k = 8, 8, 128
    for (r, c) in [(0, 0), (7, 127), (3, 77), (5, 16)]:
        codes = np.zeros((n, k), dtype=np.int32)
        codes[r, c] = 15
        packed = qo.int4_tile_pack(codes, ikt).view(np.uint32)
        nz = packed[packed != 0]
        assert len(nz) == 1 and bin(int(nz[0])).count("1") == 4


@pytest.mark.parametrize("g", [32, 128])
def test_int4_linear_oracle_against_brute_force_and_library(g):
    n, k, m, ikt = 16, 256, 3, 8
    w = bf16_to_np(randn_bf16((n, k), std=0.02, seed=21))
    codes, sz = qo.int4_group_quantize(w, 4, g)
    x = randn_bf16((m, k), seed=22)
    xf = bf16_to_np(x)
    y = qo.int4_linear_fp32(xf, codes, sz, g)
    ref = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            acc = 0.0
            for kk in range(k):
                acc += float(xf[i, kk]) * ((int(codes[j, kk]) - 8) * float(sz[kk // g, j, 0]) + float(sz[kk // g, j, 1]))
            ref[i, j] = acc
    np.testing.assert_allclose(y, ref, rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(qo.int4_linear_packed_fp32(xf, qo.int4_tile_pack(codes, ikt), sz, g, ikt), y)
    # independent library kernel with the same math (its own packed layout): bf16 output -> loose tolerance
    packed_cpu = torch.ops.aten._convert_weight_to_int4pack_for_cpu(torch.from_numpy(codes), ikt)
    y_lib = torch.ops.aten._weight_int4pack_mm_for_cpu(x, packed_cpu, g, torch.from_numpy(sz).to(torch.bfloat16))
    assert qo.normwise_rel_err(y_lib.float().numpy(), y) < 1e-2
    # dequantized weights approximate the original ones (quantization error only)
    assert np.abs(qo.int4_dequantize_fp32(codes, sz, g) - w).max() < 0.02


def test_metrics():
    a = np.array([1.0, -2.0, 4.0])
    assert qo.normwise_rel_err(a, a) == 0.0
    assert abs(qo.normwise_rel_err(a + np.array([0, 0.04, 0]), a) - 0.01) < 1e-12
    assert qo.elementwise_violations(a, a) == 0.0

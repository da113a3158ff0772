"""Writes the committed fixtures of this directory.

The reference ships no golden vectors, known-answer tests or fixtures for its quantization path, so these are
regression vectors: seeded inputs with edge rows, and the outputs of the CPU oracle (oracle/quant_oracle.py),
whose functions are pinned separately (library kernels, closed forms, brute force) in tests/test_oracle_*.py.
They fix the oracle's behaviour in time and give the GPU tests data that does not depend on the oracle module
at run time.  Nothing here reads or runs the reference.

    python tests/golden/make_fixtures.py        # rewrites tests/golden/*.npz

bfloat16 arrays are stored as uint16 bit patterns; everything loads with numpy.load(allow_pickle=False).
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import quant_oracle as qo  # noqa: E402
from tests.helpers import bf16_to_np, randn_bf16, weight_with_edge_rows  # noqa: E402

N, K, M = 16, 512, 5
GROUPS = (32, 64, 128, 256)
IKTS = (2, 4, 8)


def int8_fixture():
    w = bf16_to_np(weight_with_edge_rows(N, K, 128, std=0.02, seed=11)).astype(np.float32)
    # float32-only rows: values that are not bf16-exact, a .5-tie ladder, a denormal-scale row
    rng = np.random.default_rng(5)
    w[8] = rng.standard_normal(K).astype(np.float32) * 0.02
    w[9] = (np.arange(K, dtype=np.float32) - K / 2 + 0.5) * (127.5 / (K / 2 - 0.5)) / 127.5
    w[10] = 1e-9
    q, scales, _ = qo.int8_quantize_per_channel(w)
    x = bf16_to_np(randn_bf16((M, K), seed=12))
    s_bf16 = qo.bf16_round(scales)
    return dict(w=w, q=q.astype(np.int8), scales_f32=scales.astype(np.float32), scales_bf16_bits=qo.bf16_bits(s_bf16),
                x_bits=qo.bf16_bits(x), y_fp32=qo.int8_linear_fp32(x, q, s_bf16).astype(np.float32),
                y_reference_rounding_bits=qo.bf16_bits(qo.int8_linear_reference_rounding(x, q, s_bf16)))


def int4_fixture():
    out = {}
    x = bf16_to_np(randn_bf16((M, K), seed=22))
    out["x_bits"] = qo.bf16_bits(x)
    for g in GROUPS:
        w = bf16_to_np(weight_with_edge_rows(N, K, g, std=0.02, seed=20 + g))
        codes, sz = qo.int4_group_quantize(w, 4, g)
        out[f"w_bits_g{g}"] = qo.bf16_bits(w)
        out[f"codes_g{g}"] = codes.astype(np.uint8)
        out[f"sz_bits_g{g}"] = qo.bf16_bits(sz)
        out[f"dequant_bits_g{g}"] = qo.bf16_bits(qo.int4_dequantize_from_qparams(codes, *qo.unpack_scales_and_zeros(sz), 4, g))
        out[f"y_fp32_g{g}"] = qo.int4_linear_fp32(x, codes, sz, g).astype(np.float32)
        for ikt in IKTS:
            out[f"packed_g{g}_ikt{ikt}"] = qo.int4_tile_pack(codes, ikt).astype(np.int32)
    return out


def main():
    np.savez_compressed(os.path.join(HERE, "int8_per_channel.npz"), **int8_fixture())
    np.savez_compressed(os.path.join(HERE, "int4_groupwise.npz"), **int4_fixture())
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()

"""CPU restatement of the weight-only quantized linear path of gpt-accelera's models/quantize.py.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this module: it is the checker
for the HIP kernels (tests/, the smoke check and the CPU-baseline leg of the benchmark), never the
thing that is measured or shipped.

Everything is plain numpy on float32 / integer arrays.  bfloat16 tensors are carried as float32
arrays whose values are exactly representable in bfloat16; `bf16_round` inserts the round-to-nearest-
even step that a torch op on a bfloat16 tensor performs after computing in float32.

Functions and the reference lines they restate (paths relative to the reference tree):

  int8_quantize_per_channel        models/quantize.py:39-71    dynamically_quantize_per_channel
  int8_linear_fp32                 models/quantize.py:428-429  WeightOnlyInt8Linear.forward, exact fp32 form
  int8_linear_reference_rounding   models/quantize.py:428-429  same, with the bf16 roundings of F.linear and `*`
  int4_group_qparams               models/quantize.py:74-92    get_group_qparams
  int4_quantize_from_qparams       models/quantize.py:118-144  group_quantize_tensor_from_qparams
  pack_scales_and_zeros            models/quantize.py:95-109   pack_scales_and_zeros
  int4_group_quantize              models/quantize.py:147-151  group_quantize_tensor
  int4_dequantize_from_qparams     models/quantize.py:154-171  group_dequantize_tensor_from_qparams
  int4_dequantize_fp32             models/quantize.py:168-170  same arithmetic carried out in float32
  int4_tile_pack / int4_tile_unpack  call sites models/quantize.py:439-441, :585-587
                                   (torch.ops.aten._convert_weight_to_int4pack, PyTorch 2.2.0 CUDA
                                   build, aten/src/ATen/native/cuda/int4mm.cu -- NOT in the reference tree)
  int4_linear_fp32                 call site models/quantize.py:445-453 (aten._weight_int4pack_mm),
                                   dequantize-then-matmul in float32
  check_linear_int4_k              models/quantize.py:456-457

Pinning status (what independent evidence each restatement is checked against in tests/):

  int8_quantize_per_channel   pinned: torch.ao.quantization PerChannelMinMaxObserver (library routine
                              with the same 127.5 divisor and eps clamp), the same op chain executed by
                              torch CPU kernels, brute-force scalar loop, reconstruction-error invariants.
  int4_group_qparams / int4_quantize_from_qparams
                              pinned: the same op chain executed by torch CPU bfloat16 kernels (an
                              independent implementation of every rounding), scalar brute force with
                              Python floats, invariants (group max -> 15, min -> 0, reconstruction error
                              <= scale/2 + rounding), constant-group closed form.
  pack_scales_and_zeros       pinned: pure index shuffle checked element by element.
  int4_dequantize_*           pinned: scalar brute force; inverse relation with the quantizer.
  int8_linear_* / int4_linear_fp32
                              pinned: float64 brute force on tiny cases and the library kernels
                              torch.ops.aten._weight_int8pack_mm and
                              aten._convert_weight_to_int4pack_for_cpu/_weight_int4pack_mm_for_cpu.
  int4_tile_pack              word format pinned on the GPU against PyTorch-ROCm's own
                              aten._convert_weight_to_int4pack (an independent library with the same bit
                              formula inside a word and another lane map): every checkpoint word is a fixed
                              gather of nibbles from two of that packer's words and must equal this function's
                              output bit for bit (tests/test_gpu_configs_at_size.py).  That pins the nibble
                              order inside a word, the pairing of two 16-wide k tiles per word and the outer
                              [N tile][K super-tile][lane][pair] order.
                              PARITY UNPINNED: the lane map of the PyTorch 2.2.0 CUDA kernel itself (lane t holds
                              row 8 * nTile + t / 4 and k = 2j, 2j+1, 2j+8, 2j+9 with j = t % 4).  That source
                              (`matrix_to_m16n8k16_Bint4_layout`) is not in the reference tree or this image and
                              the reference holds no packed checkpoint; the published algorithm is restated
                              and the CPU tests pin self-consistency only (brute-force scalar packer,
                              unpack(pack(q)) == q, end-to-end matmul agreement).
"""

import numpy as np

# --------------------------------------------------------------------------------------------
# bfloat16 helpers
# --------------------------------------------------------------------------------------------


def bf16_bits(x):
    """float32 array -> uint16 bfloat16 bit patterns, round-to-nearest-even (NaN not supported)."""
    u = np.array(x, dtype=np.float32, order="C", copy=True).view(np.uint32)
    rounding = ((u >> 16) & 1) + np.uint32(0x7FFF)
    return ((u + rounding) >> 16).astype(np.uint16)


def bf16_from_bits(b):
    """uint16 bfloat16 bit patterns -> float32 array."""
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def bf16_round(x):
    """Round a float32 array to the nearest bfloat16 value (ties to even), returned as float32."""
    return bf16_from_bits(bf16_bits(x))


def is_bf16_exact(x):
    x = np.asarray(x, dtype=np.float32)
    return bool(np.all(bf16_round(x) == x))


# --------------------------------------------------------------------------------------------
# int8 per-output-channel symmetric quantization
# --------------------------------------------------------------------------------------------

FP32_EPS = np.float32(np.finfo(np.float32).eps)  # models/quantize.py:46


def int8_quantize_per_channel(x, quant_min=-128, quant_max=127):
    """models/quantize.py:39-71.  x float32 [N, K] -> (q int8 [N, K], scales float32 [N], zero_points int64 [N]).

    All arithmetic is IEEE float32: the divisor is float(quant_max - quant_min) / 2 (= 127.5 for int8,
    :59), the scale is clamped from below at float32 eps (:61), the quotient x / scale is a true
    division (:66), rounding is half-to-even (:67) and the clamp comes last (:69).
    """
    x = np.asarray(x, dtype=np.float32)
    assert x.ndim == 2
    min_val = x.min(axis=1)  # :49
    max_val = x.max(axis=1)
    min_val_neg = np.minimum(min_val, np.float32(0))  # :53
    max_val_pos = np.maximum(max_val, np.float32(0))  # :54
    max_val_pos = np.maximum(-min_val_neg, max_val_pos)  # :58
    half_range = np.float32(float(quant_max - quant_min) / 2)
    scales = (max_val_pos / half_range).astype(np.float32)  # :59
    scales = np.maximum(scales, FP32_EPS)  # :61
    zero_points = np.zeros(x.shape[0], dtype=np.int64)  # :62
    x_div = (x / scales[:, None]).astype(np.float32)  # :66
    x_round = np.rint(x_div)  # :67  (half to even)
    quant = np.clip(x_round, quant_min, quant_max).astype(np.int8)  # :68-69
    return quant, scales, zero_points


def int8_linear_fp32(x, q, scales):
    """Exact form of models/quantize.py:428-429: (x @ q^T) * scales, all in float32 (float64 accumulate).

    x: [M, K] values (bf16-exact float32), q: int8 [N, K], scales: [N] (the stored bf16 scales as float32).
    """
    acc = np.asarray(x, dtype=np.float64) @ np.asarray(q, dtype=np.float64).T
    return (acc * np.asarray(scales, dtype=np.float64)[None, :]).astype(np.float32)


def int8_linear_reference_rounding(x, q, scales):
    """models/quantize.py:428-429 with the two bfloat16 roundings the reference performs:
    F.linear returns bf16 (float32 accumulate rounded once), then `* scales` rounds again."""
    acc = (np.asarray(x, dtype=np.float64) @ np.asarray(q, dtype=np.float64).T).astype(np.float32)
    t = bf16_round(acc)
    return bf16_round(t * np.asarray(scales, dtype=np.float32)[None, :])


# --------------------------------------------------------------------------------------------
# int4 group-wise asymmetric quantization (bfloat16 arithmetic, one rounding per op)
# --------------------------------------------------------------------------------------------


def int4_group_qparams(w, n_bit=4, groupsize=128):
    """models/quantize.py:74-92.  w: float32 [N, K] holding bf16-exact values.

    Returns (scales, zeros), float32 [N, K/g] holding bf16-exact values.  Each line below is one torch
    op on a bfloat16 tensor: computed in float32, then rounded to bfloat16.
    """
    w = np.asarray(w, dtype=np.float32)
    if groupsize > w.shape[-1]:  # :76-77
        groupsize = w.shape[-1]
    assert groupsize > 1  # :78
    assert w.shape[-1] % groupsize == 0  # :79
    assert w.ndim == 2  # :80
    to_quant = w.reshape(-1, groupsize)  # :82
    assert not np.isnan(to_quant).any()  # :83
    max_val = to_quant.max(axis=1, keepdims=True)  # :85
    min_val = to_quant.min(axis=1, keepdims=True)  # :86
    max_int = 2**n_bit - 1  # :87
    rng = bf16_round(max_val - min_val)  # :88  (a - b)
    rng = np.maximum(rng, bf16_round(np.float32(1e-6)))  # :88  .clamp(min=1e-6) on a bf16 tensor
    scales = bf16_round(rng / np.float32(max_int))  # :88  / max_int
    half = bf16_round(scales * np.float32(2 ** (n_bit - 1)))  # :89  scales * 8
    zeros = bf16_round(min_val + half)  # :89
    return scales.reshape(w.shape[0], -1), zeros.reshape(w.shape[0], -1)  # :90-92


def int4_quantize_from_qparams(w, scales, zeros, n_bit=4, groupsize=128):
    """models/quantize.py:118-144.  Returns int32 codes [N, K] in [0, 2^n_bit - 1]."""
    w = np.asarray(w, dtype=np.float32)
    assert groupsize > 1  # :119
    if groupsize > w.shape[-1] and scales.shape[-1] == 1:  # :121-122
        groupsize = w.shape[-1]
    assert w.shape[-1] % groupsize == 0  # :124
    assert w.ndim == 2  # :125
    to_quant = w.reshape(-1, groupsize)  # :127
    assert not np.isnan(to_quant).any()  # :128
    scales = np.asarray(scales, dtype=np.float32).reshape(-1, 1)  # :130
    zeros = np.asarray(zeros, dtype=np.float32).reshape(-1, 1)  # :131
    min_val = bf16_round(zeros - bf16_round(scales * np.float32(2 ** (n_bit - 1))))  # :132
    max_int = 2**n_bit - 1  # :133
    t = bf16_round(to_quant - min_val)  # :136  .sub
    t = bf16_round(t / scales)  # :137  .div
    t = np.rint(t)  # :138  .round (half to even)
    t = np.clip(t, 0, max_int)  # :139
    return t.astype(np.int32).reshape(w.shape)  # :140-141


def pack_scales_and_zeros(scales, zeros):
    """models/quantize.py:95-109.  Two [N, K/g] arrays -> [K/g, N, 2] ([..., 0] scale, [..., 1] zero)."""
    assert scales.shape == zeros.shape  # :96
    return np.ascontiguousarray(np.stack([scales, zeros], axis=2).transpose(1, 0, 2))


def unpack_scales_and_zeros(scales_and_zeros):
    """Inverse of pack_scales_and_zeros (models/quantize.py:112-115 without its float32 assert)."""
    assert scales_and_zeros.ndim == 3 and scales_and_zeros.shape[2] == 2
    t = scales_and_zeros.transpose(1, 0, 2)
    return np.ascontiguousarray(t[..., 0]), np.ascontiguousarray(t[..., 1])


def int4_group_quantize(w, n_bit=4, groupsize=128):
    """models/quantize.py:147-151.  -> (codes int32 [N, K], scales_and_zeros float32(bf16-exact) [K/g, N, 2])."""
    scales, zeros = int4_group_qparams(w, n_bit, groupsize)
    codes = int4_quantize_from_qparams(w, scales, zeros, n_bit, groupsize)
    return codes, pack_scales_and_zeros(scales, zeros)


def int4_dequantize_from_qparams(codes, scales, zeros, n_bit=4, groupsize=128):
    """models/quantize.py:154-171 evaluated on bfloat16 qparams: the int32 - 8 is exact, `.mul(scales)`
    promotes to bfloat16 and rounds, `.add(zeros)` rounds again."""
    codes = np.asarray(codes)
    assert groupsize > 1  # :157
    if groupsize > codes.shape[-1] and scales.shape[-1] == 1:  # :159-160
        groupsize = codes.shape[-1]
    assert codes.shape[-1] % groupsize == 0  # :161
    assert codes.ndim == 2  # :162
    grouped = codes.reshape(-1, groupsize).astype(np.float32)  # :164
    s = np.asarray(scales, dtype=np.float32).reshape(-1, 1)  # :165
    z = np.asarray(zeros, dtype=np.float32).reshape(-1, 1)  # :166
    t = bf16_round((grouped - np.float32(2 ** (n_bit - 1))) * s)  # :169 .sub(8).mul(scales)
    return bf16_round(t + z).reshape(codes.shape)  # :169 .add(zeros)


def int4_dequantize_fp32(codes, scales_and_zeros, groupsize):
    """(q - 8) * scale + zero (models/quantize.py:168-170) in float64, returned as float32 [N, K].

    This is the weight matrix of the parity oracle: dequantize-then-matmul in float32."""
    codes = np.asarray(codes)
    n, k = codes.shape
    sz = np.asarray(scales_and_zeros, dtype=np.float64)
    assert sz.shape == (k // groupsize, n, 2)
    s = np.repeat(sz[:, :, 0].T, groupsize, axis=1)
    z = np.repeat(sz[:, :, 1].T, groupsize, axis=1)
    return ((codes.astype(np.float64) - 8.0) * s + z).astype(np.float32)


def check_linear_int4_k(k, groupsize=1, inner_k_tiles=1):
    """models/quantize.py:456-457."""
    return k % groupsize == 0 and k % (inner_k_tiles * 16) == 0


# --------------------------------------------------------------------------------------------
# tile-packed int4 weight layout (torch.ops.aten._convert_weight_to_int4pack, PyTorch 2.2.0 CUDA)
# --------------------------------------------------------------------------------------------

# Nibble i (bits 4i .. 4i+3) of a packed word holds v[_NIBBLE_SRC[i]], where v[0..7] are the eight
# codes a lane gathers: from the first 16-wide k-tile at k offsets {2j, 2j+1, 2j+8, 2j+9} and from the
# second k-tile at the same offsets (j = lane & 3).
_NIBBLE_SRC = (0, 2, 4, 6, 1, 3, 5, 7)


def _k_offsets(j):
    return (2 * j, 2 * j + 1, 2 * j + 8, 2 * j + 9, 16 + 2 * j, 16 + 2 * j + 1, 16 + 2 * j + 8, 16 + 2 * j + 9)


def int4_tile_pack(codes, inner_k_tiles):
    """int32 codes [N, K] (0..15) -> int32 [N/8, K/(16*ikt), 32, ikt/2].

    Word [nTile][kOuter][t][p] belongs to row n = 8*nTile + t//4; with j = t % 4 and
    k0 = (kOuter*ikt + 2p)*16 it packs codes[n, k0 + _k_offsets(j)[s]] for s = _NIBBLE_SRC[i] into nibble i.
    """
    codes = np.asarray(codes)
    n, k = codes.shape
    ikt = inner_k_tiles
    assert ikt in (2, 4, 8)
    assert n % 8 == 0 and k % (16 * ikt) == 0
    assert codes.min() >= 0 and codes.max() <= 15
    q = codes.astype(np.uint32)
    out = np.zeros((n // 8, k // (16 * ikt), 32, ikt // 2), dtype=np.uint32)
    rows = np.arange(n).reshape(n // 8, 8)  # [nTile][t//4]
    for k_outer in range(k // (16 * ikt)):
        for p in range(ikt // 2):
            k0 = (k_outer * ikt + 2 * p) * 16
            for j in range(4):
                offs = _k_offsets(j)
                word = np.zeros((n // 8, 8), dtype=np.uint32)
                for i, s in enumerate(_NIBBLE_SRC):
                    word |= q[rows, k0 + offs[s]] << np.uint32(4 * i)
                out[:, k_outer, j::4, p] = word  # t = 4*(t//4) + j
    return out.view(np.int32)


def int4_tile_unpack(packed, inner_k_tiles):
    """Inverse of int4_tile_pack: int32 [N/8, K/(16*ikt), 32, ikt/2] -> int32 codes [N, K]."""
    packed = np.asarray(packed).view(np.uint32)
    ikt = inner_k_tiles
    n_tiles, k_outers, lanes, pairs = packed.shape
    assert lanes == 32 and pairs == ikt // 2
    n, k = n_tiles * 8, k_outers * 16 * ikt
    codes = np.zeros((n, k), dtype=np.int32)
    rows = np.arange(n).reshape(n_tiles, 8)
    for k_outer in range(k_outers):
        for p in range(pairs):
            k0 = (k_outer * ikt + 2 * p) * 16
            for j in range(4):
                offs = _k_offsets(j)
                word = packed[:, k_outer, j::4, p]
                for i, s in enumerate(_NIBBLE_SRC):
                    codes[rows, k0 + offs[s]] = (word >> np.uint32(4 * i)) & np.uint32(15)
    return codes


def int4_tile_pack_scalar(codes, inner_k_tiles):
    """Literal scalar restatement of the published packing loop, for brute-force checks on tiny inputs."""
    codes = np.asarray(codes)
    n, k = codes.shape
    ikt = inner_k_tiles
    out = np.zeros((n // 8, k // (16 * ikt), 32, ikt // 2), dtype=np.uint32)
    for n_tile in range(n // 8):
        for k_outer in range(k // (16 * ikt)):
            for t in range(32):
                for inner in range(0, ikt, 2):
                    row = n_tile * 8 + t // 4
                    k_base0 = (k_outer * ikt + inner) * 16
                    k_base1 = k_base0 + 16
                    ks = [0] * 8
                    ks[0] = k_base0 + (t % 4) * 2
                    ks[1] = ks[0] + 1
                    ks[2] = ks[0] + 8
                    ks[3] = ks[0] + 8 + 1
                    ks[4] = k_base1 + (t % 4) * 2
                    ks[5] = ks[4] + 1
                    ks[6] = ks[4] + 8
                    ks[7] = ks[4] + 8 + 1
                    v = [int(codes[row, kk]) for kk in ks]
                    word = (
                        (v[7] << 28) | (v[5] << 24) | (v[3] << 20) | (v[1] << 16)
                        | (v[6] << 12) | (v[4] << 8) | (v[2] << 4) | v[0]
                    )
                    out[n_tile, k_outer, t, inner // 2] = word
    return out.view(np.int32)


# --------------------------------------------------------------------------------------------
# linear forward oracles
# --------------------------------------------------------------------------------------------


def int4_linear_fp32(x, codes, scales_and_zeros, groupsize):
    """Dequantize-then-matmul parity oracle for aten._weight_int4pack_mm (models/quantize.py:445-453):
    y[m, n] = sum_k x[m, k] * ((q[n, k] - 8) * scale[g, n] + zero[g, n]), float64 accumulate -> float32."""
    w = int4_dequantize_fp32(codes, scales_and_zeros, groupsize).astype(np.float64)
    return (np.asarray(x, dtype=np.float64) @ w.T).astype(np.float32)


def int4_linear_packed_fp32(x, packed, scales_and_zeros, groupsize, inner_k_tiles):
    """Same, starting from the tile-packed weight (what WeightOnlyInt4Linear.forward receives, :658-666)."""
    return int4_linear_fp32(x, int4_tile_unpack(packed, inner_k_tiles), scales_and_zeros, groupsize)


# --------------------------------------------------------------------------------------------
# parity metrics
# --------------------------------------------------------------------------------------------


def normwise_rel_err(y, y_ref):
    """max|y - y_ref| / max|y_ref| -- the pass/fail gate (<= 1e-2 for bf16 outputs)."""
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    denom = np.abs(y_ref).max()
    if denom == 0:
        return float(np.abs(y).max())
    return float(np.abs(y - y_ref).max() / denom)


def elementwise_violations(y, y_ref, rtol=1e-2):
    """Fraction of elements with |y - y_ref| > rtol*|y_ref| + rtol*rms(y_ref)."""
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    atol = rtol * np.sqrt(np.mean(y_ref**2))
    return float(np.mean(np.abs(y - y_ref) > rtol * np.abs(y_ref) + atol))

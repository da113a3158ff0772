"""MI355X-native weight-only quantized linear path (int8 per-channel, int4 group-wise) of gpt-accelera.

Public surface mirrors the reference's models/quantize.py; see quantize.py.  The HIP kernels live in
libe2h_quant.so (C ABI: include/e2h_quant.h) and are loaded on first use.
"""

from . import _lib, ops  # noqa: F401
from . import _traced as _traced

_traced.install()  # e2h:: custom ops behind the public names of ops.py while a torch.compile trace is taken
from .quantize import (  # noqa: F401
    QuantHandler,
    WeightOnlyInt4Linear,
    WeightOnlyInt4QuantHandler,
    WeightOnlyInt8Linear,
    WeightOnlyInt8QuantHandler,
    _check_linear_int4_k,
    dynamically_quantize_per_channel,
    find_multiple,
    get_group_qparams,
    group_dequantize_tensor,
    group_dequantize_tensor_from_qparams,
    group_quantize_tensor,
    group_quantize_tensor_from_qparams,
    linear_forward_int4,
    pack_scales_and_zeros,
    prepare_int4_weight_and_scales_and_zeros,
    quantize,
    replace_linear_int4,
    replace_linear_weight_only_int8_per_channel,
    replace_linear_weight_only_int8_per_channel_on_the_fly,
    unpack_scales_and_zeros,
)

__all__ = [n for n in dir() if not n.startswith("__")]

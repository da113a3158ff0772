"""ctypes binding of libe2h_quant.so (C ABI: include/e2h_quant.h).

The library is loaded from the package directory.  If it has not been built, loading raises: there is
no fallback implementation behind these entry points.
"""

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

from ._build import LIB_PATH, build_library

_P = c_void_p
_SIGNATURES = {
    # name: (restype, argtypes)
    "e2h_abi_version": (c_int, []),
    "e2h_status_string": (c_char_p, [c_int]),
    "e2h_set_option": (c_int, [c_char_p, c_int]),
    "e2h_int8_quantize_per_channel": (c_int, [_P, c_int, _P, _P, _P, c_int64, c_int64, _P]),
    "e2h_int8_mm": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, _P, c_int64, _P]),
    "e2h_int4_group_qparams": (c_int, [_P, _P, _P, c_int64, c_int64, c_int, _P]),
    "e2h_int4_quantize_from_qparams": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int, _P]),
    "e2h_int4_group_quantize": (c_int, [_P, _P, _P, c_int64, c_int64, c_int, _P]),
    "e2h_int4_pack": (c_int, [_P, _P, c_int64, c_int64, c_int, _P]),
    "e2h_int4_unpack": (c_int, [_P, _P, c_int64, c_int64, c_int, _P]),
    "e2h_int4_quantize_pack": (c_int, [_P, _P, _P, c_int64, c_int64, c_int, c_int, _P]),
    "e2h_int4_dequantize": (c_int, [_P, _P, _P, c_int64, c_int64, c_int, c_int, _P]),
    "e2h_int4_dequantize_codes": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int, _P]),
    "e2h_int4_mm": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int, c_int, _P, c_int64, _P]),
    "e2h_workspace_bytes": (c_int64, []),
    "e2h_int4_mm_static_scratch": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int, c_int, _P]),
    "e2h_int4_mm_static_scratch_bytes": (c_int64, []),
    "e2h_decode_attention": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_float, _P]),
    "e2h_rmsnorm": (c_int, [_P, _P, _P, c_int64, c_int64, c_float, _P]),
    "e2h_add_rmsnorm": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int64, c_float, _P]),
    "e2h_int4_mm_partial_slices": (c_int, [c_int64, c_int64, c_int64, c_int, c_int]),
    "e2h_int4_mm_partials": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int, c_int, c_int, _P]),
    "e2h_int8_mm_partial_slices": (c_int, [c_int64, c_int64, c_int64]),
    "e2h_int8_mm_partials": (c_int, [_P, _P, _P, c_int64, c_int64, c_int64, c_int, _P]),
    "e2h_add_rmsnorm_partials": (c_int, [_P, _P, c_int, _P, _P, _P, _P, c_int64, c_int64, c_float, _P]),
    "e2h_rope_kv_write": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, _P]),
    "e2h_rope_kv_write_seq": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, _P]),
    "e2h_silu_mul": (c_int, [_P, _P, _P, c_int64, _P]),
    "e2h_int4_mm_rope_kv": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, _P]),
    "e2h_sample_top_k": (c_int, [_P, c_int64, _P, _P, _P, c_int64, c_int64, c_float, c_int, _P]),
    "e2h_argmax_rows": (c_int, [_P, c_int64, _P, c_int64, c_int64, _P]),
    "e2h_int8_mm_silu_gate": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, _P]),
    "e2h_int8_mm_rope_kv": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, _P]),
    "e2h_int4_mm_silu_gate": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int, c_int, _P]),
    "e2h_int4_staged_bytes": (c_int64, [c_int64, c_int64]),
    "e2h_int4_stage_x": (c_int, [_P, _P, c_int64, c_int64, _P]),
    "e2h_int4_mm_staged_supported": (c_int, [c_int64, c_int64, c_int64, c_int, c_int]),
    "e2h_int4_mm_staged": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int, _P]),
    "e2h_int4_mm_staged_argmax_scratch_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int]),
    "e2h_int4_mm_staged_argmax": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int, _P]),
    "e2h_int4_mm_staged_partial_slices": (c_int, [c_int64, c_int64, c_int64, c_int]),
    "e2h_int4_mm_staged_partials": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int, c_int, _P]),
    "e2h_int4_mm_staged_silu_gate": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int, _P]),
    "e2h_int4_mm_staged_rope_kv": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, _P]),
    "e2h_add_rmsnorm_staged": (c_int, [_P, _P, _P, c_int, _P, _P, _P, _P, _P, c_int64, c_int64, c_float, _P]),
    "e2h_stream_read_probe": (c_int, [_P, c_int64, _P, c_int64, _P, _P]),
    "e2h_decode_attention_staged": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_float, _P]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


class E2HLibraryError(RuntimeError):
    pass


def load(build_if_missing=False):
    """Return the loaded library.  `build_if_missing` compiles it first when the .so is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        if not build_if_missing:
            raise E2HLibraryError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no fallback path for the quantized-linear kernels)"
            )
        build_library()
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.e2h_abi_version() != 1:
        raise E2HLibraryError(f"{LIB_PATH}: ABI version {lib.e2h_abi_version()} != 1; rebuild the library")
    _lib = lib
    return lib


def status_string(code):
    return load().e2h_status_string(code).decode()


def check(code, what):
    if code != 0:
        raise RuntimeError(f"{what}: {status_string(code)} (status {code})")


def set_option(name, value):
    check(load().e2h_set_option(name.encode(), int(value)), f"e2h_set_option({name})")

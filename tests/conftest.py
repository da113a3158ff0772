import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch

        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# every experiment option of the library (e2h_set_option) and every fusion switch of the model module: a test that
# changes one and fails half way must not leave it set for the tests after it
_LIBRARY_OPTIONS = (
    "int4_rows_per_wave", "int8_rows_per_wave", "int4_k_slices", "int4_k_groups", "int4_col_waves", "int8_k_groups",
    "int8_force_generic", "int8_k_slices", "int4_no_xsum", "int4_no_gemm32", "int4_gemm32_min_rows", "row_tiles",
    "attention_waves", "int8_gemm_waves", "int8_gemm_wave_cols", "int4_gemm_tile", "int8_gemm_tile", "attention_no_mfma", "staged_tiles", "staged_slices", "staged_no_rows64",
)
_MODEL_SWITCHES = ("FUSED_DECODE", "FUSE_GATE", "FUSE_ROPE_PROJECTION", "DEFER_SPLIT_K", "STAGED_DECODE", "STAGED_HEAD", "FUSE_HEAD_ARGMAX")


@pytest.fixture(autouse=True)
def _restore_library_options_and_model_switches():
    yield
    try:
        from easy_to_hard_amd import _lib
        from easy_to_hard_amd import model as model_mod
    except Exception:
        return
    for name in _MODEL_SWITCHES:
        setattr(model_mod, name, True)
    if _lib.LIB_PATH.exists():
        for name in _LIBRARY_OPTIONS:
            _lib.set_option(name, 0)

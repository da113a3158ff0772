"""The entry point that allocates nothing (e2h_int4_mm_static_scratch: split-K scratch in a fixed buffer inside the
library) against e2h_int4_mm with a caller-owned workspace, through the C ABI: identical bits on two calls in a row, the
second with a smaller input, and a clear error beyond its limits."""

import ctypes

import pytest
import torch

import easy_to_hard_amd as e2h
from easy_to_hard_amd import _lib, ops
from tests.helpers import randn_bf16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(lib, x, packed, sz, g):
    m, k = x.shape
    n = packed.shape[0] * 8
    ws = ops._workspace(x.device)
    y_ws = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    y_static = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=x.device)
    rc = lib.e2h_int4_mm(ops._ptr(x), ops._ptr(packed), ops._ptr(sz), ops._ptr(y_ws), m, n, k, g, 8, ops._ptr(ws), ws.numel(), ops._stream(x))
    _lib.check(rc, "e2h_int4_mm")
    rc = lib.e2h_int4_mm_static_scratch(ops._ptr(x), ops._ptr(packed), ops._ptr(sz), ops._ptr(y_static), m, n, k, g, 8, ops._stream(x))
    _lib.check(rc, "e2h_int4_mm_static_scratch")
    torch.cuda.synchronize()
    return y_ws, y_static


def test_static_scratch_entry_point_equals_the_workspace_one_on_two_calls_in_a_row():
    lib = _lib.load()
    assert lib.e2h_int4_mm_static_scratch_bytes() == 64 * 1024 + (8 << 20)
    g = 128
    # 4096 x 4096 at 32 rows splits K four ways over workgroups: tickets and partial tiles are in use
    w = randn_bf16((4096, 4096), std=0.02, seed=31).to(DEV)
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(w, g, 8)
    x = randn_bf16((32, 4096), seed=32).to(DEV)
    y_ws, y_static = _both(lib, x, packed, sz, g)
    assert torch.equal(y_ws, y_static)
    # second call, smaller in every dimension, on the scratch the first call left behind
    w2 = randn_bf16((1024, 2048), std=0.02, seed=33).to(DEV)
    packed2, sz2 = e2h.prepare_int4_weight_and_scales_and_zeros(w2, g, 8)
    x2 = randn_bf16((5, 2048), seed=34).to(DEV)
    y_ws2, y_static2 = _both(lib, x2, packed2, sz2, g)
    assert torch.equal(y_ws2, y_static2)
    # and the first shape once more
    y_ws3, y_static3 = _both(lib, x, packed, sz, g)
    assert torch.equal(y_static3, y_static) and torch.equal(y_ws3, y_ws)


def test_static_scratch_entry_point_rejects_what_exceeds_its_buffer():
    lib = _lib.load()
    g = 128
    w = randn_bf16((64, 256), std=0.02, seed=35).to(DEV)
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(w, g, 8)
    x = randn_bf16((65, 256), seed=36).to(DEV)
    y = torch.empty((65, 64), dtype=torch.bfloat16, device=DEV)
    rc = lib.e2h_int4_mm_static_scratch(ops._ptr(x), ops._ptr(packed), ops._ptr(sz), ops._ptr(y), 65, 64, 256, g, 8, ops._stream(x))
    assert rc == -9 and "scratch" in _lib.status_string(rc)
    rc = lib.e2h_int4_mm_static_scratch(None, ops._ptr(packed), ops._ptr(sz), ops._ptr(y), 4, 64, 256, g, 8, ops._stream(x))
    assert rc == -1


def test_static_scratch_entry_point_leaves_device_memory_as_it_found_it_and_replays_from_a_graph():
    """What the entry point is for: a warmed call changes neither the free device memory nor needs anything a HIP graph
    capture forbids; replays of the captured call, with eager work between them, give the eager result every time."""
    lib = _lib.load()
    g = 128
    w = randn_bf16((4096, 4096), std=0.02, seed=41).to(DEV)
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(w, g, 8)
    x = randn_bf16((32, 4096), seed=42).to(DEV)
    y = torch.empty((32, 4096), dtype=torch.bfloat16, device=DEV)

    def call():
        rc = lib.e2h_int4_mm_static_scratch(ops._ptr(x), ops._ptr(packed), ops._ptr(sz), ops._ptr(y), 32, 4096, 4096, g, 8, ops._stream(x))
        _lib.check(rc, "e2h_int4_mm_static_scratch")

    call()  # resolves the buffer's address on this device
    torch.cuda.synchronize()
    eager = y.clone()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    assert torch.equal(y, eager)

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        call()
    for i in range(4):
        y.fill_(float("nan"))
        # eager work on the shared scratch between the replays
        x2 = randn_bf16((7, 4096), seed=50 + i).to(DEV)
        y2 = torch.empty((7, 4096), dtype=torch.bfloat16, device=DEV)
        rc = lib.e2h_int4_mm_static_scratch(ops._ptr(x2), ops._ptr(packed), ops._ptr(sz), ops._ptr(y2), 7, 4096, 4096, g, 8, ops._stream(x2))
        _lib.check(rc, "e2h_int4_mm_static_scratch")
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay {i}"

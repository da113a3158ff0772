"""Tensor-level wrappers of the C ABI (include/e2h_quant.h) and their torch.library registrations.

PyTorch is plumbing here: it owns the device memory (caching allocator) and the stream; every
arithmetic step runs in the HIP kernels of libe2h_quant.so.  Inputs must live on the GPU -- there is no
CPU implementation behind these functions.

The `e2h::*` custom ops carry fake (meta) implementations so that modules using them trace under
torch.compile(fullgraph=True) and capture into HIP graphs (fixed launch geometry, no host sync, no
allocation outside the caching allocator, kernels on the current stream).
"""

import ctypes

import torch

from . import _lib

_VALID_GROUPS = (32, 64, 128, 256)
_VALID_IKT = (2, 4, 8)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _need_gpu(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                "e2h quantized-linear ops run only on the GPU (HIP kernels); got a tensor on %s" % t.device
            )


_workspaces = {}  # (device index, stream handle) -> scratch tensor; ("capture", device index) -> the one used under capture


def _new_workspace(device):
    return torch.zeros(int(_lib.load().e2h_workspace_bytes()), dtype=torch.uint8, device=device)


def _workspace(device):
    """Zero-initialised scratch for the split-K tickets and partial tiles, one per (device, stream): launches on one
    stream are ordered and may share it, launches on different streams must not (they would race on the tickets).

    Work recorded into a HIP graph uses one further workspace per device, allocated eagerly together with the first
    eager one: allocating it during capture would put it into the graph's private pool and record its zero fill
    into the graph.  Graphs captured on one device therefore share scratch and must not replay concurrently."""
    if torch.cuda.is_current_stream_capturing():
        ws = _workspaces.get(("capture", device.index))
        if ws is None:
            raise RuntimeError(
                "e2h: the first quantized-linear call on a device must run eagerly (it allocates the split-K scratch); "
                "run one warm-up call before capturing a HIP graph"
            )
        return ws
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None:
        if ("capture", device.index) not in _workspaces:
            _workspaces[("capture", device.index)] = _new_workspace(device)
        ws = _new_workspace(device)
        _workspaces[key] = ws
    return ws


class _OnDevice:
    """The library's entry points launch on the current device: calls for tensors of another device run under a
    device guard (the caller's current device is left as it was)."""

    def __init__(self, lib, device):
        self._lib, self._device = lib, device

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        device = self._device

        def call(*args):
            with torch.cuda.device(device):
                return fn(*args)

        return call


def _lib_for(t):
    lib = _lib.load()
    if t.device.index == torch.cuda.current_device():
        return lib
    return _OnDevice(lib, t.device)


# ---------------------------------------------------------------------------------------------
# int8
# ---------------------------------------------------------------------------------------------


def int8_quantize_per_channel(w):
    """w [N, K] float32 or bfloat16 on the GPU -> (q int8 [N, K], scales float32 [N]).

    HIP restatement of dynamically_quantize_per_channel(w.float(), -128, 127, torch.int8)
    (reference models/quantize.py:39-71)."""
    _need_gpu(w)
    assert w.dim() == 2
    if w.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"int8_quantize_per_channel: float32 or bfloat16 expected, got {w.dtype}")
    w = w.contiguous()
    n, k = w.shape
    q = torch.empty((n, k), dtype=torch.int8, device=w.device)
    scales = torch.empty((n,), dtype=torch.float32, device=w.device)
    lib = _lib_for(w)
    rc = lib.e2h_int8_quantize_per_channel(_ptr(w), int(w.dtype == torch.bfloat16), _ptr(q), _ptr(scales), None, n, k, _stream(w))
    _lib.check(rc, "e2h_int8_quantize_per_channel")
    return q, scales


def _int8_mm_impl(x, q, scales):
    _need_gpu(x, q, scales)
    if x.dtype != torch.bfloat16 or q.dtype != torch.int8 or scales.dtype != torch.bfloat16:
        raise TypeError(f"int8_mm: expected (bfloat16, int8, bfloat16), got ({x.dtype}, {q.dtype}, {scales.dtype})")
    assert x.dim() == 2 and q.dim() == 2 and scales.dim() == 1
    m, k = x.shape
    n = q.shape[0]
    if q.shape[1] != k or scales.shape[0] != n:
        raise RuntimeError(f"int8_mm: shape mismatch x{tuple(x.shape)} q{tuple(q.shape)} scales{tuple(scales.shape)}")
    x, q, scales = x.contiguous(), q.contiguous(), scales.contiguous()
    y = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    if m == 0:
        return y
    ws = _workspace(x.device)
    rc = _lib_for(x).e2h_int8_mm(_ptr(x), _ptr(q), _ptr(scales), _ptr(y), m, n, k, _ptr(ws), ws.numel(), _stream(x))
    _lib.check(rc, "e2h_int8_mm")
    return y


# ---------------------------------------------------------------------------------------------
# int4
# ---------------------------------------------------------------------------------------------


def _check_bf16_2d(w, what):
    _need_gpu(w)
    if w.dtype != torch.bfloat16:
        raise TypeError(f"{what}: bfloat16 weight expected (the reference quantizes int4 in bfloat16), got {w.dtype}")
    assert w.dim() == 2


def int4_group_qparams(w, groupsize):
    """get_group_qparams (reference models/quantize.py:74-92): bf16 [N, K] -> scales, zeros bf16 [N, K/g]."""
    _check_bf16_2d(w, "int4_group_qparams")
    w = w.contiguous()
    n, k = w.shape
    scales = torch.empty((n, k // groupsize), dtype=torch.bfloat16, device=w.device)
    zeros = torch.empty_like(scales)
    rc = _lib_for(w).e2h_int4_group_qparams(_ptr(w), _ptr(scales), _ptr(zeros), n, k, groupsize, _stream(w))
    _lib.check(rc, "e2h_int4_group_qparams")
    return scales, zeros


def int4_quantize_from_qparams(w, scales, zeros, groupsize):
    """group_quantize_tensor_from_qparams (reference :118-144) -> int32 codes [N, K]."""
    _check_bf16_2d(w, "int4_quantize_from_qparams")
    _need_gpu(scales, zeros)
    if scales.dtype != torch.bfloat16 or zeros.dtype != torch.bfloat16:
        raise TypeError("int4_quantize_from_qparams: bfloat16 qparams expected")
    w = w.contiguous()
    n, k = w.shape
    scales = scales.reshape(n, -1).contiguous()
    zeros = zeros.reshape(n, -1).contiguous()
    assert scales.shape == (n, k // groupsize) and zeros.shape == scales.shape
    codes = torch.empty((n, k), dtype=torch.int32, device=w.device)
    rc = _lib_for(w).e2h_int4_quantize_from_qparams(_ptr(w), _ptr(scales), _ptr(zeros), _ptr(codes), n, k, groupsize, _stream(w))
    _lib.check(rc, "e2h_int4_quantize_from_qparams")
    return codes


def int4_group_quantize(w, groupsize):
    """group_quantize_tensor (reference :147-151) -> (codes int32 [N, K], scales_and_zeros bf16 [K/g, N, 2])."""
    _check_bf16_2d(w, "int4_group_quantize")
    w = w.contiguous()
    n, k = w.shape
    codes = torch.empty((n, k), dtype=torch.int32, device=w.device)
    sz = torch.empty((k // groupsize, n, 2), dtype=torch.bfloat16, device=w.device)
    rc = _lib_for(w).e2h_int4_group_quantize(_ptr(w), _ptr(codes), _ptr(sz), n, k, groupsize, _stream(w))
    _lib.check(rc, "e2h_int4_group_quantize")
    return codes, sz


def int4_dequantize_codes(codes, scales, zeros, groupsize):
    """group_dequantize_tensor_from_qparams (reference :154-171) on bfloat16 qparams -> bf16 [N, K]."""
    _need_gpu(codes, scales, zeros)
    if codes.dtype != torch.int32 or scales.dtype != torch.bfloat16 or zeros.dtype != torch.bfloat16:
        raise TypeError("int4_dequantize_codes: expected (int32, bfloat16, bfloat16)")
    n, k = codes.shape
    codes = codes.contiguous()
    scales = scales.reshape(n, -1).contiguous()
    zeros = zeros.reshape(n, -1).contiguous()
    assert scales.shape == (n, k // groupsize) and zeros.shape == scales.shape
    out = torch.empty((n, k), dtype=torch.bfloat16, device=codes.device)
    rc = _lib_for(codes).e2h_int4_dequantize_codes(_ptr(codes), _ptr(scales), _ptr(zeros), _ptr(out), n, k, groupsize, _stream(codes))
    _lib.check(rc, "e2h_int4_dequantize_codes")
    return out


def _int4_pack_impl(codes, inner_k_tiles):
    _need_gpu(codes)
    if codes.dtype != torch.int32:
        raise TypeError(f"int4_pack: int32 codes expected, got {codes.dtype}")
    assert codes.dim() == 2
    codes = codes.contiguous()
    n, k = codes.shape
    if inner_k_tiles not in _VALID_IKT or n % 8 != 0 or k % (16 * inner_k_tiles) != 0:
        raise RuntimeError(f"int4_pack: need n % 8 == 0, inner_k_tiles in (2,4,8) and k % (16*inner_k_tiles) == 0; got n={n} k={k} ikt={inner_k_tiles}")
    packed = torch.empty((n // 8, k // (16 * inner_k_tiles), 32, inner_k_tiles // 2), dtype=torch.int32, device=codes.device)
    rc = _lib_for(codes).e2h_int4_pack(_ptr(codes), _ptr(packed), n, k, inner_k_tiles, _stream(codes))
    _lib.check(rc, "e2h_int4_pack")
    return packed


def _packed_dims(packed):
    if packed.dim() != 4 or packed.shape[2] != 32 or packed.dtype != torch.int32:
        raise RuntimeError(f"expected a tile-packed int32 weight [N/8, K/(16*ikt), 32, ikt/2], got {packed.dtype}{tuple(packed.shape)}")
    ikt = packed.shape[3] * 2
    if ikt not in _VALID_IKT:
        raise RuntimeError(f"tile-packed weight has inner_k_tiles={ikt}, expected 2, 4 or 8")
    return packed.shape[0] * 8, packed.shape[1] * 16 * ikt, ikt


def int4_unpack(packed):
    """Inverse of int4_pack: tile-packed int32 -> int32 codes [N, K]."""
    _need_gpu(packed)
    n, k, ikt = _packed_dims(packed)
    packed = packed.contiguous()
    codes = torch.empty((n, k), dtype=torch.int32, device=packed.device)
    rc = _lib_for(packed).e2h_int4_unpack(_ptr(packed), _ptr(codes), n, k, ikt, _stream(packed))
    _lib.check(rc, "e2h_int4_unpack")
    return codes


def int4_quantize_pack(w, groupsize, inner_k_tiles):
    """prepare_int4_weight_and_scales_and_zeros (reference :435-442), fused on the GPU.

    Falls back to the two-kernel route (quantize, then pack) for K not a multiple of 256."""
    _check_bf16_2d(w, "int4_quantize_pack")
    w = w.contiguous()
    n, k = w.shape
    if groupsize not in _VALID_GROUPS or inner_k_tiles not in _VALID_IKT:
        raise RuntimeError(f"int4_quantize_pack: unsupported groupsize={groupsize} / inner_k_tiles={inner_k_tiles}")
    if n % 8 != 0 or k % groupsize != 0 or k % (16 * inner_k_tiles) != 0:
        raise RuntimeError(f"int4_quantize_pack: unsupported shape n={n} k={k} for groupsize={groupsize}, inner_k_tiles={inner_k_tiles}")
    if k % 256 != 0:
        codes, sz = int4_group_quantize(w, groupsize)
        return _int4_pack_impl(codes, inner_k_tiles), sz
    packed = torch.empty((n // 8, k // (16 * inner_k_tiles), 32, inner_k_tiles // 2), dtype=torch.int32, device=w.device)
    sz = torch.empty((k // groupsize, n, 2), dtype=torch.bfloat16, device=w.device)
    rc = _lib_for(w).e2h_int4_quantize_pack(_ptr(w), _ptr(packed), _ptr(sz), n, k, groupsize, inner_k_tiles, _stream(w))
    _lib.check(rc, "e2h_int4_quantize_pack")
    return packed, sz


def int4_dequantize(packed, scales_and_zeros, groupsize):
    """Tile-packed weight + scales_and_zeros -> bf16 [N, K] with the rounding of reference :154-171."""
    _need_gpu(packed, scales_and_zeros)
    n, k, ikt = _packed_dims(packed)
    if scales_and_zeros.dtype != torch.bfloat16 or tuple(scales_and_zeros.shape) != (k // groupsize, n, 2):
        raise RuntimeError(f"int4_dequantize: scales_and_zeros must be bf16 [{k // groupsize}, {n}, 2], got {scales_and_zeros.dtype}{tuple(scales_and_zeros.shape)}")
    packed, sz = packed.contiguous(), scales_and_zeros.contiguous()
    out = torch.empty((n, k), dtype=torch.bfloat16, device=packed.device)
    rc = _lib_for(packed).e2h_int4_dequantize(_ptr(packed), _ptr(sz), _ptr(out), n, k, groupsize, ikt, _stream(packed))
    _lib.check(rc, "e2h_int4_dequantize")
    return out


def _int4_mm_impl(x, packed, groupsize, scales_and_zeros):
    _need_gpu(x, packed, scales_and_zeros)
    if x.dtype != torch.bfloat16 or scales_and_zeros.dtype != torch.bfloat16:
        raise TypeError(f"int4_mm: bfloat16 activations and scales_and_zeros expected, got {x.dtype}, {scales_and_zeros.dtype}")
    assert x.dim() == 2
    n, k, ikt = _packed_dims(packed)
    m = x.shape[0]
    if x.shape[1] != k:
        raise RuntimeError(f"int4_mm: x has K={x.shape[1]}, packed weight has K={k}")
    if groupsize not in _VALID_GROUPS or k % groupsize != 0:
        raise RuntimeError(f"int4_mm: groupsize={groupsize} must be one of {_VALID_GROUPS} and divide K={k}")
    if tuple(scales_and_zeros.shape) != (k // groupsize, n, 2):
        raise RuntimeError(f"int4_mm: scales_and_zeros must be [{k // groupsize}, {n}, 2], got {tuple(scales_and_zeros.shape)}")
    x, packed, sz = x.contiguous(), packed.contiguous(), scales_and_zeros.contiguous()
    y = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    if m == 0:
        return y
    ws = _workspace(x.device)
    rc = _lib_for(x).e2h_int4_mm(_ptr(x), _ptr(packed), _ptr(sz), _ptr(y), m, n, k, groupsize, ikt, _ptr(ws), ws.numel(), _stream(x))
    _lib.check(rc, "e2h_int4_mm")
    return y


def int4_gate_supported(x, w_gate, w_up):
    """True when (x, two WeightOnlyInt4Linear modules) fit e2h_int4_mm_silu_gate's contract."""
    if not (x.is_cuda and x.dtype == torch.bfloat16 and x.numel() // x.shape[-1] <= 64):
        return False
    pg, pu = w_gate.weight, w_up.weight
    if pg.shape != pu.shape or pg.dim() != 4 or pg.shape[3] != 4 or w_gate.groupsize != w_up.groupsize:
        return False
    return w_gate.groupsize in (32, 64, 128) and w_gate.scales_and_zeros.shape == w_up.scales_and_zeros.shape


def int4_mm_silu_gate(x, packed_gate, sz_gate, packed_up, sz_up, groupsize):
    """bf16(bf16(silu(int4_mm(x, gate))) * int4_mm(x, up)) in one launch; x bf16 [M <= 64, K]."""
    _need_gpu(x, packed_gate, sz_gate, packed_up, sz_up)
    if x.dtype != torch.bfloat16 or sz_gate.dtype != torch.bfloat16 or sz_up.dtype != torch.bfloat16:
        raise TypeError("int4_mm_silu_gate: bfloat16 activations and scales_and_zeros expected")
    assert x.dim() == 2
    n, k, ikt = _packed_dims(packed_gate)
    if _packed_dims(packed_up) != (n, k, ikt):
        raise RuntimeError("int4_mm_silu_gate: the two packed weights differ in shape")
    m = x.shape[0]
    if x.shape[1] != k:
        raise RuntimeError(f"int4_mm_silu_gate: x has K={x.shape[1]}, packed weights have K={k}")
    for sz in (sz_gate, sz_up):
        if tuple(sz.shape) != (k // groupsize, n, 2):
            raise RuntimeError(f"int4_mm_silu_gate: scales_and_zeros must be [{k // groupsize}, {n}, 2], got {tuple(sz.shape)}")
    x, packed_gate, sz_gate = x.contiguous(), packed_gate.contiguous(), sz_gate.contiguous()
    packed_up, sz_up = packed_up.contiguous(), sz_up.contiguous()
    y = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    rc = _lib_for(x).e2h_int4_mm_silu_gate(_ptr(x), _ptr(packed_gate), _ptr(sz_gate), _ptr(packed_up), _ptr(sz_up), _ptr(y),
                                           m, n, k, groupsize, ikt, _stream(x))
    _lib.check(rc, "e2h_int4_mm_silu_gate")
    return y


# ---------------------------------------------------------------------------------------------
# torch.library registrations (operator boundary that replaces the two aten int4 ops and the
# F.linear * scales pair of the reference)
# ---------------------------------------------------------------------------------------------


@torch.library.custom_op("e2h::int4_mm", mutates_args=(), device_types="cuda")
def int4_mm(x: torch.Tensor, packed: torch.Tensor, groupsize: int, scales_and_zeros: torch.Tensor) -> torch.Tensor:
    """Drop-in for torch.ops.aten._weight_int4pack_mm(x, packed, groupsize, scales_and_zeros)."""
    return _int4_mm_impl(x, packed, groupsize, scales_and_zeros)


@int4_mm.register_fake
def _(x, packed, groupsize, scales_and_zeros):
    return x.new_empty((x.shape[0], packed.shape[0] * 8))


@torch.library.custom_op("e2h::int4_pack", mutates_args=(), device_types="cuda")
def int4_pack(codes: torch.Tensor, inner_k_tiles: int) -> torch.Tensor:
    """Drop-in for torch.ops.aten._convert_weight_to_int4pack(codes_int32[N, K], inner_k_tiles) (PyTorch 2.2 signature)."""
    return _int4_pack_impl(codes, inner_k_tiles)


@int4_pack.register_fake
def _(codes, inner_k_tiles):
    n, k = codes.shape
    return codes.new_empty((n // 8, k // (16 * inner_k_tiles), 32, inner_k_tiles // 2))


@torch.library.custom_op("e2h::int8_mm", mutates_args=(), device_types="cuda")
def int8_mm(x: torch.Tensor, q: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """F.linear(x, q.to(bf16)) * scales  (reference models/quantize.py:428-429) in one kernel."""
    return _int8_mm_impl(x, q, scales)


@int8_mm.register_fake
def _(x, q, scales):
    return x.new_empty((x.shape[0], q.shape[0]))


def int4_mm_direct(x, packed, groupsize, scales_and_zeros):
    """Same as the e2h::int4_mm op without the dispatcher round trip (eager hot loops)."""
    return _int4_mm_impl(x, packed, groupsize, scales_and_zeros)


def int8_mm_direct(x, q, scales):
    return _int8_mm_impl(x, q, scales)


# ---------------------------------------------------------------------------------------------
# decode-step kernels around the linears (harness side; stock torch ops are the fallback only off the GPU)
# ---------------------------------------------------------------------------------------------


def rmsnorm(x, weight, eps):
    """bf16 [..., dim] -> bf16, reference RMSNorm rounding (models/model.py:363-377)."""
    _need_gpu(x, weight)
    assert x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
    x = x.contiguous()
    y = torch.empty_like(x)
    dim = x.shape[-1]
    rc = _lib_for(x).e2h_rmsnorm(_ptr(x), _ptr(weight), _ptr(y), x.numel() // dim, dim, float(eps), _stream(x))
    _lib.check(rc, "e2h_rmsnorm")
    return y


def int4_partial_slices(rows: int, lin) -> int:
    """Number of K slices the library splits `lin` (a WeightOnlyInt4Linear) into for `rows` rows of x when its result is
    handed on as partial sums; 0 where that form does not apply (more than 64 rows, padded K, other geometries)."""
    if getattr(lin, "padding", False) and getattr(lin, "origin_in_features", lin.in_features) != lin.in_features:
        return 0
    if lin.inner_k_tiles != 8 or rows < 1 or rows > 64:
        return 0
    s = _lib.load().e2h_int4_mm_partial_slices(rows, lin.out_features, lin.in_features, lin.groupsize, lin.inner_k_tiles)
    return s if s > 0 else 0


def int4_mm_partials(x, weight_int4pack, groupsize, scales_and_zeros, slices):
    """x [M, K] bf16 -> float32 [slices, M, N]: the sums over `slices` contiguous parts of K, left for add_rmsnorm to add
    (in slice order) instead of meeting inside the matmul launch."""
    _need_gpu(x, weight_int4pack, scales_and_zeros)
    assert x.dtype == torch.bfloat16 and x.dim() == 2
    x = x.contiguous()
    n = weight_int4pack.shape[0] * 8
    m, k = x.shape
    out = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
    rc = _lib_for(x).e2h_int4_mm_partials(_ptr(x), _ptr(weight_int4pack), _ptr(scales_and_zeros), _ptr(out), m, n, k, groupsize,
                                          weight_int4pack.shape[3] * 2, slices, _stream(x))
    _lib.check(rc, "e2h_int4_mm_partials")
    return out


def int8_partial_slices(rows: int, lin) -> int:
    """As int4_partial_slices, for a WeightOnlyInt8Linear."""
    if rows < 1 or rows > 64 or lin.in_features % 128 != 0 or lin.out_features % 8 != 0:
        return 0
    s = _lib.load().e2h_int8_mm_partial_slices(rows, lin.out_features, lin.in_features)
    return s if s > 0 else 0


class ScaledPartials:
    """float32 K-slice sums [slices, rows, N] of an int8 matmul together with the column scales that turn them into the
    linear's output; add_rmsnorm takes it in place of `delta`."""

    def __init__(self, partials, scales):
        self.partials, self.scales = partials, scales


def int8_mm_partials(x, q, scales, slices):
    """x [M, K] bf16, q int8 [N, K] -> ScaledPartials (unscaled float32 sums over `slices` parts of K + the bf16 scales)."""
    _need_gpu(x, q, scales)
    assert x.dtype == torch.bfloat16 and x.dim() == 2 and q.dtype == torch.int8 and scales.dtype == torch.bfloat16
    x = x.contiguous()
    m, k = x.shape
    n = q.shape[0]
    out = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
    rc = _lib_for(x).e2h_int8_mm_partials(_ptr(x), _ptr(q), _ptr(out), m, n, k, slices, _stream(x))
    _lib.check(rc, "e2h_int8_mm_partials")
    return ScaledPartials(out, scales)


def add_rmsnorm(x, delta, weight, eps):
    """h = bf16(x + delta); returns (h, RMSNorm(h)) -- the residual add and the following norm in one kernel.  `delta` is
    either a bfloat16 tensor of x's shape, or float32 partial sums [slices, rows, dim] from int4_mm_partials, in which case
    the term added is bf16(sum over slices, in order), or the ScaledPartials of int8_mm_partials."""
    col_scales = None
    if isinstance(delta, ScaledPartials):
        delta, col_scales = delta.partials, delta.scales
    if delta.dtype == torch.float32:
        _need_gpu(x, delta, weight)
        assert x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and delta.dim() == 3 and delta.is_contiguous()
        x = x.contiguous()
        dim = x.shape[-1]
        rows = x.numel() // dim
        assert delta.shape[1] == rows and delta.shape[2] == dim
        h = torch.empty_like(x)
        y = torch.empty_like(x)
        rc = _lib_for(x).e2h_add_rmsnorm_partials(_ptr(x), _ptr(delta), delta.shape[0], _ptr(col_scales) if col_scales is not None else None,
                                                  _ptr(weight), _ptr(h), _ptr(y), rows, dim, float(eps), _stream(x))
        _lib.check(rc, "e2h_add_rmsnorm_partials")
        return h, y
    _need_gpu(x, delta, weight)
    assert x.dtype == torch.bfloat16 and delta.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.shape == delta.shape
    x, delta = x.contiguous(), delta.contiguous()
    h = torch.empty_like(x)
    y = torch.empty_like(x)
    dim = x.shape[-1]
    rc = _lib_for(x).e2h_add_rmsnorm(_ptr(x), _ptr(delta), _ptr(weight), _ptr(h), _ptr(y), x.numel() // dim, dim, float(eps), _stream(x))
    _lib.check(rc, "e2h_add_rmsnorm")
    return h, y


def silu_mul(a, b):
    """bf16(bf16(silu(a)) * b), same shape."""
    _need_gpu(a, b)
    assert a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16 and a.shape == b.shape
    a, b = a.contiguous(), b.contiguous()
    y = torch.empty_like(a)
    rc = _lib_for(a).e2h_silu_mul(_ptr(a), _ptr(b), _ptr(y), a.numel(), _stream(a))
    _lib.check(rc, "e2h_silu_mul")
    return y


def rope_kv_write(qkv, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim):
    """qkv bf16 [B, (H + 2 Hkv) * D] of one new token per sequence -> rotated q [B, H, D]; rotated k and v are
    written into the caches [Bmax, Hkv, S, D] at input_pos (int64 device tensor with one element)."""
    _need_gpu(qkv, freqs_cis, k_cache, v_cache, input_pos)
    assert qkv.dtype == torch.bfloat16 and freqs_cis.dtype == torch.bfloat16 and input_pos.dtype == torch.int64
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and freqs_cis.is_contiguous()
    qkv = qkv.contiguous()
    bsz = qkv.shape[0]
    assert qkv.shape[1] == (n_head + 2 * n_kv_head) * head_dim and k_cache.shape[1] == n_kv_head and k_cache.shape[3] == head_dim
    q = torch.empty((bsz, n_head, head_dim), dtype=torch.bfloat16, device=qkv.device)
    rc = _lib_for(qkv).e2h_rope_kv_write(_ptr(qkv), _ptr(freqs_cis), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(input_pos), bsz,
                                         n_head, n_kv_head, k_cache.shape[2], head_dim, _stream(qkv))
    _lib.check(rc, "e2h_rope_kv_write")
    return q


def rope_kv_write_seq(qkv, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim, rows_by_token=False):
    """qkv bf16 [B, T, (H + 2 Hkv) * D] -> rotated q [B, H, T, D]; rotated k and v are written into the caches
    [>= B, Hkv, S, D] at rows input_pos [T] (int64 on the device), or at rows 0 .. T-1 with rows_by_token (no KV cache)."""
    _need_gpu(qkv, freqs_cis, k_cache, v_cache, input_pos)
    assert qkv.dtype == torch.bfloat16 and freqs_cis.dtype == torch.bfloat16 and input_pos.dtype == torch.int64 and qkv.dim() == 3
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and freqs_cis.is_contiguous()
    qkv = qkv.contiguous()
    bsz, t = qkv.shape[0], qkv.shape[1]
    assert input_pos.numel() == t and qkv.shape[2] == (n_head + 2 * n_kv_head) * head_dim
    assert k_cache.shape[0] >= bsz and k_cache.shape[1] == n_kv_head and k_cache.shape[3] == head_dim and v_cache.shape == k_cache.shape
    assert rows_by_token or freqs_cis.shape[0] >= k_cache.shape[2]  # (with rows_by_token the positions must index freqs_cis)
    q = torch.empty((bsz, n_head, t, head_dim), dtype=torch.bfloat16, device=qkv.device)
    rc = _lib_for(qkv).e2h_rope_kv_write_seq(_ptr(qkv), _ptr(freqs_cis), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(input_pos.contiguous()),
                                             bsz, t, n_head, n_kv_head, k_cache.shape[2], head_dim, 1 if rows_by_token else 0, _stream(qkv))
    _lib.check(rc, "e2h_rope_kv_write_seq")
    return q


def int4_rope_kv_supported(x, wqkv, freqs_cis, k_cache):
    """True when the fused projection + RoPE + cache write covers (x [B, 1, K], a WeightOnlyInt4Linear)."""
    if not (x.is_cuda and x.dtype == torch.bfloat16 and x.numel() // x.shape[-1] <= 64):
        return False
    p = wqkv.weight
    if p.dim() != 4 or p.shape[3] != 4 or wqkv.groupsize not in (32, 64, 128) or wqkv.padding:
        return False
    return freqs_cis.shape[0] >= k_cache.shape[2]


def int4_mm_rope_kv(x, packed, scales_and_zeros, groupsize, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim):
    """x bf16 [B <= 64, K] (one new token per sequence) times the tile-packed fused q|k|v weight, then RoPE and
    the cache write of rope_kv_write, in one launch.  Returns the rotated q [B, H, D]."""
    _need_gpu(x, packed, scales_and_zeros, freqs_cis, k_cache, v_cache, input_pos)
    assert x.dtype == torch.bfloat16 and scales_and_zeros.dtype == torch.bfloat16 and freqs_cis.dtype == torch.bfloat16
    assert input_pos.dtype == torch.int64 and input_pos.numel() >= 1 and k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and freqs_cis.is_contiguous() and x.dim() == 2
    n, k, ikt = _packed_dims(packed)
    bsz = x.shape[0]
    if n != (n_head + 2 * n_kv_head) * head_dim or x.shape[1] != k:
        raise RuntimeError(f"int4_mm_rope_kv: weight is [{n}, {k}], expected [{(n_head + 2 * n_kv_head) * head_dim}, {x.shape[1]}]")
    if tuple(scales_and_zeros.shape) != (k // groupsize, n, 2):
        raise RuntimeError(f"int4_mm_rope_kv: scales_and_zeros must be [{k // groupsize}, {n}, 2], got {tuple(scales_and_zeros.shape)}")
    if k_cache.shape[0] < bsz or k_cache.shape[1] != n_kv_head or k_cache.shape[3] != head_dim or v_cache.shape != k_cache.shape:
        raise RuntimeError("int4_mm_rope_kv: caches must be [>= B, Hkv, S, D]")
    if freqs_cis.shape[0] < k_cache.shape[2] or tuple(freqs_cis.shape[1:]) != (head_dim // 2, 2):
        raise RuntimeError("int4_mm_rope_kv: freqs_cis must be [>= S, D/2, 2]")
    x, packed, sz = x.contiguous(), packed.contiguous(), scales_and_zeros.contiguous()
    q = torch.empty((bsz, n_head, head_dim), dtype=torch.bfloat16, device=x.device)
    rc = _lib_for(x).e2h_int4_mm_rope_kv(_ptr(x), _ptr(packed), _ptr(sz), _ptr(freqs_cis), _ptr(q), _ptr(k_cache), _ptr(v_cache),
                                         _ptr(input_pos), bsz, n_head, n_kv_head, head_dim, k_cache.shape[2], k, groupsize, ikt,
                                         _stream(x))
    _lib.check(rc, "e2h_int4_mm_rope_kv")
    return q


def _int8_fusable(x, *mods):
    if not (x.is_cuda and x.dtype == torch.bfloat16 and x.numel() // x.shape[-1] <= 64 and x.shape[-1] % 128 == 0):
        return False
    for m in mods:
        if m.weight.dtype != torch.int8 or m.weight.dim() != 2 or m.scales.dtype != torch.bfloat16 or m.weight.shape[1] != x.shape[-1]:
            return False
        if m.weight.shape[0] * m.weight.shape[1] >= 2 ** 32:
            return False
    return True


def int8_gate_supported(x, w_gate, w_up):
    """True when (x, two WeightOnlyInt8Linear modules) fit e2h_int8_mm_silu_gate's contract."""
    return _int8_fusable(x, w_gate, w_up) and w_gate.weight.shape == w_up.weight.shape


def int8_mm_silu_gate(x, q_gate, scales_gate, q_up, scales_up):
    """bf16(bf16(silu(int8_mm(x, gate))) * int8_mm(x, up)) in one launch; x bf16 [M <= 64, K]."""
    _need_gpu(x, q_gate, scales_gate, q_up, scales_up)
    assert x.dtype == torch.bfloat16 and x.dim() == 2 and q_gate.dtype == torch.int8 and q_up.dtype == torch.int8
    assert scales_gate.dtype == torch.bfloat16 and scales_up.dtype == torch.bfloat16
    n, k = q_gate.shape
    if q_up.shape != q_gate.shape or x.shape[1] != k or scales_gate.numel() != n or scales_up.numel() != n:
        raise RuntimeError("int8_mm_silu_gate: shapes of the two linears and x do not match")
    x, q_gate, q_up = x.contiguous(), q_gate.contiguous(), q_up.contiguous()
    scales_gate, scales_up = scales_gate.contiguous(), scales_up.contiguous()
    y = torch.empty((x.shape[0], n), dtype=torch.bfloat16, device=x.device)
    rc = _lib_for(x).e2h_int8_mm_silu_gate(_ptr(x), _ptr(q_gate), _ptr(scales_gate), _ptr(q_up), _ptr(scales_up), _ptr(y), x.shape[0], n, k,
                                           _stream(x))
    _lib.check(rc, "e2h_int8_mm_silu_gate")
    return y


def int8_rope_kv_supported(x, wqkv, freqs_cis, k_cache):
    """True when the fused projection + RoPE + cache write covers (x [B, 1, K], a WeightOnlyInt8Linear)."""
    return _int8_fusable(x, wqkv) and freqs_cis.shape[0] >= k_cache.shape[2]


def int8_mm_rope_kv(x, q_weight, scales, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim):
    """x bf16 [B <= 64, K] (one new token per sequence) times the int8 fused q|k|v weight, then RoPE and the cache write
    of rope_kv_write, in one launch.  Returns the rotated q [B, H, D]."""
    _need_gpu(x, q_weight, scales, freqs_cis, k_cache, v_cache, input_pos)
    assert x.dtype == torch.bfloat16 and q_weight.dtype == torch.int8 and scales.dtype == torch.bfloat16 and freqs_cis.dtype == torch.bfloat16
    assert input_pos.dtype == torch.int64 and input_pos.numel() >= 1 and k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and freqs_cis.is_contiguous() and x.dim() == 2
    n, k = q_weight.shape
    bsz = x.shape[0]
    if n != (n_head + 2 * n_kv_head) * head_dim or x.shape[1] != k or scales.numel() != n:
        raise RuntimeError(f"int8_mm_rope_kv: weight is [{n}, {k}], expected [{(n_head + 2 * n_kv_head) * head_dim}, {x.shape[1]}]")
    if k_cache.shape[0] < bsz or k_cache.shape[1] != n_kv_head or k_cache.shape[3] != head_dim or v_cache.shape != k_cache.shape:
        raise RuntimeError("int8_mm_rope_kv: caches must be [>= B, Hkv, S, D]")
    if freqs_cis.shape[0] < k_cache.shape[2] or tuple(freqs_cis.shape[1:]) != (head_dim // 2, 2):
        raise RuntimeError("int8_mm_rope_kv: freqs_cis must be [>= S, D/2, 2]")
    x, q_weight, scales = x.contiguous(), q_weight.contiguous(), scales.contiguous()
    q = torch.empty((bsz, n_head, head_dim), dtype=torch.bfloat16, device=x.device)
    rc = _lib_for(x).e2h_int8_mm_rope_kv(_ptr(x), _ptr(q_weight), _ptr(scales), _ptr(freqs_cis), _ptr(q), _ptr(k_cache), _ptr(v_cache),
                                         _ptr(input_pos), bsz, n_head, n_kv_head, head_dim, k_cache.shape[2], k, _stream(x))
    _lib.check(rc, "e2h_int8_mm_rope_kv")
    return q


def sample_top_k(logits, q, temperature=1.0, top_k=None):
    """logits bf16 [B, V] (rows may be strided), q float32 [B, V] of Exp(1) draws -> (idx int32 [B, 1], probs float32 [B, V]):
    softmax(top-k-masked logits / max(temperature, 1e-5)) and argmax(probs / q), in one launch."""
    _need_gpu(logits, q)
    assert logits.dtype == torch.bfloat16 and logits.dim() == 2 and q.dtype == torch.float32 and q.shape == logits.shape
    if logits.stride(1) != 1:
        logits = logits.contiguous()
    q = q.contiguous()
    rows, vocab = logits.shape
    probs = torch.empty((rows, vocab), dtype=torch.float32, device=logits.device)
    idx = torch.empty((rows, 1), dtype=torch.int32, device=logits.device)
    k = 0 if top_k is None else min(int(top_k), vocab)
    rc = _lib_for(logits).e2h_sample_top_k(_ptr(logits), logits.stride(0), _ptr(q), _ptr(probs), _ptr(idx), rows, vocab,
                                          float(temperature), k, _stream(logits))
    _lib.check(rc, "e2h_sample_top_k")
    return idx, probs


def argmax_rows(logits):
    """logits bf16 [B, V] (rows may be strided) -> int64 [B, 1]: torch.argmax(logits.float(), dim=-1, keepdim=True) in one launch
    (lowest index among ties, a NaN counts as the maximum)."""
    _need_gpu(logits)
    assert logits.dtype == torch.bfloat16 and logits.dim() == 2
    if logits.stride(1) != 1:
        logits = logits.contiguous()
    rows, vocab = logits.shape
    idx = torch.empty((rows, 1), dtype=torch.int64, device=logits.device)
    rc = _lib_for(logits).e2h_argmax_rows(_ptr(logits), logits.stride(0), _ptr(idx), rows, vocab, _stream(logits))
    _lib.check(rc, "e2h_argmax_rows")
    return idx


def decode_attention(q, k_cache, v_cache, input_pos, left_pad_mask_pos=None, scale=None):
    """q bf16 [B, H, D] against caches [Bmax, Hkv, S, D] up to and including input_pos -> bf16 [B, H, D]."""
    _need_gpu(q, k_cache, v_cache, input_pos)
    assert q.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and input_pos.dtype == torch.int64
    q = q.contiguous()
    bsz, n_head, head_dim = q.shape
    if scale is None:
        scale = head_dim ** -0.5
    lp = None
    if left_pad_mask_pos is not None:
        lp = left_pad_mask_pos.to(torch.int64).contiguous()
    out = torch.empty_like(q)
    rc = _lib_for(q).e2h_decode_attention(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(input_pos), _ptr(lp) if lp is not None else None,
                                          bsz, n_head, k_cache.shape[1], k_cache.shape[2], head_dim, float(scale), _stream(q))
    _lib.check(rc, "e2h_decode_attention")
    return out


# ---------------------------------------------------------------------------------------------
# decode batches on staged activations: the int4 kernels of csrc/e2h_int4_staged.hip read their activations in
# matrix-core operand order, written by the kernel that produces them (norm, attention, gated feed-forward) or
# by stage_x for activations that arrive row-major
# ---------------------------------------------------------------------------------------------

STAGED_PLAIN, STAGED_GATE, STAGED_ROPE, STAGED_PARTIAL, STAGED_ARGMAX = 0, 1, 2, 3, 4


class StagedActivations:
    """`rows` x `k` bfloat16 activations in the operand order of the decode-batch int4 kernels, plus their sums over
    runs of 16 (csrc/e2h_staged.h describes the layout).  `buf` is the flat uint8 device buffer."""

    def __init__(self, buf, rows, k):
        self.buf, self.rows, self.k = buf, rows, k

    @property
    def device(self):
        return self.buf.device


def staged_empty(rows, k, device):
    nbytes = int(_lib.load().e2h_int4_staged_bytes(rows, k))
    if nbytes <= 0:
        raise RuntimeError(f"staged activations need 1 <= rows <= 64 and k % 128 == 0, got rows={rows}, k={k}")
    return StagedActivations(torch.empty((nbytes,), dtype=torch.uint8, device=device), rows, k)


def stage_x(x):
    """x bf16 [rows <= 64, k] row-major -> StagedActivations (one pass over x)."""
    _need_gpu(x)
    assert x.dtype == torch.bfloat16 and x.dim() == 2
    x = x.contiguous()
    out = staged_empty(x.shape[0], x.shape[1], x.device)
    rc = _lib_for(x).e2h_int4_stage_x(_ptr(x), _ptr(out.buf), x.shape[0], x.shape[1], _stream(x))
    _lib.check(rc, "e2h_int4_stage_x")
    return out


def int4_staged_supported(rows, lin, epilogue):
    """True when the staged decode-batch kernel covers `lin` (a WeightOnlyInt4Linear) at `rows` rows with the epilogue."""
    if getattr(lin, "padding", False) or lin.inner_k_tiles != 8 or lin.weight.dim() != 4 or not lin.weight.is_cuda:
        return False
    if lin.scales_and_zeros.dtype != torch.bfloat16:
        return False
    return bool(_lib.load().e2h_int4_mm_staged_supported(rows, lin.out_features, lin.in_features, lin.groupsize, epilogue))


def _staged_dims(xs, packed, sz, groupsize, what):
    n, k, ikt = _packed_dims(packed)
    if ikt != 8 or xs.k != k:
        raise RuntimeError(f"{what}: staged activations have K={xs.k}, packed weight has K={k}, inner_k_tiles={ikt} (8 expected)")
    if tuple(sz.shape) != (k // groupsize, n, 2) or sz.dtype != torch.bfloat16:
        raise RuntimeError(f"{what}: scales_and_zeros must be bfloat16 [{k // groupsize}, {n}, 2], got {sz.dtype} {tuple(sz.shape)}")
    return n, k


def int4_mm_staged(xs, packed, groupsize, scales_and_zeros):
    """int4_mm on staged activations -> bf16 [rows, N]."""
    _need_gpu(xs.buf, packed, scales_and_zeros)
    n, k = _staged_dims(xs, packed, scales_and_zeros, groupsize, "int4_mm_staged")
    y = torch.empty((xs.rows, n), dtype=torch.bfloat16, device=xs.device)
    rc = _lib_for(y).e2h_int4_mm_staged(_ptr(xs.buf), _ptr(packed), _ptr(scales_and_zeros), _ptr(y), xs.rows, n, k, groupsize, _stream(y))
    _lib.check(rc, "e2h_int4_mm_staged")
    return y


def int4_mm_staged_argmax(xs, packed, groupsize, scales_and_zeros):
    """argmax over the columns of int4_mm_staged(xs, ...) without storing the product -> int64 [rows, 1] (greedy token from
    the LM head; lowest index among ties, a NaN counts as the maximum, as argmax_rows)."""
    _need_gpu(xs.buf, packed, scales_and_zeros)
    n, k = _staged_dims(xs, packed, scales_and_zeros, groupsize, "int4_mm_staged_argmax")
    lib = _lib_for(xs.buf)
    nbytes = int(lib.e2h_int4_mm_staged_argmax_scratch_bytes(xs.rows, n, k, groupsize))
    if nbytes <= 0:
        _lib.check(nbytes if nbytes < 0 else -2, "e2h_int4_mm_staged_argmax_scratch_bytes")
    scratch = torch.empty((nbytes // 8,), dtype=torch.int64, device=xs.device)
    tokens = torch.empty((xs.rows, 1), dtype=torch.int64, device=xs.device)
    rc = lib.e2h_int4_mm_staged_argmax(_ptr(xs.buf), _ptr(packed), _ptr(scales_and_zeros), _ptr(scratch), _ptr(tokens), xs.rows, n, k,
                                       groupsize, _stream(tokens))
    _lib.check(rc, "e2h_int4_mm_staged_argmax")
    return tokens


def int4_staged_partial_slices(rows, lin):
    s = _lib.load().e2h_int4_mm_staged_partial_slices(rows, lin.out_features, lin.in_features, lin.groupsize)
    return s if s > 0 else 0


def int4_mm_staged_partials(xs, packed, groupsize, scales_and_zeros, slices):
    """-> float32 [slices, rows, N]: the sums over `slices` contiguous parts of K, for add_rmsnorm_staged to add in order."""
    _need_gpu(xs.buf, packed, scales_and_zeros)
    n, k = _staged_dims(xs, packed, scales_and_zeros, groupsize, "int4_mm_staged_partials")
    out = torch.empty((slices, xs.rows, n), dtype=torch.float32, device=xs.device)
    rc = _lib_for(out).e2h_int4_mm_staged_partials(_ptr(xs.buf), _ptr(packed), _ptr(scales_and_zeros), _ptr(out), xs.rows, n, k, groupsize,
                                                   slices, _stream(out))
    _lib.check(rc, "e2h_int4_mm_staged_partials")
    return out


def int4_mm_staged_silu_gate(xs, packed_gate, sz_gate, packed_up, sz_up, groupsize, want_rows=False, want_staged=True):
    """bf16(bf16(silu(gate x)) * up x) for two packed weights of equal shape.  Returns (y or None, StagedActivations or None):
    the row-major result and / or its staged form for the next linear (N % 128 == 0 then)."""
    _need_gpu(xs.buf, packed_gate, sz_gate, packed_up, sz_up)
    n, k = _staged_dims(xs, packed_gate, sz_gate, groupsize, "int4_mm_staged_silu_gate")
    if _staged_dims(xs, packed_up, sz_up, groupsize, "int4_mm_staged_silu_gate") != (n, k):
        raise RuntimeError("int4_mm_staged_silu_gate: the two packed weights differ in shape")
    y = torch.empty((xs.rows, n), dtype=torch.bfloat16, device=xs.device) if want_rows else None
    out = staged_empty(xs.rows, n, xs.device) if want_staged else None
    rc = _lib_for(xs.buf).e2h_int4_mm_staged_silu_gate(_ptr(xs.buf), _ptr(packed_gate), _ptr(sz_gate), _ptr(packed_up), _ptr(sz_up),
                                                       _ptr(y) if y is not None else None, _ptr(out.buf) if out is not None else None,
                                                       xs.rows, n, k, groupsize, _stream(xs.buf))
    _lib.check(rc, "e2h_int4_mm_staged_silu_gate")
    return y, out


def int4_mm_staged_rope_kv(xs, packed, scales_and_zeros, groupsize, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim):
    """int4_mm_rope_kv on staged activations: fused q|k|v projection, RoPE, cache write; returns the rotated q [B, H, D]."""
    _need_gpu(xs.buf, packed, scales_and_zeros, freqs_cis, k_cache, v_cache, input_pos)
    assert freqs_cis.dtype == torch.bfloat16 and input_pos.dtype == torch.int64 and input_pos.numel() >= 1
    assert k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and freqs_cis.is_contiguous()
    n, k = _staged_dims(xs, packed, scales_and_zeros, groupsize, "int4_mm_staged_rope_kv")
    bsz = xs.rows
    if n != (n_head + 2 * n_kv_head) * head_dim:
        raise RuntimeError(f"int4_mm_staged_rope_kv: weight has N={n}, expected {(n_head + 2 * n_kv_head) * head_dim}")
    if k_cache.shape[0] < bsz or k_cache.shape[1] != n_kv_head or k_cache.shape[3] != head_dim or v_cache.shape != k_cache.shape:
        raise RuntimeError("int4_mm_staged_rope_kv: caches must be [>= B, Hkv, S, D]")
    if freqs_cis.shape[0] < k_cache.shape[2] or tuple(freqs_cis.shape[1:]) != (head_dim // 2, 2):
        raise RuntimeError("int4_mm_staged_rope_kv: freqs_cis must be [>= S, D/2, 2]")
    q = torch.empty((bsz, n_head, head_dim), dtype=torch.bfloat16, device=xs.device)
    rc = _lib_for(q).e2h_int4_mm_staged_rope_kv(_ptr(xs.buf), _ptr(packed), _ptr(scales_and_zeros), _ptr(freqs_cis), _ptr(q), _ptr(k_cache),
                                                _ptr(v_cache), _ptr(input_pos), bsz, n_head, n_kv_head, head_dim, k_cache.shape[2], k,
                                                groupsize, _stream(q))
    _lib.check(rc, "e2h_int4_mm_staged_rope_kv")
    return q


def add_rmsnorm_staged(x, delta, weight, eps, want_rows=False):
    """RMSNorm of h = x (delta None) or h = bf16(x + delta) (delta bf16 of x's shape, or float32 partial sums
    [slices, rows, dim]) with the normalised rows handed on as StagedActivations.  Returns (h, y or None, staged)."""
    _need_gpu(x, weight)
    assert x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
    x = x.contiguous()
    dim = x.shape[-1]
    rows = x.numel() // dim
    staged = staged_empty(rows, dim, x.device)
    y = torch.empty_like(x) if want_rows else None
    d16 = part = None
    slices = 0
    h = x
    if delta is not None:
        h = torch.empty_like(x)
        if delta.dtype == torch.float32:
            assert delta.dim() == 3 and delta.is_contiguous() and delta.shape[1] == rows and delta.shape[2] == dim
            part, slices = delta, delta.shape[0]
        else:
            assert delta.dtype == torch.bfloat16 and delta.shape == x.shape
            d16 = delta.contiguous()
    rc = _lib_for(x).e2h_add_rmsnorm_staged(_ptr(x), _ptr(d16) if d16 is not None else None, _ptr(part) if part is not None else None, slices,
                                            None, _ptr(weight), _ptr(h) if delta is not None else None, _ptr(y) if y is not None else None,
                                            _ptr(staged.buf), rows, dim, float(eps), _stream(x))
    _lib.check(rc, "e2h_add_rmsnorm_staged")
    return h, y, staged


def decode_attention_staged(q, k_cache, v_cache, input_pos, left_pad_mask_pos=None, scale=None):
    """decode_attention with the result [B, H * D] handed on as StagedActivations (the input of the output projection)."""
    _need_gpu(q, k_cache, v_cache, input_pos)
    assert q.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and input_pos.dtype == torch.int64
    q = q.contiguous()
    bsz, n_head, head_dim = q.shape
    if scale is None:
        scale = head_dim ** -0.5
    lp = None
    if left_pad_mask_pos is not None:
        lp = left_pad_mask_pos.to(torch.int64).contiguous()
    staged = staged_empty(bsz, n_head * head_dim, q.device)
    rc = _lib_for(q).e2h_decode_attention_staged(_ptr(q), _ptr(k_cache), _ptr(v_cache), None, _ptr(staged.buf), _ptr(input_pos),
                                                 _ptr(lp) if lp is not None else None, bsz, n_head, k_cache.shape[1], k_cache.shape[2],
                                                 head_dim, float(scale), _stream(q))
    _lib.check(rc, "e2h_decode_attention_staged")
    return staged

"""`e2h::` custom ops for every kernel the model code calls, so that the fused decode step traces under
torch.compile(fullgraph=True) -- the call mode of the reference's decode loop (inference_generate.py:346-349) -- with
the same kernels as the eager step.

Each op is the tensor-level wrapper of ops.py behind an annotated signature, plus a fake (meta) kernel that only
allocates outputs of the right shape.  The public names in ops.py are rebound to small dispatchers: while a trace is
being taken they go through the registered op (opaque to the tracer: the ctypes launch inside is never traced), in
eager execution they call the wrapper directly, which spares the hot loop the dispatcher round trip.  The caches the
RoPE launches write are declared as mutated arguments.
"""

from typing import NamedTuple, Optional, Tuple

import torch
from torch import Tensor

from . import _lib
from . import ops as _ops

_registered = {}


def _register(name, impl, fake, mutates=()):
    op = torch.library.custom_op("e2h::" + name, impl, mutates_args=mutates, device_types="cuda")
    op.register_fake(fake)
    _registered[name] = op

    def call(*args):
        if torch.compiler.is_compiling():
            return op(*args)
        return impl(*args)

    call.__name__ = name
    call.__doc__ = impl.__doc__
    return call


def _staged_bytes(rows: int, k: int) -> int:
    mpad = (rows + 15) // 16 * 16
    return mpad * k * 2 + (k // 128) * mpad * 32


# ---- shape queries answered by the library: constants as far as a trace is concerned -------------------------------------

@torch.compiler.assume_constant_result
def _query(name: str, *args: int) -> int:
    return int(getattr(_lib.load(), name)(*args))


# ---- row-major decode-step kernels -----------------------------------------------------------------------------------------

_rmsnorm_eager = _ops.rmsnorm


def _rmsnorm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    return _rmsnorm_eager(x, weight, eps)


_add_rmsnorm_eager = _ops.add_rmsnorm


def _add_rmsnorm(x: Tensor, delta: Tensor, weight: Tensor, eps: float) -> Tuple[Tensor, Tensor]:
    return _add_rmsnorm_eager(x, delta, weight, eps)


def _add_rmsnorm_scaled(x: Tensor, partials: Tensor, scales: Tensor, weight: Tensor, eps: float) -> Tuple[Tensor, Tensor]:
    return _add_rmsnorm_eager(x, _ops.ScaledPartials(partials, scales), weight, eps)


_silu_mul_eager = _ops.silu_mul


def _silu_mul(a: Tensor, b: Tensor) -> Tensor:
    return _silu_mul_eager(a, b)


_rope_kv_write_eager = _ops.rope_kv_write


def _rope_kv_write(qkv: Tensor, freqs_cis: Tensor, k_cache: Tensor, v_cache: Tensor, input_pos: Tensor, n_head: int, n_kv_head: int,
                   head_dim: int) -> Tensor:
    return _rope_kv_write_eager(qkv, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim)


_rope_kv_write_seq_eager = _ops.rope_kv_write_seq


def _rope_kv_write_seq(qkv: Tensor, freqs_cis: Tensor, k_cache: Tensor, v_cache: Tensor, input_pos: Tensor, n_head: int, n_kv_head: int,
                       head_dim: int, rows_by_token: bool) -> Tensor:
    return _rope_kv_write_seq_eager(qkv, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim, rows_by_token)


_decode_attention_eager = _ops.decode_attention


def _decode_attention(q: Tensor, k_cache: Tensor, v_cache: Tensor, input_pos: Tensor, left_pad_mask_pos: Optional[Tensor],
                      scale: Optional[float]) -> Tensor:
    return _decode_attention_eager(q, k_cache, v_cache, input_pos, left_pad_mask_pos, scale)


_argmax_rows_eager = _ops.argmax_rows


def _argmax_rows(logits: Tensor) -> Tensor:
    return _argmax_rows_eager(logits)


_int4_gate_eager = _ops.int4_mm_silu_gate


def _int4_mm_silu_gate(x: Tensor, packed_gate: Tensor, sz_gate: Tensor, packed_up: Tensor, sz_up: Tensor, groupsize: int) -> Tensor:
    return _int4_gate_eager(x, packed_gate, sz_gate, packed_up, sz_up, groupsize)


_int4_rope_eager = _ops.int4_mm_rope_kv


def _int4_mm_rope_kv(x: Tensor, packed: Tensor, scales_and_zeros: Tensor, groupsize: int, freqs_cis: Tensor, k_cache: Tensor,
                     v_cache: Tensor, input_pos: Tensor, n_head: int, n_kv_head: int, head_dim: int) -> Tensor:
    return _int4_rope_eager(x, packed, scales_and_zeros, groupsize, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim)


_int4_partials_eager = _ops.int4_mm_partials


def _int4_mm_partials(x: Tensor, packed: Tensor, groupsize: int, scales_and_zeros: Tensor, slices: int) -> Tensor:
    return _int4_partials_eager(x, packed, groupsize, scales_and_zeros, slices)


_int8_gate_eager = _ops.int8_mm_silu_gate


def _int8_mm_silu_gate(x: Tensor, q_gate: Tensor, scales_gate: Tensor, q_up: Tensor, scales_up: Tensor) -> Tensor:
    return _int8_gate_eager(x, q_gate, scales_gate, q_up, scales_up)


_int8_rope_eager = _ops.int8_mm_rope_kv


def _int8_mm_rope_kv(x: Tensor, q_weight: Tensor, scales: Tensor, freqs_cis: Tensor, k_cache: Tensor, v_cache: Tensor, input_pos: Tensor,
                     n_head: int, n_kv_head: int, head_dim: int) -> Tensor:
    return _int8_rope_eager(x, q_weight, scales, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim)


_int8_partials_eager = _ops.int8_mm_partials


def _int8_mm_partial_sums(x: Tensor, q: Tensor, scales: Tensor, slices: int) -> Tensor:
    return _int8_partials_eager(x, q, scales, slices).partials


def _like(x, shape, dtype=None):
    return x.new_empty(shape, dtype=dtype if dtype is not None else x.dtype)


rmsnorm = _register("rmsnorm", _rmsnorm, lambda x, weight, eps: torch.empty_like(x))
_add_rmsnorm_op = _register("add_rmsnorm", _add_rmsnorm, lambda x, delta, weight, eps: (torch.empty_like(x), torch.empty_like(x)))
_add_rmsnorm_scaled_op = _register("add_rmsnorm_scaled", _add_rmsnorm_scaled,
                                   lambda x, partials, scales, weight, eps: (torch.empty_like(x), torch.empty_like(x)))
silu_mul = _register("silu_mul", _silu_mul, lambda a, b: torch.empty_like(a))
rope_kv_write = _register("rope_kv_write", _rope_kv_write,
                          lambda qkv, f, kc, vc, pos, h, hk, d: _like(qkv, (qkv.shape[0], h, d)), mutates=("k_cache", "v_cache"))
_rope_kv_write_seq_op = _register("rope_kv_write_seq", _rope_kv_write_seq,
                                  lambda qkv, f, kc, vc, pos, h, hk, d, by_token: _like(qkv, (qkv.shape[0], h, qkv.shape[1], d)),
                                  mutates=("k_cache", "v_cache"))
_decode_attention_op = _register("decode_attention", _decode_attention, lambda q, kc, vc, pos, lp, scale: torch.empty_like(q))
argmax_rows = _register("argmax_rows", _argmax_rows, lambda logits: _like(logits, (logits.shape[0], 1), torch.int64))
int4_mm_silu_gate = _register("int4_mm_silu_gate", _int4_mm_silu_gate,
                              lambda x, pg, sg, pu, su, g: _like(x, (x.shape[0], pg.shape[0] * 8)))
int4_mm_rope_kv = _register("int4_mm_rope_kv", _int4_mm_rope_kv,
                            lambda x, p, sz, g, f, kc, vc, pos, h, hk, d: _like(x, (x.shape[0], h, d)), mutates=("k_cache", "v_cache"))
int4_mm_partials = _register("int4_mm_partials", _int4_mm_partials,
                             lambda x, p, g, sz, s: _like(x, (s, x.shape[0], p.shape[0] * 8), torch.float32))
int8_mm_silu_gate = _register("int8_mm_silu_gate", _int8_mm_silu_gate, lambda x, qg, sg, qu, su: _like(x, (x.shape[0], qg.shape[0])))
int8_mm_rope_kv = _register("int8_mm_rope_kv", _int8_mm_rope_kv,
                            lambda x, q, s, f, kc, vc, pos, h, hk, d: _like(x, (x.shape[0], h, d)), mutates=("k_cache", "v_cache"))
_int8_partial_sums_op = _register("int8_mm_partial_sums", _int8_mm_partial_sums,
                                  lambda x, q, scales, s: _like(x, (s, x.shape[0], q.shape[0]), torch.float32))


class ScaledPartials(NamedTuple):
    """float32 K-slice sums [slices, rows, N] of an int8 matmul together with the column scales that turn them into the
    linear's output; add_rmsnorm takes it in place of `delta`."""

    partials: Tensor
    scales: Tensor


def int8_mm_partials(x, q, scales, slices):
    """x [M, K] bf16, q int8 [N, K] -> ScaledPartials (unscaled float32 sums over `slices` parts of K + the bf16 scales)."""
    return ScaledPartials(_int8_partial_sums_op(x, q, scales, slices), scales)


def add_rmsnorm(x, delta, weight, eps):
    """h = bf16(x + delta); returns (h, RMSNorm(h)).  `delta`: a bfloat16 tensor of x's shape, float32 partial sums
    [slices, rows, dim] of int4_mm_partials, or the ScaledPartials of int8_mm_partials."""
    if isinstance(delta, (ScaledPartials, _ops.ScaledPartials)):
        return _add_rmsnorm_scaled_op(x, delta.partials, delta.scales, weight, eps)
    return _add_rmsnorm_op(x, delta, weight, eps)


def rope_kv_write_seq(qkv, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim, rows_by_token=False):
    return _rope_kv_write_seq_op(qkv, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim, bool(rows_by_token))


def decode_attention(q, k_cache, v_cache, input_pos, left_pad_mask_pos=None, scale=None):
    return _decode_attention_op(q, k_cache, v_cache, input_pos, left_pad_mask_pos, scale)


# ---- staged decode-batch kernels: the staged buffer travels as a flat uint8 tensor with its (rows, k) --------------------

class StagedActivations(NamedTuple):
    """`rows` x `k` bfloat16 activations in the operand order of the decode-batch int4 kernels, plus their sums over runs
    of 16 (csrc/e2h_staged.h describes the layout).  `buf` is the flat uint8 device buffer."""

    buf: Tensor
    rows: int
    k: int

    @property
    def device(self):
        return self.buf.device


def _as_eager(buf, rows, k):
    return _ops.StagedActivations(buf, rows, k)


_stage_x_eager = _ops.stage_x


def _stage_x(x: Tensor) -> Tensor:
    return _stage_x_eager(x).buf


_mm_staged_eager = _ops.int4_mm_staged


def _mm_staged(buf: Tensor, rows: int, k: int, packed: Tensor, groupsize: int, scales_and_zeros: Tensor) -> Tensor:
    return _mm_staged_eager(_as_eager(buf, rows, k), packed, groupsize, scales_and_zeros)


_mm_staged_argmax_eager = _ops.int4_mm_staged_argmax


def _mm_staged_argmax(buf: Tensor, rows: int, k: int, packed: Tensor, groupsize: int, scales_and_zeros: Tensor) -> Tensor:
    return _mm_staged_argmax_eager(_as_eager(buf, rows, k), packed, groupsize, scales_and_zeros)


_mm_staged_partials_eager = _ops.int4_mm_staged_partials


def _mm_staged_partials(buf: Tensor, rows: int, k: int, packed: Tensor, groupsize: int, scales_and_zeros: Tensor, slices: int) -> Tensor:
    return _mm_staged_partials_eager(_as_eager(buf, rows, k), packed, groupsize, scales_and_zeros, slices)


_mm_staged_gate_eager = _ops.int4_mm_staged_silu_gate


def _mm_staged_silu_gate(buf: Tensor, rows: int, k: int, packed_gate: Tensor, sz_gate: Tensor, packed_up: Tensor, sz_up: Tensor,
                         groupsize: int, want_rows: bool, want_staged: bool) -> Tuple[Tensor, Tensor]:
    y, out = _mm_staged_gate_eager(_as_eager(buf, rows, k), packed_gate, sz_gate, packed_up, sz_up, groupsize, want_rows, want_staged)
    return (y if y is not None else buf.new_empty((0,), dtype=torch.bfloat16), out.buf if out is not None else buf.new_empty((0,)))


_mm_staged_rope_eager = _ops.int4_mm_staged_rope_kv


def _mm_staged_rope_kv(buf: Tensor, rows: int, k: int, packed: Tensor, scales_and_zeros: Tensor, groupsize: int, freqs_cis: Tensor,
                       k_cache: Tensor, v_cache: Tensor, input_pos: Tensor, n_head: int, n_kv_head: int, head_dim: int) -> Tensor:
    return _mm_staged_rope_eager(_as_eager(buf, rows, k), packed, scales_and_zeros, groupsize, freqs_cis, k_cache, v_cache, input_pos,
                                 n_head, n_kv_head, head_dim)


_add_rmsnorm_staged_eager = _ops.add_rmsnorm_staged


def _add_rmsnorm_staged(x: Tensor, delta: Optional[Tensor], weight: Tensor, eps: float, want_rows: bool) -> Tuple[Tensor, Tensor, Tensor]:
    h, y, staged = _add_rmsnorm_staged_eager(x, delta, weight, eps, want_rows)
    return (h if delta is not None else x.new_empty((0,)), y if y is not None else x.new_empty((0,)), staged.buf)


_attention_staged_eager = _ops.decode_attention_staged


def _decode_attention_staged(q: Tensor, k_cache: Tensor, v_cache: Tensor, input_pos: Tensor, left_pad_mask_pos: Optional[Tensor],
                             scale: Optional[float]) -> Tensor:
    return _attention_staged_eager(q, k_cache, v_cache, input_pos, left_pad_mask_pos, scale).buf


def _u8(t, n):
    return t.new_empty((n,), dtype=torch.uint8)


_stage_x_op = _register("int4_stage_x", _stage_x, lambda x: _u8(x, _staged_bytes(x.shape[0], x.shape[1])))
_mm_staged_op = _register("int4_mm_staged", _mm_staged, lambda buf, rows, k, p, g, sz: _like(sz, (rows, p.shape[0] * 8)))
_mm_staged_argmax_op = _register("int4_mm_staged_argmax", _mm_staged_argmax,
                                 lambda buf, rows, k, p, g, sz: _like(sz, (rows, 1), torch.int64))
_mm_staged_partials_op = _register("int4_mm_staged_partials", _mm_staged_partials,
                                   lambda buf, rows, k, p, g, sz, s: _like(sz, (s, rows, p.shape[0] * 8), torch.float32))
_mm_staged_gate_op = _register(
    "int4_mm_staged_silu_gate", _mm_staged_silu_gate,
    lambda buf, rows, k, pg, sg, pu, su, g, want_rows, want_staged: (
        _like(sg, (rows, pg.shape[0] * 8) if want_rows else (0,)), _u8(buf, _staged_bytes(rows, pg.shape[0] * 8) if want_staged else 0)))
_mm_staged_rope_op = _register("int4_mm_staged_rope_kv", _mm_staged_rope_kv,
                               lambda buf, rows, k, p, sz, g, f, kc, vc, pos, h, hk, d: _like(sz, (rows, h, d)),
                               mutates=("k_cache", "v_cache"))
_add_rmsnorm_staged_op = _register(
    "add_rmsnorm_staged", _add_rmsnorm_staged,
    lambda x, delta, weight, eps, want_rows: (
        torch.empty_like(x) if delta is not None else x.new_empty((0,)), torch.empty_like(x) if want_rows else x.new_empty((0,)),
        _u8(x, _staged_bytes(x.numel() // x.shape[-1], x.shape[-1]))))
_attention_staged_op = _register("decode_attention_staged", _decode_attention_staged,
                                 lambda q, kc, vc, pos, lp, scale: _u8(q, _staged_bytes(q.shape[0], q.shape[1] * q.shape[2])))


def stage_x(x):
    """x bf16 [rows <= 64, k] row-major -> StagedActivations (one pass over x)."""
    return StagedActivations(_stage_x_op(x), x.shape[0], x.shape[1])


def int4_mm_staged(xs, packed, groupsize, scales_and_zeros):
    """int4_mm on staged activations -> bf16 [rows, N]."""
    return _mm_staged_op(xs.buf, xs.rows, xs.k, packed, groupsize, scales_and_zeros)


def int4_mm_staged_argmax(xs, packed, groupsize, scales_and_zeros):
    """argmax over the columns of int4_mm_staged(xs, ...) without storing the product -> int64 [rows, 1]."""
    return _mm_staged_argmax_op(xs.buf, xs.rows, xs.k, packed, groupsize, scales_and_zeros)


def int4_mm_staged_partials(xs, packed, groupsize, scales_and_zeros, slices):
    """-> float32 [slices, rows, N]: the sums over `slices` contiguous parts of K, for add_rmsnorm_staged to add in order."""
    return _mm_staged_partials_op(xs.buf, xs.rows, xs.k, packed, groupsize, scales_and_zeros, slices)


def int4_mm_staged_silu_gate(xs, packed_gate, sz_gate, packed_up, sz_up, groupsize, want_rows=False, want_staged=True):
    """bf16(bf16(silu(gate x)) * up x) for two packed weights of equal shape.  Returns (y or None, StagedActivations or None)."""
    y, out = _mm_staged_gate_op(xs.buf, xs.rows, xs.k, packed_gate, sz_gate, packed_up, sz_up, groupsize, bool(want_rows), bool(want_staged))
    return (y if want_rows else None), (StagedActivations(out, xs.rows, packed_gate.shape[0] * 8) if want_staged else None)


def int4_mm_staged_rope_kv(xs, packed, scales_and_zeros, groupsize, freqs_cis, k_cache, v_cache, input_pos, n_head, n_kv_head, head_dim):
    """Fused q|k|v projection on staged activations, RoPE, cache write; returns the rotated q [B, H, D]."""
    return _mm_staged_rope_op(xs.buf, xs.rows, xs.k, packed, scales_and_zeros, groupsize, freqs_cis, k_cache, v_cache, input_pos, n_head,
                              n_kv_head, head_dim)


def add_rmsnorm_staged(x, delta, weight, eps, want_rows=False):
    """RMSNorm of h = x (delta None) or h = bf16(x + delta) with the normalised rows handed on as StagedActivations.
    Returns (h, y or None, staged)."""
    h, y, buf = _add_rmsnorm_staged_op(x, delta, weight, eps, bool(want_rows))
    dim = x.shape[-1]
    return (h if delta is not None else x), (y if want_rows else None), StagedActivations(buf, x.numel() // dim, dim)


def decode_attention_staged(q, k_cache, v_cache, input_pos, left_pad_mask_pos=None, scale=None):
    """decode_attention with the result [B, H * D] handed on as StagedActivations."""
    return StagedActivations(_attention_staged_op(q, k_cache, v_cache, input_pos, left_pad_mask_pos, scale), q.shape[0],
                             q.shape[1] * q.shape[2])


# ---- one-off conversion ops ------------------------------------------------------------------------------------------------

_q8_eager, _q4_eager, _unpack_eager = _ops.int8_quantize_per_channel, _ops.int4_group_quantize, _ops.int4_unpack


def _quantize_int8_per_channel(w: Tensor) -> Tuple[Tensor, Tensor]:
    return _q8_eager(w)


def _quantize_int4_group(w: Tensor, groupsize: int) -> Tuple[Tensor, Tensor]:
    return _q4_eager(w, groupsize)


def _int4_unpack(packed: Tensor) -> Tensor:
    return _unpack_eager(packed)


int8_quantize_per_channel = _register("quantize_int8_per_channel", _quantize_int8_per_channel,
                                      lambda w: (_like(w, tuple(w.shape), torch.int8), _like(w, (w.shape[0],), torch.float32)))
int4_group_quantize = _register("quantize_int4_group", _quantize_int4_group,
                                lambda w, g: (_like(w, tuple(w.shape), torch.int32), _like(w, (w.shape[1] // g, w.shape[0], 2))))
int4_unpack = _register("int4_unpack", _int4_unpack,
                        lambda p: _like(p, (p.shape[0] * 8, p.shape[1] * 16 * p.shape[3] * 2)))


# ---- shape queries ----------------------------------------------------------------------------------------------------------

def _static_rows(rows):
    """The row count as a plain int.  A trace taken with a dynamic batch dimension hands over a symbolic size, and the
    launch geometry is chosen per row count: len(range(.)) makes the tracer specialise the trace on the value."""
    return len(range(rows)) if torch.compiler.is_compiling() else rows


def int4_partial_slices(rows, lin):
    rows = _static_rows(rows)
    if getattr(lin, "padding", False) and getattr(lin, "origin_in_features", lin.in_features) != lin.in_features:
        return 0
    if lin.inner_k_tiles != 8 or rows < 1 or rows > 64:
        return 0
    s = _query("e2h_int4_mm_partial_slices", rows, lin.out_features, lin.in_features, lin.groupsize, lin.inner_k_tiles)
    return s if s > 0 else 0


def int8_partial_slices(rows, lin):
    rows = _static_rows(rows)
    if rows < 1 or rows > 64 or lin.in_features % 128 != 0 or lin.out_features % 8 != 0:
        return 0
    s = _query("e2h_int8_mm_partial_slices", rows, lin.out_features, lin.in_features)
    return s if s > 0 else 0


def int4_staged_supported(rows, lin, epilogue):
    rows = _static_rows(rows)
    if getattr(lin, "padding", False) or lin.inner_k_tiles != 8 or lin.weight.dim() != 4 or not lin.weight.is_cuda:
        return False
    if lin.scales_and_zeros.dtype != torch.bfloat16:
        return False
    return bool(_query("e2h_int4_mm_staged_supported", rows, lin.out_features, lin.in_features, lin.groupsize, epilogue))


def int4_staged_partial_slices(rows, lin):
    rows = _static_rows(rows)
    s = _query("e2h_int4_mm_staged_partial_slices", rows, lin.out_features, lin.in_features, lin.groupsize)
    return s if s > 0 else 0


_REBOUND = (
    "rmsnorm", "add_rmsnorm", "silu_mul", "rope_kv_write", "rope_kv_write_seq", "decode_attention", "argmax_rows", "int4_mm_silu_gate",
    "int4_mm_rope_kv", "int4_mm_partials", "int8_mm_silu_gate", "int8_mm_rope_kv", "int8_mm_partials", "ScaledPartials",
    "StagedActivations", "stage_x", "int4_mm_staged", "int4_mm_staged_argmax", "int4_mm_staged_partials", "int4_mm_staged_silu_gate", "int4_mm_staged_rope_kv",
    "add_rmsnorm_staged", "decode_attention_staged", "int8_quantize_per_channel", "int4_group_quantize", "int4_unpack",
    "int4_partial_slices", "int8_partial_slices", "int4_staged_supported", "int4_staged_partial_slices",
)


def install():
    """Rebind the public names of ops.py to the dispatchers above (done once, when the package is imported)."""
    for name in _REBOUND:
        setattr(_ops, name, globals()[name])

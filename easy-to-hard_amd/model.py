"""Minimal Llama-family decoder that hosts the quantized linears (harness for the decode / reward configs).

It reproduces the forward semantics and the state-dict key names of the reference's models/model.py
(Transformer :132-252, TransformerBlock :255-283, Attention :286-349, FeedForward :352-360, RMSNorm
:363-386, RoPE cache :389-412, KVCache :112-129, configs :78-109) so that a QuantHandler from
quantize.py can swap its nn.Linear children and a reference checkpoint loads key for key.  On the GPU with
bfloat16 tensors the single-token decode step runs entirely on this package's kernels (quantized linears, RMSNorm with
the residual add, RoPE + cache write, decode attention, SiLU gate); other passes use them where a fused form exists and
stock PyTorch ops elsewhere.
"""

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from . import ops
from .quantize import WeightOnlyInt4Linear, WeightOnlyInt8Linear, find_multiple

# When True (default) and the tensors are bf16 on the GPU, RMSNorm, SiLU*mul and -- for single-token steps with
# a KV cache -- RoPE + cache write + attention run as this package's fused kernels instead of chains of stock ops.
FUSED_DECODE = True
# finer switches under FUSED_DECODE (both on by default; tests and measurements turn them off to compare)
FUSE_GATE = True            # silu(w1 x) * w3 x as one int4 launch
FUSE_ROPE_PROJECTION = True  # q|k|v projection + RoPE + cache write as one int4 launch
DEFER_SPLIT_K = True         # wo / w2 hand float32 K-slice sums to the residual add + RMSNorm instead of combining them
STAGED_DECODE = True         # int4 decode step: activations travel between the kernels in matrix-core operand order
STAGED_HEAD = True           # ... including the LM head
FUSE_HEAD_ARGMAX = True      # greedy decoding: the LM head launch reduces its columns to the arg-max, no logits are stored
STAGED_MAX_ROWS = 64         # 33 .. 64 rows: wo and w2 run the one-pass 64-row kernel, the other launches two 32-row slabs


def _fusable(t: Tensor) -> bool:
    return FUSED_DECODE and t.is_cuda and t.dtype == torch.bfloat16


@dataclass
class ModelArgs:
    """reference models/model.py:42-75."""

    block_size: int = 2048
    vocab_size: int = 32000
    n_layer: int = 32
    n_head: int = 32
    dim: int = 4096
    intermediate_size: Optional[int] = None
    n_local_heads: int = -1
    head_dim: int = 64
    rope_base: float = 10000
    norm_eps: float = 1e-5

    def __post_init__(self):
        if self.n_local_heads == -1:
            self.n_local_heads = self.n_head
        if self.intermediate_size is None:
            self.intermediate_size = find_multiple(int(2 * (4 * self.dim) / 3), 256)
        self.head_dim = self.dim // self.n_head

    @classmethod
    def from_name(cls, name: str):
        if name in transformer_configs:
            return cls(**transformer_configs[name])
        matches = [c for c in transformer_configs if c in str(name).upper() or c in str(name)]
        assert len(matches) >= 1, name
        return cls(**transformer_configs[matches[0]])


# reference models/model.py:78-109 (shapes only), plus small shapes for tests
transformer_configs = {
    "CodeLlama-7b-Python-hf": dict(block_size=16384, vocab_size=32000, n_layer=32, dim=4096, rope_base=1000000),
    "llemma-7b": dict(block_size=4096, n_layer=32, n_head=32, dim=4096),
    "deepseek-math-7b": dict(block_size=4096, vocab_size=102400, n_layer=30, n_head=32, dim=4096,
                             intermediate_size=11008, rope_base=10000, norm_eps=1e-6),
    "7B": dict(n_layer=32, n_head=32, dim=4096),
    "13B": dict(n_layer=40, n_head=40, dim=5120),
    "30B": dict(n_layer=60, n_head=52, dim=6656),
    "34B": dict(block_size=4096, n_layer=48, n_head=64, dim=8192, vocab_size=32000, n_local_heads=8,
                intermediate_size=22016, rope_base=1000000),
    "70B": dict(n_layer=80, n_head=64, dim=8192, n_local_heads=8, intermediate_size=28672),
    "tiny-test": dict(block_size=256, vocab_size=512, n_layer=2, n_head=4, dim=256, intermediate_size=512),
    "tiny-gqa-test": dict(block_size=256, vocab_size=512, n_layer=2, n_head=8, n_local_heads=2, dim=512,
                          intermediate_size=1024),
}


class KVCache(nn.Module):
    """bf16 [B, H_kv, S_max, D] key and value caches written at `input_pos` (reference :112-129)."""

    def __init__(self, max_batch_size, max_seq_length, n_heads, head_dim, dtype=torch.bfloat16, device=None):
        super().__init__()
        shape = (max_batch_size, n_heads, max_seq_length, head_dim)
        self.register_buffer("k_cache", torch.zeros(shape, dtype=dtype, device=device))
        self.register_buffer("v_cache", torch.zeros(shape, dtype=dtype, device=device))

    def update(self, input_pos, k_val, v_val):
        assert input_pos.shape[0] == k_val.shape[2]
        bsz = k_val.size(0)
        self.k_cache[:bsz].index_copy_(2, input_pos, k_val)
        self.v_cache[:bsz].index_copy_(2, input_pos, v_val)
        return self.k_cache[:bsz], self.v_cache[:bsz]


class RMSNorm(nn.Module):
    """x * rsqrt(mean(x^2) + eps) in float32, cast back, times weight (reference :363-377)."""

    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: Tensor) -> Tensor:
        if _fusable(x) and self.weight.dtype == torch.bfloat16 and x.shape[-1] % 8 == 0:
            return ops.rmsnorm(x, self.weight, self.eps)
        xf = x.float()
        normed = xf * torch.rsqrt(torch.mean(xf * xf, dim=-1, keepdim=True) + self.eps)
        return normed.to(dtype=x.dtype) * self.weight


def precompute_freqs_cis(seq_len: int, n_elem: int, base: float = 10000, device=None) -> Tensor:
    """[seq_len, n_elem/2, 2] (cos, sin) table stored in bfloat16 (reference :389-397)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, n_elem, 2, device=device)[: n_elem // 2].float() / n_elem))
    angles = torch.outer(torch.arange(seq_len, device=device), inv_freq)
    return torch.stack([torch.cos(angles), torch.sin(angles)], dim=-1).to(dtype=torch.bfloat16)


def apply_rotary_emb(x: Tensor, freqs_cis: Tensor) -> Tensor:
    """Rotate interleaved pairs (x[2i], x[2i+1]) by the cached angle; float32 math (reference :400-412).

    x [B, S, H, D], freqs_cis [S, D/2, 2]."""
    pairs = x.float().reshape(*x.shape[:-1], -1, 2)
    fc = freqs_cis.view(1, pairs.size(1), 1, pairs.size(3), 2)
    re = pairs[..., 0] * fc[..., 0] - pairs[..., 1] * fc[..., 1]
    im = pairs[..., 1] * fc[..., 0] + pairs[..., 0] * fc[..., 1]
    return torch.stack([re, im], dim=-1).flatten(3).type_as(x)


def _project_deferred(lin, y2d: Tensor, lead_shape) -> Tensor:
    """`lin(y)` for the fused path, y2d [rows, K] bfloat16.  Where the library would split K over several workgroups the
    result comes back as float32 partial sums [slices, rows, N] for ops.add_rmsnorm to add, which spares the launch the
    meeting of its slices; otherwise the projection itself, shaped [*lead_shape, N]."""
    rows = y2d.shape[0]
    if isinstance(lin, WeightOnlyInt4Linear) and y2d.dtype == torch.bfloat16:
        slices = ops.int4_partial_slices(rows, lin)
        if slices > 1:
            return ops.int4_mm_partials(y2d, lin.weight, lin.groupsize, lin.scales_and_zeros, slices)
    if isinstance(lin, WeightOnlyInt8Linear) and y2d.dtype == torch.bfloat16 and lin.scales.dtype == torch.bfloat16:
        slices = ops.int8_partial_slices(rows, lin)
        if slices > 1:
            return ops.int8_mm_partials(y2d, lin.weight, lin.scales, slices)
    return lin(y2d.view(*lead_shape, -1))


class Attention(nn.Module):
    def __init__(self, config: ModelArgs):
        super().__init__()
        assert config.dim % config.n_head == 0
        total_head_dim = (config.n_head + 2 * config.n_local_heads) * config.head_dim
        self.wqkv = nn.Linear(config.dim, total_head_dim, bias=False)  # rows ordered [q | k | v]
        self.wo = nn.Linear(config.dim, config.dim, bias=False)
        self.kv_cache = None
        self.freqs_table = None        # full (cos, sin) table, set by Transformer.setup_caches
        self.left_pad_mask_pos = None  # per-step padding mask positions, set by Transformer.forward
        self.n_head = config.n_head
        self.head_dim = config.head_dim
        self.n_local_heads = config.n_local_heads
        self.dim = config.dim
        self._register_load_state_dict_pre_hook(self._fuse_qkv_hook)

    @staticmethod
    def _fuse_qkv_hook(state_dict, prefix, *args):
        # checkpoints with separate wq/wk/wv are fused on load (reference :303-308)
        if prefix + "wq.weight" in state_dict:
            parts = [state_dict.pop(prefix + n + ".weight") for n in ("wq", "wk", "wv")]
            state_dict[prefix + "wqkv.weight"] = torch.cat(parts)

    def can_fuse_decode(self, x: Tensor, fully_causal: bool) -> bool:
        return (x.shape[1] == 1 and not fully_causal and self.kv_cache is not None and _fusable(x)
                and self.freqs_table is not None and self.head_dim in (64, 128)
                and (self.n_head // self.n_local_heads) in (1, 2, 4, 8))

    def _can_fuse_prefill_rope(self, x: Tensor, input_pos: Optional[Tensor], fully_causal: bool) -> bool:
        if not (_fusable(x) and self.freqs_table is not None and self.freqs_table.dtype == torch.bfloat16):
            return False
        if input_pos is None or input_pos.dtype != torch.int64 or input_pos.numel() != x.shape[1] or self.head_dim % 2:
            return False
        if fully_causal:
            return True
        return self.kv_cache is not None and self.freqs_table.shape[0] >= self.kv_cache.k_cache.shape[2]

    def forward(self, x: Tensor, freqs_cis: Optional[Tensor], mask: Optional[Tensor], input_pos: Optional[Tensor] = None,
                fully_causal: bool = False, defer_output: bool = False) -> Tensor:
        """defer_output (fused decode step only): the output projection may come back as float32 partial sums over K
        slices, to be added by the residual add + RMSNorm that follows (ops.add_rmsnorm takes either form)."""
        bsz, seqlen, _ = x.shape
        kv_size = self.n_local_heads * self.head_dim
        if self.can_fuse_decode(x, fully_causal):
            # one new token per sequence: RoPE + cache write in one kernel, then attention over the live positions only
            w = self.wqkv
            if FUSE_ROPE_PROJECTION and isinstance(w, WeightOnlyInt4Linear) and ops.int4_rope_kv_supported(x, w, self.freqs_table, self.kv_cache.k_cache):
                # projection, rotation and cache write in one launch
                q = ops.int4_mm_rope_kv(x.view(bsz, -1), w.weight, w.scales_and_zeros, w.groupsize, self.freqs_table,
                                        self.kv_cache.k_cache, self.kv_cache.v_cache, input_pos, self.n_head,
                                        self.n_local_heads, self.head_dim)
            elif FUSE_ROPE_PROJECTION and isinstance(w, WeightOnlyInt8Linear) and ops.int8_rope_kv_supported(x, w, self.freqs_table, self.kv_cache.k_cache):
                q = ops.int8_mm_rope_kv(x.view(bsz, -1), w.weight, w.scales, self.freqs_table, self.kv_cache.k_cache,
                                        self.kv_cache.v_cache, input_pos, self.n_head, self.n_local_heads, self.head_dim)
            else:
                qkv = w(x).view(bsz, -1)
                q = ops.rope_kv_write(qkv, self.freqs_table, self.kv_cache.k_cache, self.kv_cache.v_cache, input_pos,
                                      self.n_head, self.n_local_heads, self.head_dim)
            y = ops.decode_attention(q, self.kv_cache.k_cache, self.kv_cache.v_cache, input_pos, self.left_pad_mask_pos)
            if defer_output:
                return _project_deferred(self.wo, y.view(bsz, self.dim), (bsz, 1))
            return self.wo(y.view(bsz, 1, self.dim))
        if self._can_fuse_prefill_rope(x, input_pos, fully_causal):
            # many new tokens per sequence: rotation, head-major layout and cache write in one pass over qkv
            qkv = self.wqkv(x)
            if fully_causal:
                # no cache: k and v of exactly this length, rows in token order; the angles are those of input_pos
                k = torch.empty((bsz, self.n_local_heads, seqlen, self.head_dim), dtype=torch.bfloat16, device=x.device)
                v = torch.empty_like(k)
            else:
                k, v = self.kv_cache.k_cache, self.kv_cache.v_cache
            q = ops.rope_kv_write_seq(qkv, self.freqs_table, k, v, input_pos, self.n_head, self.n_local_heads, self.head_dim,
                                      rows_by_token=fully_causal)
            k, v = k[:bsz], v[:bsz]
        else:
            q, k, v = self.wqkv(x).split([self.dim, kv_size, kv_size], dim=-1)
            q = apply_rotary_emb(q.view(bsz, seqlen, self.n_head, self.head_dim), freqs_cis).transpose(1, 2)
            k = apply_rotary_emb(k.view(bsz, seqlen, self.n_local_heads, self.head_dim), freqs_cis).transpose(1, 2)
            v = v.view(bsz, seqlen, self.n_local_heads, self.head_dim).transpose(1, 2)
            if not fully_causal:
                k, v = self.kv_cache.update(input_pos, k, v)
        rep = self.n_head // self.n_local_heads
        if rep > 1:
            k = k.repeat_interleave(rep, dim=1)
            v = v.repeat_interleave(rep, dim=1)
        if fully_causal and q.size(2) == k.size(2):
            y = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        else:
            y = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
        y = y.transpose(1, 2).contiguous().view(bsz, seqlen, self.dim)
        return self.wo(y)


class FeedForward(nn.Module):
    def __init__(self, config: ModelArgs) -> None:
        super().__init__()
        self.w1 = nn.Linear(config.dim, config.intermediate_size, bias=False)
        self.w3 = nn.Linear(config.dim, config.intermediate_size, bias=False)
        self.w2 = nn.Linear(config.intermediate_size, config.dim, bias=False)

    def _gate_fusable(self, x: Tensor) -> bool:
        w1, w3 = self.w1, self.w3
        if not (FUSED_DECODE and FUSE_GATE and isinstance(w1, WeightOnlyInt4Linear) and isinstance(w3, WeightOnlyInt4Linear)):
            return False
        if w1.padding or w3.padding:
            return False
        return ops.int4_gate_supported(x, w1, w3)

    def _gate_fusable_int8(self, x: Tensor) -> bool:
        w1, w3 = self.w1, self.w3
        if not (FUSED_DECODE and FUSE_GATE and isinstance(w1, WeightOnlyInt8Linear) and isinstance(w3, WeightOnlyInt8Linear)):
            return False
        return ops.int8_gate_supported(x, w1, w3)

    def forward(self, x: Tensor, defer_output: bool = False) -> Tensor:
        if defer_output and self._gate_fusable_int8(x):
            y = ops.int8_mm_silu_gate(x.reshape(-1, x.shape[-1]), self.w1.weight, self.w1.scales, self.w3.weight, self.w3.scales)
            return _project_deferred(self.w2, y, x.shape[:-1])
        if defer_output and self._gate_fusable(x):
            y = ops.int4_mm_silu_gate(x.reshape(-1, x.shape[-1]), self.w1.weight, self.w1.scales_and_zeros,
                                      self.w3.weight, self.w3.scales_and_zeros, self.w1.groupsize)
            return _project_deferred(self.w2, y, x.shape[:-1])
        if self._gate_fusable_int8(x):
            y = ops.int8_mm_silu_gate(x.reshape(-1, x.shape[-1]), self.w1.weight, self.w1.scales, self.w3.weight, self.w3.scales)
            return self.w2(y.reshape(*x.shape[:-1], y.shape[-1]))
        if self._gate_fusable(x):
            # silu(w1 x) * w3 x in one launch: both products share the activation stream
            y = ops.int4_mm_silu_gate(x.reshape(-1, x.shape[-1]), self.w1.weight, self.w1.scales_and_zeros,
                                      self.w3.weight, self.w3.scales_and_zeros, self.w1.groupsize)
            return self.w2(y.reshape(*x.shape[:-1], y.shape[-1]))
        a, b = self.w1(x), self.w3(x)
        if _fusable(a) and a.numel() % 8 == 0:
            return self.w2(ops.silu_mul(a, b))
        return self.w2(F.silu(a) * b)


class TransformerBlock(nn.Module):
    def __init__(self, config: ModelArgs) -> None:
        super().__init__()
        self.attention = Attention(config)
        self.feed_forward = FeedForward(config)
        self.ffn_norm = RMSNorm(config.dim, config.norm_eps)
        self.attention_norm = RMSNorm(config.dim, config.norm_eps)

    def forward(self, x: Tensor, input_pos: Tensor, freqs_cis: Tensor, mask: Optional[Tensor], fully_causal: bool = False) -> Tensor:
        return self._after_norm(x, self.attention_norm(x), input_pos, freqs_cis, mask, fully_causal)

    def _after_norm(self, x, normed, input_pos, freqs_cis, mask, fully_causal):
        attn = self.attention(normed, freqs_cis, mask, input_pos, fully_causal)
        if _fusable(x) and self.ffn_norm.weight.dtype == torch.bfloat16 and x.shape[-1] % 8 == 0:
            h, normed = ops.add_rmsnorm(x, attn, self.ffn_norm.weight, self.ffn_norm.eps)
            return h + self.feed_forward(normed)
        h = x + attn
        return h + self.feed_forward(self.ffn_norm(h))

    def forward_deferred(self, x: Tensor, delta: Optional[Tensor], input_pos, freqs_cis, mask, fully_causal: bool = False):
        """Fused-path variant: `delta` is the previous block's feed-forward output that has not been added to the
        residual stream yet; the add is folded into this block's first norm.  Returns (h, this block's pending delta)."""
        if delta is None:
            normed = ops.rmsnorm(x, self.attention_norm.weight, self.attention_norm.eps)
        else:
            x, normed = ops.add_rmsnorm(x, delta, self.attention_norm.weight, self.attention_norm.eps)
        attn = self.attention(normed, freqs_cis, mask, input_pos, fully_causal, defer_output=DEFER_SPLIT_K)
        h, normed2 = ops.add_rmsnorm(x, attn, self.ffn_norm.weight, self.ffn_norm.eps)
        return h, self.feed_forward(normed2, defer_output=DEFER_SPLIT_K)


def _staged_block_supported(blk: "TransformerBlock", rows: int) -> bool:
    """True when every linear of the block has a decode-batch kernel on staged activations for `rows` rows."""
    att, ff = blk.attention, blk.feed_forward
    lins = (att.wqkv, att.wo, ff.w1, ff.w3, ff.w2)
    if not all(isinstance(m, WeightOnlyInt4Linear) for m in lins):
        return False
    if ff.w1.groupsize != ff.w3.groupsize or ff.w1.weight.shape != ff.w3.weight.shape or ff.w1.out_features % 128 != 0:
        return False
    return (ops.int4_staged_supported(rows, att.wqkv, ops.STAGED_ROPE) and ops.int4_staged_supported(rows, att.wo, ops.STAGED_PARTIAL)
            and ops.int4_staged_supported(rows, ff.w1, ops.STAGED_GATE) and ops.int4_staged_supported(rows, ff.w2, ops.STAGED_PARTIAL))


def _staged_block_forward(blk: "TransformerBlock", x: Tensor, delta, input_pos: Tensor):
    """One decoder block of the single-token step on staged activations (reference models/model.py:279-283 with
    Attention.forward :310-349 and FeedForward.forward :359-360).  `delta` is what the previous block left to be added to
    the residual stream (float32 K-slice sums of its w2, or None); returns (residual stream, this block's w2 sums)."""
    att, ff = blk.attention, blk.feed_forward
    rows = x.shape[0]
    h, _, xs = ops.add_rmsnorm_staged(x, delta, blk.attention_norm.weight, blk.attention_norm.eps)
    w = att.wqkv
    q = ops.int4_mm_staged_rope_kv(xs, w.weight, w.scales_and_zeros, w.groupsize, att.freqs_table, att.kv_cache.k_cache,
                                   att.kv_cache.v_cache, input_pos, att.n_head, att.n_local_heads, att.head_dim)
    ys = ops.decode_attention_staged(q, att.kv_cache.k_cache, att.kv_cache.v_cache, input_pos, att.left_pad_mask_pos)
    wo = att.wo
    attn = ops.int4_mm_staged_partials(ys, wo.weight, wo.groupsize, wo.scales_and_zeros, ops.int4_staged_partial_slices(rows, wo))
    h, _, xs2 = ops.add_rmsnorm_staged(h, attn, blk.ffn_norm.weight, blk.ffn_norm.eps)
    _, gs = ops.int4_mm_staged_silu_gate(xs2, ff.w1.weight, ff.w1.scales_and_zeros, ff.w3.weight, ff.w3.scales_and_zeros, ff.w1.groupsize)
    w2 = ff.w2
    return h, ops.int4_mm_staged_partials(gs, w2.weight, w2.groupsize, w2.scales_and_zeros, ops.int4_staged_partial_slices(rows, w2))


class Transformer(nn.Module):
    def __init__(self, config: ModelArgs) -> None:
        super().__init__()
        self.config = config
        self.tok_embeddings = nn.Embedding(config.vocab_size, config.dim)
        self.layers = nn.ModuleList(TransformerBlock(config) for _ in range(config.n_layer))
        self.norm = RMSNorm(config.dim, eps=config.norm_eps)
        self.output = nn.Linear(config.dim, config.vocab_size, bias=False)
        self.freqs_cis: Optional[Tensor] = None
        self.causal_mask: Optional[Tensor] = None
        self.self_mask: Optional[Tensor] = None
        self.max_batch_size = -1
        self.max_seq_length = -1
        self.kv_cache_enabled = False

    @classmethod
    def from_name(cls, name: str):
        return cls(ModelArgs.from_name(name))

    def setup_caches(self, max_batch_size, max_seq_length, kv_cache=True):
        """reference :172-210.  Caches are created on the device of the embedding table."""
        if self.max_seq_length >= max_seq_length and self.max_batch_size >= max_batch_size:
            if self.kv_cache_enabled or not kv_cache:
                return
        device = self.tok_embeddings.weight.device
        cfg = self.config
        max_seq_length = find_multiple(max_seq_length, 8)
        self.max_seq_length = max_seq_length
        self.max_batch_size = max_batch_size
        for blk in self.layers:
            blk.attention.kv_cache = (
                KVCache(max_batch_size, max_seq_length, cfg.n_local_heads, cfg.head_dim, device=device) if kv_cache else None
            )
        self.kv_cache_enabled = kv_cache
        self.freqs_cis = precompute_freqs_cis(max(cfg.block_size, max_seq_length), cfg.head_dim, cfg.rope_base, device=device)
        for blk in self.layers:
            blk.attention.freqs_table = self.freqs_cis
        self.causal_mask = torch.tril(torch.ones(max_seq_length, max_seq_length, dtype=torch.bool, device=device))
        self.self_mask = torch.eye(max_seq_length, dtype=torch.bool, device=device)

    def staged_step_supported(self, rows: int) -> bool:
        """True when a single-token step of `rows` sequences runs on the decode-batch int4 kernels with staged activations
        (an int4 model on the GPU with bfloat16 norms and caches set up, at most STAGED_MAX_ROWS sequences)."""
        if not (FUSED_DECODE and STAGED_DECODE and FUSE_GATE and FUSE_ROPE_PROJECTION and DEFER_SPLIT_K):
            return False
        if not (1 <= rows <= STAGED_MAX_ROWS and self.config.dim % 128 == 0 and self.kv_cache_enabled and self.freqs_cis is not None):
            return False
        if self.norm.weight.dtype != torch.bfloat16 or not self.norm.weight.is_cuda or self.freqs_cis.dtype != torch.bfloat16:
            return False
        att = self.layers[0].attention
        if att.kv_cache is None or self.freqs_cis.shape[0] < att.kv_cache.k_cache.shape[2]:
            return False
        return all(_staged_block_supported(blk, rows) for blk in self.layers)

    def forward(self, idx: Tensor, input_pos: Optional[Tensor] = None, left_pad_mask_pos: Optional[Tensor] = None,
                fully_causal: bool = False, greedy_token: bool = False) -> Tensor:
        """idx [B, S] token ids, input_pos [S] positions -> logits [B, S, vocab] (reference :212-248).

        greedy_token=True (not in the reference's signature; what its decode loop computes from the logits with sampling
        switched off, inference_generate.py:110-120): -> int64 [B, 1], argmax over the vocabulary of the last position's
        logits.  In the single-token step of an int4 model the LM head launch itself reduces its columns, so the
        logits are never stored."""
        logits = self._forward(idx, input_pos, left_pad_mask_pos, fully_causal, greedy_token)
        if not greedy_token or logits.dtype == torch.int64:
            return logits
        last = logits[:, -1]
        if last.is_cuda and last.dtype == torch.bfloat16:
            return ops.argmax_rows(last)
        return torch.argmax(last.float(), dim=-1, keepdim=True)

    def _forward(self, idx: Tensor, input_pos: Optional[Tensor], left_pad_mask_pos: Optional[Tensor], fully_causal: bool,
                 greedy_token: bool) -> Tensor:
        assert self.freqs_cis is not None, "Caches must be initialized first"
        assert not (fully_causal and left_pad_mask_pos is not None), "Invalid mask"
        for blk in self.layers:
            blk.attention.left_pad_mask_pos = left_pad_mask_pos
        x = self.tok_embeddings(idx)
        mask = None
        fused_step = self.layers[0].attention.can_fuse_decode(x, fully_causal)
        if not fully_causal and not fused_step:
            mask = self.causal_mask[None, None, input_pos]
            if left_pad_mask_pos is not None:
                visible = torch.arange(mask.size(-1), device=mask.device).view(1, -1) >= left_pad_mask_pos.view(-1, 1)
                mask = torch.logical_and(mask, visible[:, None, None, :])
                mask = torch.logical_or(mask, self.self_mask[None, None, input_pos])
        freqs_cis = None if fused_step else self.freqs_cis[input_pos].to(dtype=x.dtype)
        if fused_step and input_pos.dtype != torch.int64:
            # the reference decodes with an int32 position tensor (inference_generate.py:205); the fused kernels read int64
            input_pos = input_pos.to(torch.int64)
        if fused_step and self.staged_step_supported(x.shape[0]):
            # single-token step of an int4 model: every activation between two kernels travels in operand order
            rows = x.shape[0]
            h, delta = x.view(rows, -1), None
            for blk in self.layers:
                h, delta = _staged_block_forward(blk, h, delta, input_pos)
            out = self.output
            if isinstance(out, WeightOnlyInt4Linear) and STAGED_HEAD and ops.int4_staged_supported(rows, out, ops.STAGED_PLAIN):
                _, _, xs = ops.add_rmsnorm_staged(h, delta, self.norm.weight, self.norm.eps)
                if greedy_token and FUSE_HEAD_ARGMAX and ops.int4_staged_supported(rows, out, ops.STAGED_ARGMAX):
                    return ops.int4_mm_staged_argmax(xs, out.weight, out.groupsize, out.scales_and_zeros)
                return ops.int4_mm_staged(xs, out.weight, out.groupsize, out.scales_and_zeros).view(rows, 1, -1)
            _, normed = ops.add_rmsnorm(h, delta, self.norm.weight, self.norm.eps)
            return self.output(normed.view(rows, 1, -1))
        if _fusable(x) and x.shape[-1] % 8 == 0 and self.norm.weight.dtype == torch.bfloat16:
            delta = None
            for layer in self.layers:
                x, delta = layer.forward_deferred(x, delta, input_pos, freqs_cis, mask, fully_causal)
            _, normed = ops.add_rmsnorm(x, delta, self.norm.weight, self.norm.eps)
            return self.output(normed)
        for layer in self.layers:
            x = layer(x, input_pos, freqs_cis, mask, fully_causal)
        return self.output(self.norm(x))


class RewardModel(nn.Module):
    """Backbone whose `output` is a small score head; per-token reward = mean over head rows
    (reference models/reward_model.py:69-92: `Linear(dim, 2)` head followed by `.mean(-1)`)."""

    def __init__(self, config: ModelArgs, head_rows: int = 2) -> None:
        super().__init__()
        self.backbone = Transformer(config)
        self.backbone.output = nn.Linear(config.dim, head_rows, bias=False)

    def forward(self, idx: Tensor, eos_pos: Optional[Tensor] = None) -> Tensor:
        input_pos = torch.arange(0, idx.size(-1), device=idx.device)
        rewards = self.backbone(idx, input_pos=input_pos, fully_causal=True).mean(dim=-1)
        if eos_pos is not None:
            rewards = rewards.gather(dim=-1, index=eos_pos.unsqueeze(-1)).squeeze(-1)
        return rewards

    @property
    def backbone_model(self) -> "Transformer":
        """The reference's name for the backbone (models/reward_model.py:72)."""
        return self.backbone

    @classmethod
    def from_name(cls, name: str, head_rows: int = 2) -> "RewardModel":
        return cls(ModelArgs.from_name(name), head_rows)


def apply_reward_modeling_head(transformer: "Transformer", requires_grad: bool = False, init_scheme: Optional[str] = None,
                               init_sceheme: Optional[str] = None) -> None:
    """Turn a language model's `output` projection into the two-row score head, in place (reference
    models/reward_model.py:95-133): "zeros" (the default) starts from a zero head, "semantic" from the rows of the tokens
    "2" (id 29906) and, negated, "1" (id 29896) of the existing projection, "random" from a Kaiming-uniform draw (seed 42)
    scaled by sqrt(2).  The head keeps the dtype and device of the projection it replaces.  The reference spells the
    keyword `init_sceheme` (:96); both spellings are accepted."""
    import math

    if init_scheme is not None and init_sceheme is not None and init_scheme != init_sceheme:
        raise ValueError("init_scheme and init_sceheme name different schemes")
    init_scheme = init_scheme if init_scheme is not None else (init_sceheme if init_sceheme is not None else "zeros")

    out = transformer.output
    old = out.weight
    head = torch.zeros((2, old.shape[1]), dtype=old.dtype, device=old.device)
    if init_scheme == "semantic":
        with torch.no_grad():
            head[0] = old[29906]
            head[1] = -old[29896]
    elif init_scheme == "random":
        gen = torch.Generator(device=head.device).manual_seed(42)
        nn.init.kaiming_uniform_(head, a=math.sqrt(5), generator=gen)
        head = head * math.sqrt(2.0)
    elif init_scheme != "zeros":
        raise ValueError(f"Unknown init_scheme: {init_scheme}")
    out.weight = nn.Parameter(head, requires_grad=requires_grad)
    out.out_features = 2


def init_random_(model: nn.Module, seed: int = 1234, std: float = 0.02, device=None) -> nn.Module:
    """Random-init every linear and the embedding with N(0, std), norms with ones, in bfloat16.

    A seeded CPU generator makes the values identical on every machine; `device` only chooses where the
    parameters end up."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    with torch.no_grad():
        for _, p in model.named_parameters():
            if p.dim() == 1:
                new = torch.ones(p.shape, dtype=torch.bfloat16)
            else:
                new = (torch.randn(p.shape, generator=gen, dtype=torch.float32) * std).to(torch.bfloat16)
            p.data = new.to(device if device is not None else p.device)
    return model


def random_quantized_transformer(config: ModelArgs, mode: str, groupsize: int = 128, device="cuda", seed: int = 1234,
                                 std: float = 0.02, reward_head_rows: int = 0, seed_on: str = "device") -> nn.Module:
    """Random-init model of the given shape whose linears are already quantized, built layer by layer on
    the GPU: each bf16 weight ~ N(0, std) exists only long enough to be quantized by this package's
    kernels, so a 34B-parameter model never needs its bf16 form in memory.

    mode "int4": WeightOnlyInt4Linear (groupsize, inner_k_tiles 8); mode "int8": WeightOnlyInt8Linear;
    mode "bf16": plain nn.Linear.  `reward_head_rows` > 0 wraps the backbone in a RewardModel with that many
    head rows.  seed_on "cpu": the values come from a CPU torch.Generator (the same on every machine, about 8 s per
    billion parameters); "device": from the GPU's generator (fast; the same for one GPU model and torch build)."""
    import importlib

    qz = importlib.import_module(__package__ + ".quantize")  # the package attribute `quantize` is the function

    dev = torch.device(device)
    with torch.device("meta"):
        model = RewardModel(config, reward_head_rows) if reward_head_rows else Transformer(config)
    backbone = model.backbone if reward_head_rows else model
    if mode == "int4":
        qz.WeightOnlyInt4QuantHandler(model, groupsize=groupsize).convert_for_runtime()
    elif mode == "int8":
        qz.WeightOnlyInt8QuantHandler(model).convert_for_runtime()
    else:
        assert mode == "bf16", mode
    assert seed_on in ("cpu", "device"), seed_on
    gen = torch.Generator(device="cpu" if seed_on == "cpu" else dev).manual_seed(seed)

    def rand_bf16(shape):
        if seed_on == "cpu":
            return torch.randn(shape, generator=gen, dtype=torch.float32).mul_(std).to(torch.bfloat16).to(dev)
        return (torch.randn(shape, generator=gen, device=dev, dtype=torch.float32) * std).to(torch.bfloat16)

    for _, mod in model.named_modules():
        if isinstance(mod, qz.WeightOnlyInt4Linear):
            w = rand_bf16((mod.out_features, mod.in_features))
            mod.weight, mod.scales_and_zeros = qz.prepare_int4_weight_and_scales_and_zeros(w, mod.groupsize, mod.inner_k_tiles)
        elif isinstance(mod, qz.WeightOnlyInt8Linear):
            w = rand_bf16((mod.out_features, mod.in_features))
            q, scales, _ = qz.dynamically_quantize_per_channel(w.float(), -128, 127, torch.int8)
            mod.weight, mod.scales = q, scales.to(torch.bfloat16)
        elif isinstance(mod, nn.Linear):
            mod.weight = nn.Parameter(rand_bf16(tuple(mod.weight.shape)), requires_grad=False)
        elif isinstance(mod, nn.Embedding):
            mod.weight = nn.Parameter(rand_bf16(tuple(mod.weight.shape)), requires_grad=False)
        elif isinstance(mod, RMSNorm):
            mod.weight = nn.Parameter(torch.ones(mod.weight.shape, dtype=torch.bfloat16, device=dev), requires_grad=False)
    assert not any(p.is_meta for p in model.parameters()) and not any(b.is_meta for b in model.buffers())
    backbone.eval()
    return model.eval()

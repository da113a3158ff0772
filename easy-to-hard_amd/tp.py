"""Tensor-parallel shard views of the quantized linears (host-side slicing only; nothing here communicates).

Mirrors `_apply_tp_linear` of the reference (models/tp.py:122-195): a linear is cut column-wise (output features:
`wqkv`, `w1`, `w3`, `output`) or row-wise (input features: `wo`, `w2`) into `world_size` equal parts and the module
keeps part `rank`.  The reference reads rank and world size from its process group; here they are arguments, so one
process can build every shard -- which is how the single-GPU tests check that the shards reproduce the full layer
(column shards concatenate to it, row shards sum to it; the sum is the all-reduce a multi-GPU run would do).

Buffers stay plain tensors in the checkpoint formats:
  int8  weight [N, K] int8, scales [N] bf16             colwise: weight dim 0 and scales; rowwise: weight dim 1
  int4  weight [N/8, K/128, 32, 4] int32 (inner_k_tiles 8), scales_and_zeros [K/g, N, 2] bf16
        colwise: weight dim 0 in units of 8 rows, scales_and_zeros dim 1
        rowwise: weight dim 1 in whole 128-wide k blocks, scales_and_zeros dim 0 in whole groups
"""

from typing import List, Optional

import torch
import torch.nn as nn

from .quantize import WeightOnlyInt4Linear

_DIM = {"colwise": (0, "out_features"), "rowwise": (1, "in_features")}


def apply_tp_linear(linear: nn.Module, style: str, rank: int, world_size: int, weight_splits: Optional[List[int]] = None,
                    requires_grad: bool = False) -> None:
    """In-place shard of an nn.Linear / WeightOnlyInt8Linear / WeightOnlyInt4Linear (reference models/tp.py:122-195).

    `weight_splits` = [q, k, v] sizes shards a fused qkv projection part by part, so that every rank keeps whole heads
    of each (reference :148-170)."""
    assert style in _DIM
    assert 0 <= rank < world_size
    shard_dim, size_attr = _DIM[style]
    assert getattr(linear, size_attr) % world_size == 0  # "ensure we can shard evenly" (:140)

    def shard(x, dim):
        assert x.size(dim=dim) % world_size == 0
        return torch.tensor_split(x, world_size, dim=dim)[rank]

    def shard_qkv(qkv, dim, splits):
        q, k, v = qkv.split(splits, dim=dim)
        return torch.cat((shard(q, dim), shard(k, dim), shard(v, dim)), dim=dim)

    is_int4 = isinstance(linear, WeightOnlyInt4Linear)
    if weight_splits:
        assert len(weight_splits) == 3
        if is_int4:
            sharded_weight = shard_qkv(linear.weight, shard_dim, [i // 8 for i in weight_splits])
            linear.scales_and_zeros = shard_qkv(linear.scales_and_zeros, 1 - shard_dim, weight_splits)
        else:
            sharded_weight = shard_qkv(linear.weight, shard_dim, weight_splits)
        if hasattr(linear, "scales") and style == "colwise":
            linear.scales = shard_qkv(linear.scales, 0, weight_splits)
    else:
        sharded_weight = shard(linear.weight, shard_dim)
        if is_int4:
            linear.scales_and_zeros = shard(linear.scales_and_zeros, 1 - shard_dim)
            if style == "rowwise":
                # the reference checks the same consistency with its default group size written in as a constant
                # (`shape[0] * 32`, :175-179); here the module's own group size is used
                k_shard = sharded_weight.shape[1] * sharded_weight.shape[2] * sharded_weight.shape[3]
                assert linear.scales_and_zeros.shape[0] * linear.groupsize == k_shard
                assert linear.scales_and_zeros.shape[1] == sharded_weight.shape[0] * 8
        if hasattr(linear, "scales") and style == "colwise":
            linear.scales = shard(linear.scales, 0)

    sharded_weight = sharded_weight.contiguous()
    if is_int4:
        linear.scales_and_zeros = linear.scales_and_zeros.contiguous()
    if isinstance(linear.weight, nn.Parameter):
        linear.weight = nn.Parameter(sharded_weight, requires_grad=requires_grad)
    else:
        linear.register_buffer("weight", sharded_weight)
    setattr(linear, size_attr, getattr(linear, size_attr) // world_size)
    if is_int4 and style == "rowwise" and getattr(linear, "padding", False):
        # a padded layer pads its input up to in_features in forward: the shard sees only its slice of the input
        linear.origin_in_features = linear.in_features

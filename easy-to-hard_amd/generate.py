"""Batched greedy decoding and reward scoring on top of model.Transformer (harness for the decode configs).

Follows the control flow of the reference's inference_generate.py (`prefill` :98-107, `decode_one_token`
:110-120, `decode_n_tokens` :123-157, `generate` :164-221) with greedy argmax by default and the reference's
temperature / top-k sampling (`sample` :72-85) on request, and of
inference_reward.py `model_score` (:67-91).  The decode step can be captured once into a HIP graph and
replayed per token: every kernel of this package enqueues on the current stream with a launch geometry
that depends on shapes only.
"""

from typing import Optional

import torch
from torch import Tensor

from . import ops


def greedy_token(logits: Tensor) -> Tensor:
    """argmax over the vocabulary of the last position, in float32 -> [B, 1] int64."""
    last = logits[:, -1]
    if last.is_cuda and last.dtype == torch.bfloat16:
        return ops.argmax_rows(last)
    return torch.argmax(last.float(), dim=-1, keepdim=True)


def multinomial_sample_one_no_sync(probs_sort: Tensor) -> Tensor:
    """reference inference_generate.py:53-58: exponential race, no host synchronisation."""
    q = torch.empty_like(probs_sort).exponential_(1)
    return torch.argmax(probs_sort / q, dim=-1, keepdim=True).to(dtype=torch.int)


def logits_to_probs(logits: Tensor, temperature: float = 1.0, top_k: Optional[int] = None) -> Tensor:
    """reference inference_generate.py:61-69 with stock ops (used for inputs the fused kernel does not take)."""
    logits = logits / max(temperature, 1e-5)
    if top_k is not None:
        v, _ = torch.topk(logits, min(top_k, logits.size(-1)), dim=-1)
        pivot = v.select(-1, -1).view(-1, 1)
        logits = torch.where(logits < pivot, -float("Inf"), logits)
    return torch.nn.functional.softmax(logits, dim=-1)


def sample(logits: Tensor, temperature: float = 1.0, top_k: Optional[int] = None):
    """reference inference_generate.py:72-85 (one GPU, so no vocab-parallel gather): logits [B, S, V] ->
    (idx_next int32 [B, 1], probs float32 [B, V]) for the last position.  bfloat16 logits on the GPU take the
    fused kernel; the Exp(1) draws come from torch's generator exactly as in the reference."""
    last = logits[:, -1]
    if last.is_cuda and last.dtype == torch.bfloat16:
        q = torch.empty(last.shape, dtype=torch.float32, device=last.device).exponential_(1)
        return ops.sample_top_k(last, q, temperature, top_k)
    probs = logits_to_probs(last.float(), temperature, top_k)
    return multinomial_sample_one_no_sync(probs), probs


def _next_token(logits: Tensor, temperature: Optional[float], top_k: Optional[int]) -> Tensor:
    if temperature is None:
        return greedy_token(logits)
    return sample(logits, temperature, top_k)[0].to(torch.int64)


def _greedy_through_the_model(model) -> bool:
    """True for this package's Transformer, whose forward can return the greedy token itself (a wrapped or compiled
    module, or a stand-in with the reference's signature, is asked for logits)."""
    from .model import Transformer

    return isinstance(model, Transformer)


@torch.no_grad()
def prefill(model, x: Tensor, input_pos: Tensor, left_pad_mask_pos: Optional[Tensor] = None,
            temperature: Optional[float] = None, top_k: Optional[int] = None) -> Tensor:
    """temperature None = greedy arg-max, else the reference's sampling."""
    return _next_token(model(x, input_pos, left_pad_mask_pos), temperature, top_k)


@torch.no_grad()
def decode_one_token(model, cur_token: Tensor, input_pos: Tensor, left_pad_mask_pos: Optional[Tensor] = None,
                     temperature: Optional[float] = None, top_k: Optional[int] = None) -> Tensor:
    assert input_pos.shape[-1] == 1
    if temperature is None and _greedy_through_the_model(model):
        return model(cur_token, input_pos, left_pad_mask_pos, greedy_token=True)
    return _next_token(model(cur_token, input_pos, left_pad_mask_pos), temperature, top_k)


class GraphedDecodeStep:
    """One decode step captured into a HIP graph; `step(token, pos)` copies the inputs into the static
    buffers, replays the graph and returns the static output buffer ([B, 1] next tokens)."""

    def __init__(self, model, batch_size: int, device, left_pad_mask_pos: Optional[Tensor] = None, warmup: int = 2,
                 temperature: Optional[float] = None, top_k: Optional[int] = None):
        self.model = model
        self.cur_token = torch.zeros((batch_size, 1), dtype=torch.int64, device=device)
        self.input_pos = torch.zeros((1,), dtype=torch.int64, device=device)
        self.left_pad = left_pad_mask_pos
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side):
            for _ in range(warmup):
                decode_one_token(model, self.cur_token, self.input_pos, self.left_pad, temperature, top_k)
        torch.cuda.current_stream(device).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.next_token = decode_one_token(model, self.cur_token, self.input_pos, self.left_pad, temperature, top_k)

    def step(self, cur_token: Tensor, input_pos: Tensor) -> Tensor:
        self.cur_token.copy_(cur_token)
        self.input_pos.copy_(input_pos)
        self.graph.replay()
        return self.next_token


@torch.no_grad()
def generate(model, prompt: Tensor, max_new_tokens: int, use_graph: bool = True,
             left_pad_mask_pos: Optional[Tensor] = None, stepper: Optional[GraphedDecodeStep] = None,
             temperature: Optional[float] = None, top_k: Optional[int] = None) -> Tensor:
    """prompt [B, T] int64 on the GPU -> [B, T + max_new_tokens] (prompt followed by the new tokens: greedy when
    temperature is None, else sampled as the reference does, inference_generate.py:123-221)."""
    bsz, t = prompt.shape
    total = t + max_new_tokens
    device = prompt.device
    model.setup_caches(max_batch_size=bsz, max_seq_length=min(total, model.config.block_size))
    seq = torch.empty((bsz, total), dtype=prompt.dtype, device=device)
    seq[:, :t] = prompt
    input_pos = torch.arange(0, t, device=device)
    cur = prefill(model, prompt, input_pos, left_pad_mask_pos, temperature, top_k)
    seq[:, t] = cur[:, 0]
    if max_new_tokens > 1:
        if use_graph and stepper is None:
            stepper = GraphedDecodeStep(model, bsz, device, left_pad_mask_pos, temperature=temperature, top_k=top_k)
            # the capture warm-up wrote garbage K/V at position 0 of the cache: recompute the prompt
            cur = prefill(model, prompt, input_pos, left_pad_mask_pos, temperature, top_k)
            seq[:, t] = cur[:, 0]
        pos = torch.tensor([t], device=device, dtype=torch.int64)
        for i in range(1, max_new_tokens):
            if stepper is not None:
                cur = stepper.step(cur, pos).clone()
            else:
                cur = decode_one_token(model, cur, pos, left_pad_mask_pos, temperature, top_k)
            seq[:, t + i] = cur[:, 0]
            pos += 1
    return seq


def load_model(checkpoint_path, device, precision=torch.bfloat16, use_tp: bool = False, model_name: Optional[str] = None):
    """Counterpart of the reference's `_load_model` (inference_generate.py:224-259): the quantization mode is read off
    the file name ("int8" / "int4" substrings, group size from the `.g{G}.` component), the module tree is built on the
    meta device and converted by the matching QuantHandler, the state dict is memory-mapped with a weights-only load
    and assigned, and the model moves to `device` in `precision` (integer buffers keep their dtype).

    The architecture comes from the checkpoint's parent directory name, as in the reference, unless `model_name` names
    it.  `use_tp` is accepted for signature compatibility; this build runs on one GPU and rejects it."""
    from pathlib import Path

    from .model import Transformer
    from .quantize import WeightOnlyInt4QuantHandler, WeightOnlyInt8QuantHandler

    if use_tp:
        raise NotImplementedError("load_model: tensor parallelism is outside this one-GPU build")
    checkpoint_path = Path(checkpoint_path)
    if not checkpoint_path.is_file():
        raise FileNotFoundError(str(checkpoint_path))
    with torch.device("meta"):
        model = Transformer.from_name(model_name if model_name is not None else checkpoint_path.parent.name)

    if "int8" in str(checkpoint_path):
        print("Using int8 weight-only quantization!")
        model = WeightOnlyInt8QuantHandler(model).convert_for_runtime()

    if "int4" in str(checkpoint_path):
        print("Using int4 quantization!")
        path_comps = checkpoint_path.name.split(".")
        if len(path_comps) < 3 or not path_comps[-2].startswith("g") or not path_comps[-2][1:].isdigit():
            raise ValueError(f"load_model: {checkpoint_path.name} names no group size (expected ...int4.g<G>.pth)")
        groupsize = int(path_comps[-2][1:])
        model = WeightOnlyInt4QuantHandler(model, groupsize).convert_for_runtime()

    checkpoint = torch.load(str(checkpoint_path), mmap=True, weights_only=True)
    expected = model.state_dict()
    for key, want in expected.items():
        if key in checkpoint and tuple(checkpoint[key].shape) != tuple(want.shape):
            raise ValueError(f"load_model: {key} has shape {tuple(checkpoint[key].shape)} in {checkpoint_path.name}, "
                             f"the model built for it expects {tuple(want.shape)}")
    model.load_state_dict(checkpoint, assign=True)
    model = model.to(device=device, dtype=precision)
    return model.eval()


def load_reward_model(checkpoint_path, device, precision=torch.bfloat16, use_tp: bool = False,
                      model_name: Optional[str] = None, on_the_fly_8bit_quantization: bool = False):
    """Counterpart of the reference's `_load_reward_model` (inference_reward.py:94-118) and of the quantization step
    its `main` runs afterwards (:171-178): the checkpoint is a bfloat16 language-model state dict (quantized files are
    rejected, as there), loaded memory-mapped into the backbone built on the meta device; the `output` projection becomes
    the zero-initialised two-row score head (a fine-tuned head is loaded over it by the caller); the model moves to
    `device` in `precision`; with `on_the_fly_8bit_quantization` every linear, head included, is then quantized to int8
    per channel on the device by `WeightOnlyInt8QuantHandler.convert_for_runtime_on_the_fly`."""
    from pathlib import Path

    from .model import ModelArgs, RewardModel, Transformer, apply_reward_modeling_head
    from .quantize import WeightOnlyInt8QuantHandler

    if use_tp:
        raise NotImplementedError("load_reward_model: tensor parallelism is outside this one-GPU build")
    checkpoint_path = Path(checkpoint_path)
    if "int8" in str(checkpoint_path):
        raise NotImplementedError("int8 quantization cannot be used for reward model!")
    if "int4" in str(checkpoint_path):
        raise NotImplementedError("int4 quantization cannot be used for reward model!")
    if not checkpoint_path.is_file():
        raise FileNotFoundError(str(checkpoint_path))
    config = ModelArgs.from_name(model_name if model_name is not None else checkpoint_path.parent.name)
    with torch.device("meta"):
        model = RewardModel(config)
        model.backbone = Transformer(config)  # full vocabulary projection, as in the language-model checkpoint
    checkpoint = torch.load(str(checkpoint_path), mmap=True, weights_only=True)
    model.backbone.load_state_dict(checkpoint, assign=True)
    apply_reward_modeling_head(model.backbone)
    model = model.to(device=device, dtype=precision).eval()
    if on_the_fly_8bit_quantization:
        model = WeightOnlyInt8QuantHandler(model).convert_for_runtime_on_the_fly()
        model = model.to(device=device).eval()
    return model


@torch.no_grad()
def model_score(reward_model, prompt: Tensor, max_seq_len: Optional[int] = None) -> Tensor:
    """Per-token rewards [B, T] of a RewardModel on a fully causal pass without KV cache."""
    bsz, t = prompt.shape
    reward_model.backbone.setup_caches(max_batch_size=bsz, max_seq_length=max_seq_len or t, kv_cache=False)
    return reward_model(prompt)

"""Drop-in mirror of the weight-only quantization surface of gpt-accelera's models/quantize.py.

Same names, constructor signatures, buffer names / shapes / dtypes, assertions and state-dict keys as
the reference; the arithmetic runs in the HIP kernels of libe2h_quant.so (see ops.py).  Tensors that
arrive on the CPU (the offline `quantize()` flow keeps the model on the CPU, reference :685) are moved to
the GPU for the kernel and the results are moved back -- the same thing the reference's int4 handler
does with its hard-coded `.to("cuda")` (:538).  There is no CPU arithmetic path.

Checkpoint contract (reference :383-394, :502-545, :705-718):
  int8  {fqn}.weight int8 [N, K]                         {fqn}.scales bf16 [N]
  int4  {fqn}.weight int32 [N/8, K/(16*ikt), 32, ikt/2]  {fqn}.scales_and_zeros bf16 [K/g, N, 2]
  file  model.pth -> model{label}int8.pth / model{label}int4.g{G}.pth
"""

import time
from pathlib import Path

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops


def find_multiple(n: int, k: int) -> int:
    """reference models/model.py:36-39."""
    if n % k == 0:
        return n
    return n + k - (n % k)


def _gpu_device():
    if not torch.cuda.is_available():
        raise RuntimeError("the e2h quantization kernels need a GPU (no CPU path exists)")
    return torch.device("cuda", torch.cuda.current_device())


def _on_gpu(t):
    return t if t.is_cuda else t.to(_gpu_device())


##### Quantization Primitives ######


def dynamically_quantize_per_channel(x, quant_min, quant_max, target_dtype):
    """reference :39-71.  Symmetric, axis 0, dense; returns (quant, scales float32, zero_points int64)."""
    if (quant_min, quant_max, target_dtype) != (-128, 127, torch.int8):
        raise NotImplementedError("only the int8 configuration (-128, 127, torch.int8) used by the reference's callers is implemented")
    home = x.device
    q, scales = ops.int8_quantize_per_channel(_on_gpu(x))
    zero_points = torch.zeros(scales.shape[0], dtype=torch.int64, device=home)
    return q.to(home), scales.to(home).to(x.dtype), zero_points


def get_group_qparams(w, n_bit=4, groupsize=128):
    """reference :74-92.  bf16 [N, K] -> (scales, zeros) bf16 [N, K/groupsize]."""
    if groupsize > w.shape[-1]:
        groupsize = w.shape[-1]
    assert groupsize > 1
    assert w.shape[-1] % groupsize == 0
    assert w.dim() == 2
    assert n_bit == 4, "only n_bit == 4 is implemented"
    home = x_home = w.device
    scales, zeros = ops.int4_group_qparams(_on_gpu(w), groupsize)
    return scales.to(home), zeros.to(x_home)


def pack_scales_and_zeros(scales, zeros):
    """reference :95-109 (pure index shuffle): two [N, K/g] bf16 -> [K/g, N, 2]."""
    assert scales.shape == zeros.shape
    assert scales.dtype == torch.bfloat16
    assert zeros.dtype == torch.bfloat16
    return torch.stack([scales, zeros], dim=2).transpose(0, 1).contiguous()


def unpack_scales_and_zeros(scales_and_zeros):
    """reference :112-115, accepting the bfloat16 tensors that pack_scales_and_zeros produces."""
    assert len(scales_and_zeros.shape) == 3 and scales_and_zeros.shape[2] == 2
    return torch.split(scales_and_zeros.transpose(0, 1), 1, 2)


def group_quantize_tensor_from_qparams(w, scales, zeros, n_bit=4, groupsize=128):
    """reference :118-144 -> int32 codes [N, K]."""
    assert groupsize > 1
    if groupsize > w.shape[-1] and scales.shape[-1] == 1:
        groupsize = w.shape[-1]
    assert w.shape[-1] % groupsize == 0
    assert w.dim() == 2
    assert n_bit == 4, "only n_bit == 4 is implemented"
    home = w.device
    return ops.int4_quantize_from_qparams(_on_gpu(w), _on_gpu(scales), _on_gpu(zeros), groupsize).to(home)


def group_quantize_tensor(w, n_bit=4, groupsize=128):
    """reference :147-151 -> (int32 codes [N, K], scales_and_zeros bf16 [K/g, N, 2])."""
    if groupsize > w.shape[-1]:
        groupsize = w.shape[-1]
    assert groupsize > 1
    assert w.shape[-1] % groupsize == 0
    assert w.dim() == 2
    assert n_bit == 4, "only n_bit == 4 is implemented"
    home = w.device
    codes, sz = ops.int4_group_quantize(_on_gpu(w), groupsize)
    return codes.to(home), sz.to(home)


def group_dequantize_tensor_from_qparams(w_int32, scales, zeros, n_bit=4, groupsize=128):
    """reference :154-171 on bfloat16 qparams."""
    assert groupsize > 1
    if groupsize > w_int32.shape[-1] and scales.shape[-1] == 1:
        groupsize = w_int32.shape[-1]
    assert w_int32.shape[-1] % groupsize == 0
    assert w_int32.dim() == 2
    assert n_bit == 4, "only n_bit == 4 is implemented"
    home = w_int32.device
    return ops.int4_dequantize_codes(_on_gpu(w_int32), _on_gpu(scales), _on_gpu(zeros), groupsize).to(home)


def group_dequantize_tensor(w_int32, scales_and_zeros, n_bit=4, groupsize=128):
    """reference :174-178."""
    scales, zeros = unpack_scales_and_zeros(scales_and_zeros)
    return group_dequantize_tensor_from_qparams(w_int32, scales.contiguous(), zeros.contiguous(), n_bit, groupsize)


class QuantHandler:
    """reference :181-192."""

    def __init__(self, mod):
        self.mod = mod

    def create_quantized_state_dict(self):
        pass

    def convert_for_runtime(self):
        pass

    def convert_for_runtime_on_the_fly(self):
        pass


##### Weight-only int8 per-channel quantized code ######


def _swap_linears(module, make_replacement):
    """Walk the tree; wherever a child is an nn.Linear, `make_replacement(child)` returns the module to put
    in its place (or None to leave it).  Non-linear children are searched recursively."""
    for name, child in list(module.named_children()):
        if not isinstance(child, nn.Linear):
            _swap_linears(child, make_replacement)
            continue
        repl = make_replacement(child)
        if repl is not None:
            setattr(module, name, repl)


def replace_linear_weight_only_int8_per_channel(module):
    """reference :342-351: every nn.Linear becomes an empty WeightOnlyInt8Linear (to be filled by load_state_dict)."""
    _swap_linears(module, lambda lin: WeightOnlyInt8Linear(lin.in_features, lin.out_features))


def replace_linear_weight_only_int8_per_channel_on_the_fly(module):
    """reference :354-376: quantize each nn.Linear where it lives and carry its forward / forward-pre hooks over."""

    def convert(lin):
        q, scales, _ = dynamically_quantize_per_channel(lin.weight.detach().float(), -128, 127, torch.int8)
        repl = WeightOnlyInt8Linear(lin.in_features, lin.out_features).to(lin.weight.device)
        repl.load_state_dict({"weight": q, "scales": scales})  # float32 scales are cast into the bf16 buffer
        for hook in lin._forward_hooks.values():
            repl.register_forward_hook(hook)
        for hook in lin._forward_pre_hooks.values():
            repl.register_forward_pre_hook(hook)
        return repl

    _swap_linears(module, convert)


class WeightOnlyInt8QuantHandler:
    """reference :379-402."""

    def __init__(self, mod):
        self.mod = mod

    @torch.no_grad()
    def create_quantized_state_dict(self):
        state = self.mod.state_dict()
        for fqn, lin in self.mod.named_modules():
            if not isinstance(lin, torch.nn.Linear):
                continue
            q, scales, _ = dynamically_quantize_per_channel(lin.weight.float(), -128, 127, torch.int8)
            state[f"{fqn}.weight"] = q
            state[f"{fqn}.scales"] = scales.to(lin.weight.dtype)
        return state

    def convert_for_runtime(self):
        replace_linear_weight_only_int8_per_channel(self.mod)
        return self.mod

    def convert_for_runtime_on_the_fly(self):
        replace_linear_weight_only_int8_per_channel_on_the_fly(self.mod)
        return self.mod


class WeightOnlyInt8Linear(torch.nn.Module):
    """reference :405-429.  `bias`, `device` and `dtype` are accepted and ignored, as in the reference."""

    __constants__ = ["in_features", "out_features"]
    in_features: int
    out_features: int
    weight: torch.Tensor

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer("weight", torch.empty((out_features, in_features), dtype=torch.int8))
        self.register_buffer("scales", torch.ones(out_features, dtype=torch.bfloat16))

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        # F.linear(input, self.weight.to(dtype=input.dtype)) * self.scales, as one kernel for bfloat16 activations
        if input.dtype != torch.bfloat16:
            # float16 / float32 activations are outside the measured path: they run the reference's own two stock ops
            # on the tensors' device (reference :428-429), with its dtype promotion (float16 * bfloat16 -> float32)
            return F.linear(input, self.weight.to(dtype=input.dtype)) * self.scales
        x = input.reshape(-1, input.shape[-1])
        mm = torch.ops.e2h.int8_mm if torch.compiler.is_compiling() else ops.int8_mm_direct
        y = mm(x, self.weight, self.scales)
        return y.reshape(input.shape[:-1] + (self.out_features,))


##### weight only int4 per channel groupwise quantized code ######


def prepare_int4_weight_and_scales_and_zeros(weight_bf16, groupsize, inner_k_tiles):
    """reference :435-442 -> (tile-packed int32 weight, scales_and_zeros bf16 [K/g, N, 2])."""
    home = weight_bf16.device
    packed, sz = ops.int4_quantize_pack(_on_gpu(weight_bf16), groupsize, inner_k_tiles)
    return packed.to(home), sz.to(home)


def linear_forward_int4(x, weight_int4pack, scales_and_zeros, out_features, groupsize):
    """reference :445-453."""
    origin_x_size = x.size()
    x = x.reshape(-1, origin_x_size[-1])
    mm = torch.ops.e2h.int4_mm if torch.compiler.is_compiling() else ops.int4_mm_direct
    c = mm(x, weight_int4pack, groupsize, scales_and_zeros)
    new_shape = origin_x_size[:-1] + (out_features,)
    return c.reshape(new_shape)


def _check_linear_int4_k(k, groupsize=1, inner_k_tiles=1):
    """reference :456-457."""
    return k % groupsize == 0 and k % (inner_k_tiles * 16) == 0


def replace_linear_int4(module, groupsize, inner_k_tiles, padding):
    """reference :460-490: linears whose K fits become unpadded int4 modules; the others are padded if
    `padding`, else left as they are."""

    def convert(lin):
        fits = _check_linear_int4_k(lin.in_features, groupsize, inner_k_tiles)
        if not fits and not padding:
            return None
        return WeightOnlyInt4Linear(lin.in_features, lin.out_features, bias=False, groupsize=groupsize,
                                    inner_k_tiles=inner_k_tiles, padding=not fits)

    _swap_linears(module, convert)


class WeightOnlyInt4QuantHandler:
    """reference :493-552."""

    def __init__(self, mod, groupsize=128, inner_k_tiles=8, padding=True):
        assert groupsize in [32, 64, 128, 256]
        assert inner_k_tiles in [2, 4, 8]
        self.mod = mod
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles
        self.padding = padding

    @torch.no_grad()
    def create_quantized_state_dict(self):
        state = self.mod.state_dict()
        gpu = _gpu_device()
        for fqn, lin in self.mod.named_modules():
            if not isinstance(lin, torch.nn.Linear):
                continue
            assert not lin.bias
            k, n = lin.in_features, lin.out_features
            assert n % 8 == 0, "require out_features % 8 == 0"
            print(f"linear: {fqn}, in={k}, out={n}")
            weight = lin.weight.data
            if not _check_linear_int4_k(k, self.groupsize, self.inner_k_tiles):
                if not self.padding:
                    print(f"warning: {fqn} is skipped, int4 requires that in_features is 32, 64, or is divisible by 1024, "
                          "and that groupsize and inner_k_tiles*16 evenly divide into it")
                    continue
                print(f"warning: {fqn} is padded to satisfy in_features % 1024 == 0")
                weight = F.pad(weight, pad=(0, find_multiple(k, 1024) - k))
            packed, sz = prepare_int4_weight_and_scales_and_zeros(weight.to(torch.bfloat16).to(gpu), self.groupsize, self.inner_k_tiles)
            state[f"{fqn}.weight"] = packed.to("cpu")
            state[f"{fqn}.scales_and_zeros"] = sz.to("cpu")
        return state

    def convert_for_runtime(self):
        replace_linear_int4(self.mod, self.groupsize, self.inner_k_tiles, self.padding)
        return self.mod

    def convert_for_runtime_on_the_fly(self):
        raise NotImplementedError


class WeightOnlyInt4Linear(torch.nn.Module):
    """reference :604-666."""

    __constants__ = ["in_features", "out_features"]
    in_features: int
    out_features: int
    weight: torch.Tensor

    def __init__(self, in_features: int, out_features: int, bias=True, device=None, dtype=None,
                 groupsize: int = 128, inner_k_tiles: int = 8, padding: bool = True) -> None:
        super().__init__()
        self.padding = padding
        if padding:
            self.origin_in_features = in_features
            in_features = find_multiple(in_features, 1024)

        self.in_features = in_features
        self.out_features = out_features
        assert not bias, "require bias=False"
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles

        assert out_features % 8 == 0, "require out_features % 8 == 0"
        assert in_features % (inner_k_tiles * 16) == 0, "require in_features % (innerKTiles * 16) == 0"
        self.register_buffer(
            "weight",
            torch.empty((out_features // 8, in_features // (inner_k_tiles * 16), 32, inner_k_tiles // 2), dtype=torch.int32),
        )
        self.register_buffer(
            "scales_and_zeros", torch.empty((in_features // groupsize, out_features, 2), dtype=torch.bfloat16)
        )

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        input = input.to(torch.bfloat16)
        if self.padding:
            input = F.pad(input, pad=(0, self.in_features - self.origin_in_features))
        return linear_forward_int4(input, self.weight, self.scales_and_zeros, self.out_features, self.groupsize)


def quantize(
    checkpoint_path: Path = Path("checkpoints/meta-llama/Llama-2-7b-chat-hf/model.pth"),
    mode: str = "int8",
    groupsize: int = 128,
    label: str = "",
    model=None,
) -> Path:
    """reference :669-754 for the two weight-only modes.  Loads the bf16 state dict on the CPU, quantizes
    every nn.Linear on the GPU, and writes model{label}int8.pth / model{label}int4.g{G}.pth next to it.

    `model` may supply the module tree (the reference builds it from the directory name, :691-692); by
    default the harness Transformer is built from the checkpoint's parent directory name the same way."""
    checkpoint_path = Path(checkpoint_path)
    assert checkpoint_path.is_file(), checkpoint_path
    precision = torch.bfloat16
    print("Loading model ...")
    t0 = time.time()
    if model is None:
        from .model import Transformer

        with torch.device("meta"):
            model = Transformer.from_name(checkpoint_path.parent.name)
    checkpoint = torch.load(str(checkpoint_path), mmap=True, weights_only=True)
    model.load_state_dict(checkpoint, assign=True)
    model = model.to(dtype=precision, device="cpu")

    if mode == "int8":
        print("Quantizing model weights for int8 weight-only symmetric per-channel quantization")
        quantized_state_dict = WeightOnlyInt8QuantHandler(model).create_quantized_state_dict()
        new_base_name = checkpoint_path.name.replace(".pth", f"{label}int8.pth")
    elif mode == "int4":
        print("Quantizing model weights for int4 weight-only affine per-channel groupwise quantization")
        quantized_state_dict = WeightOnlyInt4QuantHandler(model, groupsize).create_quantized_state_dict()
        new_base_name = checkpoint_path.name.replace(".pth", f"{label}int4.g{groupsize}.pth")
    else:
        raise ValueError(f"Invalid quantization mode {mode} needs to be one of [int8, int4]")

    quantize_path = checkpoint_path.parent / new_base_name
    print(f"Writing quantized weights to {quantize_path}")
    quantize_path.unlink(missing_ok=True)
    torch.save(quantized_state_dict, quantize_path)
    print(f"Quantization complete took {time.time() - t0:.02f} seconds")
    return quantize_path


if __name__ == "__main__":
    import argparse

    parser = argparse.ArgumentParser(description="Quantize a model.")
    parser.add_argument("--checkpoint_path", type=Path, default=Path("checkpoints/meta-llama/Llama-2-7b-chat-hf/model.pth"),
                        help="Path to the model checkpoint to be quantized.")
    parser.add_argument("--mode", "-q", type=str, default="int8", choices=["int8", "int4"], help="type of quantization to perform")
    parser.add_argument("--groupsize", type=int, default=32, help="Group size for int4 quantization.")
    parser.add_argument("--label", type=str, default="_", help="label to add to output filename")
    args = parser.parse_args()
    quantize(args.checkpoint_path, args.mode, args.groupsize, args.label)

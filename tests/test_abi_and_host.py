"""CPU-side checks: the C-ABI library loads and exports every declared symbol, argument validation
returns error codes (no kernel is launched), and the host-side mirror of the reference's module /
handler interface has the reference's shapes, dtypes, keys and assertions."""

import ctypes
import re
from pathlib import Path

import pytest
import torch
import torch.nn as nn

import easy_to_hard_amd as e2h
from easy_to_hard_amd import _lib
from easy_to_hard_amd.model import ModelArgs, Transformer

ROOT = Path(__file__).resolve().parents[1]


def _declared_symbols():
    text = (ROOT / "include" / "e2h_quant.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(e2h_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 14
    for name in declared:
        assert hasattr(lib, name), name
    assert sorted(_lib.EXPORTED_SYMBOLS) == declared
    assert lib.e2h_abi_version() == 1
    assert _lib.status_string(0) == "ok"
    for code in range(-8, 0):
        assert _lib.status_string(code) != "unknown status"


def test_argument_validation_returns_codes_without_launching():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)  # never dereferenced: validation fails first
    null = ctypes.c_void_p(0)
    assert lib.e2h_int4_mm(null, p, p, p, 1, 8, 128, 128, 8, None, 0, None) == -1
    assert lib.e2h_int4_mm(p, p, p, p, 1, 8, 128, 100, 8, None, 0, None) == -3   # bad groupsize
    assert lib.e2h_int4_mm(p, p, p, p, 1, 8, 128, 128, 3, None, 0, None) == -4   # bad inner_k_tiles
    assert lib.e2h_int4_mm(p, p, p, p, 1, 12, 128, 128, 8, None, 0, None) == -2  # n % 8 != 0
    assert lib.e2h_int4_mm(p, p, p, p, 0, 8, 128, 128, 8, None, 0, None) == -2   # m < 1
    assert lib.e2h_int4_mm(p, p, p, p, 1, 8, 192, 128, 8, None, 0, None) == -3   # k % g != 0
    assert lib.e2h_int4_mm(p, p, p, p, 1, 8, 64, 32, 8, None, 0, None) == -4     # k % (16*ikt) != 0
    assert lib.e2h_int4_mm(ctypes.c_void_p(4098), p, p, p, 1, 8, 128, 128, 8, None, 0, None) == -5
    assert lib.e2h_int8_mm(p, null, p, p, 1, 8, 128, None, 0, None) == -1
    assert lib.e2h_int8_mm(p, p, p, p, 1, 0, 128, None, 0, None) == -2
    assert lib.e2h_int4_pack(p, p, 12, 128, 8, None) == -2
    assert lib.e2h_int4_pack(p, p, 8, 128, 5, None) == -4
    assert lib.e2h_int4_pack(p, p, 8, 64, 8, None) == -4
    assert lib.e2h_int4_group_qparams(p, p, p, 8, 100, 32, None) == -3
    assert lib.e2h_int4_quantize_pack(p, p, p, 8, 256, 48, 8, None) == -3
    assert lib.e2h_int8_quantize_per_channel(null, 0, p, p, p, 8, 8, None) == -1
    assert lib.e2h_set_option(b"no_such_option", 1) == -8
    assert lib.e2h_set_option(b"int4_rows_per_wave", 48) == -8
    assert lib.e2h_set_option(b"int4_rows_per_wave", 0) == 0


def test_ops_refuse_cpu_tensors():
    x = torch.zeros(1, 128, dtype=torch.bfloat16)
    packed = torch.zeros(1, 1, 32, 4, dtype=torch.int32)
    sz = torch.zeros(1, 8, 2, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="only on the GPU"):
        e2h.ops.int4_mm_direct(x, packed, 128, sz)
    with pytest.raises(RuntimeError, match="only on the GPU"):
        e2h.ops.int8_mm_direct(x, torch.zeros(8, 128, dtype=torch.int8), torch.ones(8, dtype=torch.bfloat16))


def test_custom_ops_have_fake_impls():
    # meta tensors go through the registered fake kernels: this is what torch.compile traces
    x = torch.empty(5, 256, dtype=torch.bfloat16, device="meta")
    packed = torch.empty(3, 2, 32, 4, dtype=torch.int32, device="meta")
    sz = torch.empty(2, 24, 2, dtype=torch.bfloat16, device="meta")
    y = torch.ops.e2h.int4_mm(x, packed, 128, sz)
    assert y.shape == (5, 24) and y.dtype == torch.bfloat16
    y8 = torch.ops.e2h.int8_mm(x, torch.empty(7, 256, dtype=torch.int8, device="meta"), torch.empty(7, dtype=torch.bfloat16, device="meta"))
    assert y8.shape == (5, 7)
    p = torch.ops.e2h.int4_pack(torch.empty(16, 256, dtype=torch.int32, device="meta"), 8)
    assert p.shape == (2, 2, 32, 4)


def test_int8_module_contract():
    m = e2h.WeightOnlyInt8Linear(64, 24)          # bias defaults to True and is ignored (reference :411-426)
    assert m.weight.dtype == torch.int8 and m.weight.shape == (24, 64)
    assert m.scales.dtype == torch.bfloat16 and m.scales.shape == (24,) and torch.all(m.scales == 1)
    assert set(m.state_dict()) == {"weight", "scales"}
    assert m.in_features == 64 and m.out_features == 24


def test_int4_module_contract_and_asserts():
    m = e2h.WeightOnlyInt4Linear(256, 16, bias=False, groupsize=64, inner_k_tiles=4, padding=False)
    assert m.weight.dtype == torch.int32 and m.weight.shape == (2, 4, 32, 2)
    assert m.scales_and_zeros.dtype == torch.bfloat16 and m.scales_and_zeros.shape == (4, 16, 2)
    assert set(m.state_dict()) == {"weight", "scales_and_zeros"}
    assert not hasattr(m, "origin_in_features")
    with pytest.raises(AssertionError, match="require bias=False"):
        e2h.WeightOnlyInt4Linear(256, 16)                                   # bias defaults to True (:614, :631)
    with pytest.raises(AssertionError, match="out_features % 8"):
        e2h.WeightOnlyInt4Linear(256, 12, bias=False, padding=False)
    with pytest.raises(AssertionError, match="innerKTiles"):
        e2h.WeightOnlyInt4Linear(200, 16, bias=False, padding=False)
    padded = e2h.WeightOnlyInt4Linear(200, 16, bias=False, padding=True)    # K padded to a multiple of 1024 (:623-627)
    assert padded.in_features == 1024 and padded.origin_in_features == 200
    assert padded.weight.shape == (2, 8, 32, 4) and padded.scales_and_zeros.shape == (8, 16, 2)


def test_handlers_swap_modules_like_the_reference():
    cfg = ModelArgs(block_size=64, vocab_size=64, n_layer=2, n_head=2, dim=128, intermediate_size=256)
    with torch.device("meta"):
        model = Transformer(cfg)
    keys_before = set(model.state_dict())
    h4 = e2h.WeightOnlyInt4QuantHandler(model, groupsize=32, inner_k_tiles=2)
    h4.convert_for_runtime()
    linears = ["layers.0.attention.wqkv", "layers.0.attention.wo", "layers.0.feed_forward.w1",
               "layers.0.feed_forward.w3", "layers.0.feed_forward.w2", "output"]
    mods = dict(model.named_modules())
    for fqn in linears:
        assert isinstance(mods[fqn], e2h.WeightOnlyInt4Linear), fqn
        assert mods[fqn].groupsize == 32 and mods[fqn].inner_k_tiles == 2 and mods[fqn].padding is False
    keys_after = set(model.state_dict())
    assert {k for k in keys_after if k.endswith("scales_and_zeros")} == {f + ".scales_and_zeros" for f in mods if isinstance(mods[f], e2h.WeightOnlyInt4Linear)}
    assert keys_before <= {k.replace(".scales_and_zeros", ".weight") for k in keys_after}
    with pytest.raises(NotImplementedError):
        h4.convert_for_runtime_on_the_fly()
    with pytest.raises(AssertionError):
        e2h.WeightOnlyInt4QuantHandler(model, groupsize=48)
    with pytest.raises(AssertionError):
        e2h.WeightOnlyInt4QuantHandler(model, inner_k_tiles=16)

    with torch.device("meta"):
        model8 = Transformer(cfg)
    e2h.WeightOnlyInt8QuantHandler(model8).convert_for_runtime()
    for fqn, mod in model8.named_modules():
        assert not isinstance(mod, nn.Linear), fqn
    assert isinstance(model8.output, e2h.WeightOnlyInt8Linear)
    assert "layers.1.feed_forward.w2.scales" in model8.state_dict()


def test_int4_swap_padding_rules():
    class Odd(nn.Module):
        def __init__(self):
            super().__init__()
            self.a = nn.Linear(200, 16, bias=False)
            self.b = nn.Linear(256, 16, bias=False)

    m = Odd()
    e2h.replace_linear_int4(m, 128, 8, padding=False)
    assert isinstance(m.a, nn.Linear) and isinstance(m.b, e2h.WeightOnlyInt4Linear)   # skipped (:476 not taken)
    m = Odd()
    e2h.replace_linear_int4(m, 128, 8, padding=True)
    assert m.a.padding is True and m.a.in_features == 1024 and m.b.padding is False


def test_small_helpers():
    assert e2h.find_multiple(11008, 1024) == 11264 and e2h.find_multiple(4096, 1024) == 4096
    assert e2h._check_linear_int4_k(4096, 128, 8) and not e2h._check_linear_int4_k(4000, 128, 8)
    s = torch.arange(6, dtype=torch.float32).reshape(2, 3).to(torch.bfloat16)
    z = -s
    sz = e2h.pack_scales_and_zeros(s, z)
    assert sz.shape == (3, 2, 2) and sz.is_contiguous()
    assert sz[2, 1, 0] == s[1, 2] and sz[2, 1, 1] == z[1, 2]
    s2, z2 = e2h.unpack_scales_and_zeros(sz)
    assert torch.equal(s2.squeeze(-1), s) and torch.equal(z2.squeeze(-1), z)
    with pytest.raises(AssertionError):
        e2h.pack_scales_and_zeros(s.float(), z.float())
    with pytest.raises(NotImplementedError):
        e2h.dynamically_quantize_per_channel(torch.zeros(2, 2), 0, 255, torch.uint8)


def test_model_shapes_match_reference_configs():
    a = ModelArgs.from_name("7B")
    assert (a.n_layer, a.dim, a.n_head, a.n_local_heads, a.head_dim, a.intermediate_size, a.vocab_size) == (32, 4096, 32, 32, 128, 11008, 32000)
    b = ModelArgs.from_name("CodeLlama-34B-Python-hf")
    assert (b.n_layer, b.dim, b.n_head, b.n_local_heads, b.head_dim, b.intermediate_size, b.rope_base) == (48, 8192, 64, 8, 128, 22016, 1000000)
    with torch.device("meta"):
        t = Transformer(b)
    assert t.layers[0].attention.wqkv.weight.shape == (10240, 8192)
    assert ModelArgs.from_name("llemma-7b").block_size == 4096


def test_fused_and_sampling_entry_points_validate_arguments():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)  # never dereferenced: validation fails first
    null = ctypes.c_void_p(0)
    # gated launch: at most 64 rows, inner_k_tiles 8 only, group size 32 / 64 / 128
    assert lib.e2h_int4_mm_silu_gate(p, p, p, p, p, p, 65, 64, 128, 128, 8, None) == -2
    assert lib.e2h_int4_mm_silu_gate(p, p, p, p, p, p, 32, 64, 128, 128, 4, None) == -4
    assert lib.e2h_int4_mm_silu_gate(p, p, p, p, p, p, 32, 64, 256, 256, 8, None) == -3
    assert lib.e2h_int4_mm_silu_gate(p, null, p, p, p, p, 32, 64, 128, 128, 8, None) == -1
    # projection + RoPE + cache write: odd head_dim, too many sequences, K not in whole chunks
    assert lib.e2h_int4_mm_rope_kv(p, p, p, p, p, p, p, p, 4, 2, 2, 63, 16, 128, 128, 8, None) == -2
    assert lib.e2h_int4_mm_rope_kv(p, p, p, p, p, p, p, p, 65, 2, 2, 64, 16, 128, 128, 8, None) == -2
    assert lib.e2h_int4_mm_rope_kv(p, p, p, p, p, p, p, p, 4, 2, 2, 64, 16, 192, 64, 8, None) == -4
    assert lib.e2h_rope_kv_write_seq(p, p, p, p, p, p, 2, 0, 2, 2, 16, 64, 0, None) == -2
    assert lib.e2h_rope_kv_write_seq(p, p, p, p, p, null, 2, 3, 2, 2, 16, 64, 0, None) == -1
    # sampling: row stride shorter than the vocabulary, negative top_k, misaligned q
    assert lib.e2h_sample_top_k(p, 10, p, p, p, 2, 16, 1.0, 0, None) == -2
    assert lib.e2h_sample_top_k(p, 16, p, p, p, 2, 16, 1.0, -1, None) == -2
    assert lib.e2h_sample_top_k(p, 16, ctypes.c_void_p(4098), p, p, 2, 16, 1.0, 0, None) == -5
    # int8 fused launches: too many rows, K not in whole chunks, null pointer
    assert lib.e2h_int8_mm_silu_gate(p, p, p, p, p, p, 65, 64, 128, None) == -2
    assert lib.e2h_int8_mm_silu_gate(p, p, p, p, p, p, 32, 64, 192, None) == -2
    assert lib.e2h_int8_mm_silu_gate(p, null, p, p, p, p, 32, 64, 128, None) == -1
    assert lib.e2h_int8_mm_rope_kv(p, p, p, p, p, p, p, p, 4, 2, 2, 63, 16, 128, None) == -2
    assert lib.e2h_int8_mm_rope_kv(p, p, p, p, p, p, p, null, 4, 2, 2, 64, 16, 128, None) == -1
    assert lib.e2h_argmax_rows(p, 10, p, 2, 16, None) == -2
    assert lib.e2h_argmax_rows(p, 16, null, 2, 16, None) == -1
    assert lib.e2h_argmax_rows(p, 16, ctypes.c_void_p(4100), 2, 16, None) == -5
    for name in (b"row_tiles", b"int4_no_xsum", b"int4_no_gemm32", b"int4_gemm32_min_rows"):
        assert lib.e2h_set_option(name, 0) == 0
    assert lib.e2h_set_option(b"row_tiles", 3) == -8


def test_sampling_host_path_on_cpu_tensors():
    """generate.sample falls back to the reference's op chain for inputs the kernel does not take (CPU, float32)."""
    import torch

    from easy_to_hard_amd.generate import logits_to_probs, multinomial_sample_one_no_sync, sample

    torch.manual_seed(0)
    logits = torch.randn(3, 2, 50)
    probs = logits_to_probs(logits[:, -1], temperature=0.7, top_k=5)
    assert probs.shape == (3, 50) and torch.allclose(probs.sum(-1), torch.ones(3))
    assert torch.all((probs > 0).sum(-1) == 5)
    idx = multinomial_sample_one_no_sync(probs)
    assert idx.shape == (3, 1) and idx.dtype == torch.int and torch.all(probs.gather(1, idx.long()) > 0)
    idx2, probs2 = sample(logits, temperature=0.7, top_k=5)
    assert torch.allclose(probs2, probs) and idx2.shape == (3, 1)
    # temperature -> 0 is clamped at 1e-5 and degenerates to arg-max
    idx3, _ = sample(logits, temperature=0.0, top_k=None)
    assert torch.equal(idx3[:, 0].long(), logits[:, -1].argmax(-1))


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2 and "one GPU" in proc.stderr


def test_bench_spreads_the_timed_positions_over_the_whole_decode():
    import bench

    pos = bench.spread_positions(256, 512, 20)
    assert len(pos) == 20 and pos[0] == 256 and pos[-1] == 767 and pos == sorted(pos)
    assert abs(sum(pos) / len(pos) - (256 + 767) / 2) < 1.0          # the sample's mean position is the decode's
    assert bench.spread_positions(256, 512, 511 + 1)[:3] == [256, 257, 258]
    assert bench.spread_positions(10, 5, 1) == [12] and bench.spread_positions(10, 5, 2) == [10, 14]
    threads, physical = bench._cpu_threads()
    assert threads >= 1 and physical >= 1


def test_loader_reads_mode_and_group_size_off_the_file_name(tmp_path):
    """load_model (the reference's _load_model, inference_generate.py:224-259): a plain bf16 checkpoint loads on the CPU;
    names it cannot interpret and missing files are refused before anything touches a GPU."""
    import torch

    from easy_to_hard_amd.generate import load_model
    from easy_to_hard_amd.model import Transformer, init_random_

    ckpt_dir = tmp_path / "tiny-test"
    ckpt_dir.mkdir()
    model = Transformer.from_name("tiny-test")
    init_random_(model, seed=3, std=0.05)
    torch.save(model.state_dict(), ckpt_dir / "model.pth")
    loaded = load_model(ckpt_dir / "model.pth", "cpu", torch.bfloat16)
    assert not loaded.training and loaded.output.weight.dtype == torch.bfloat16
    assert torch.equal(loaded.output.weight, model.output.weight.to(torch.bfloat16))
    assert torch.equal(loaded.layers[1].attention.wqkv.weight, model.layers[1].attention.wqkv.weight.to(torch.bfloat16))
    (ckpt_dir / "model_int4.pth").write_bytes(b"x")                     # "int4" but no .g{G}. component
    with pytest.raises(ValueError):
        load_model(ckpt_dir / "model_int4.pth", "cpu")
    with pytest.raises(FileNotFoundError):
        load_model(ckpt_dir / "absent_int8.pth", "cpu")
    with pytest.raises(NotImplementedError):
        load_model(ckpt_dir / "model.pth", "cpu", use_tp=True)


def test_reward_model_loader_builds_the_two_row_head_and_rejects_quantized_files(tmp_path):
    """load_reward_model follows the reference's _load_reward_model (inference_reward.py:94-118): a bfloat16
    language-model checkpoint goes into the backbone, `output` becomes a zero two-row head, quantized file names are
    refused; apply_reward_modeling_head covers the three initialisations of models/reward_model.py:95-133."""
    from easy_to_hard_amd.generate import load_reward_model
    from easy_to_hard_amd.model import RewardModel, apply_reward_modeling_head, init_random_

    ckpt_dir = tmp_path / "tiny-test"
    ckpt_dir.mkdir()
    lm = Transformer.from_name("tiny-test")
    init_random_(lm, seed=3, std=0.05)
    torch.save(lm.state_dict(), ckpt_dir / "model.pth")
    rm = load_reward_model(ckpt_dir / "model.pth", "cpu", torch.bfloat16)
    assert isinstance(rm, RewardModel) and rm.backbone_model is rm.backbone and not rm.training
    head = rm.backbone.output
    assert tuple(head.weight.shape) == (2, lm.config.dim) and head.out_features == 2
    assert head.weight.dtype == torch.bfloat16 and not head.weight.requires_grad and int(head.weight.count_nonzero()) == 0
    assert torch.equal(rm.backbone.layers[1].feed_forward.w2.weight, lm.layers[1].feed_forward.w2.weight)
    for bad in ("model_int8.pth", "model_int4.g128.pth"):
        (ckpt_dir / bad).write_bytes(b"")
        with pytest.raises(NotImplementedError):
            load_reward_model(ckpt_dir / bad, "cpu")
    with pytest.raises(FileNotFoundError):
        load_reward_model(ckpt_dir / "absent.pth", "cpu")
    with pytest.raises(NotImplementedError):
        load_reward_model(ckpt_dir / "model.pth", "cpu", use_tp=True)

    big = nn.Module()
    big.output = nn.Linear(8, 30000, bias=False)
    w = big.output.weight.detach().clone()
    apply_reward_modeling_head(big, init_scheme="semantic")
    assert torch.equal(big.output.weight[0], w[29906]) and torch.equal(big.output.weight[1], -w[29896])
    apply_reward_modeling_head(big, init_scheme="random")
    first = big.output.weight.detach().clone()
    apply_reward_modeling_head(big, init_scheme="random")
    assert tuple(first.shape) == (2, 8) and torch.equal(first, big.output.weight) and float(first.abs().max()) > 0
    with pytest.raises(ValueError):
        apply_reward_modeling_head(big, init_scheme="other")

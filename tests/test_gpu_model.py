"""End-to-end GPU checks on a tiny Llama-shaped model: quantize -> save -> load -> run, greedy decoding
against an oracle model whose linears are the dequantized weights applied with F.linear, and HIP-graph
replays against eager execution."""

import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

import easy_to_hard_amd as e2h
from easy_to_hard_amd.generate import GraphedDecodeStep, decode_one_token, generate, load_model, model_score, prefill
from easy_to_hard_amd.model import ModelArgs, RewardModel, Transformer, init_random_
from oracle import quant_oracle as qo
from tests.helpers import bf16_to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class OracleLinear(nn.Module):
    """x @ W^T in float32 with W = (q - 8) * scale + zero resp. q * scale (dequantize-then-F.linear)."""

    def __init__(self, w_f32):
        super().__init__()
        self.register_buffer("w", w_f32)

    def forward(self, x):
        return torch.nn.functional.linear(x.float(), self.w).to(torch.bfloat16)


def _oracle_copy(model_q, mode, g):
    """Clone of the quantized model with every quantized linear replaced by its float32 oracle."""
    oracle = copy.deepcopy(model_q)
    for name, mod in list(oracle.named_modules()):
        for child_name, child in list(mod.named_children()):
            if isinstance(child, e2h.WeightOnlyInt4Linear):
                codes = qo.int4_tile_unpack(child.weight.cpu().numpy(), child.inner_k_tiles)
                w = qo.int4_dequantize_fp32(codes, bf16_to_np(child.scales_and_zeros), g)
                setattr(mod, child_name, OracleLinear(torch.from_numpy(w).to(DEV)))
            elif isinstance(child, e2h.WeightOnlyInt8Linear):
                w = child.weight.cpu().float() * child.scales.cpu().float()[:, None]
                setattr(mod, child_name, OracleLinear(w.to(DEV)))
    return oracle


def _tiny(name="tiny-test"):
    model = Transformer.from_name(name)
    init_random_(model, seed=1234, std=0.05)
    return model


@pytest.mark.parametrize("name,g", [("tiny-test", 128), ("tiny-gqa-test", 64)])
def test_int4_checkpoint_roundtrip_and_greedy_decode(tmp_path, name, g):
    model = _tiny(name)
    torch.save(model.state_dict(), tmp_path / "model.pth")
    handler = e2h.WeightOnlyInt4QuantHandler(model, groupsize=g)
    sd = handler.create_quantized_state_dict()
    path = tmp_path / f"model_int4.g{g}.pth"
    torch.save(sd, path)
    assert sd["layers.0.attention.wqkv.weight"].dtype == torch.int32
    assert sd["output.scales_and_zeros"].shape == (model.config.dim // g, model.config.vocab_size, 2)

    # runtime path of the reference loader (inference_generate.py:224-259)
    rt = load_model(path, DEV, torch.bfloat16, model_name=name)
    assert rt.output.weight.dtype == torch.int32 and rt.output.weight.is_cuda

    oracle = _oracle_copy(rt, "int4", g)
    bsz, t, new = 4, 12, 10
    prompt = torch.randint(0, model.config.vocab_size, (bsz, t), generator=torch.Generator().manual_seed(1234)).to(DEV)
    seq_eager = generate(rt, prompt, new, use_graph=False)
    seq_graph = generate(rt, prompt, new, use_graph=True)
    assert torch.equal(seq_eager, seq_graph), "HIP-graph replays must reproduce eager decoding"

    # teacher-forced comparison with the oracle model: same prefix -> logits agree, argmax agrees wherever
    # the oracle's top-1/top-2 margin exceeds the bf16 noise of the logits
    oracle.setup_caches(bsz, t + new)
    rt.setup_caches(bsz, t + new)
    agree = total = 0
    for step in range(new):
        prefix = seq_eager[:, : t + step]
        pos = torch.arange(0, prefix.shape[1], device=DEV)
        lq = rt(prefix, pos)[:, -1].float()
        lo = oracle(prefix, pos)[:, -1].float()
        err = (lq - lo).abs().max() / lo.abs().max()
        assert err <= 2e-2, err
        top2 = lo.topk(2, dim=-1).values
        margin_ok = (top2[:, 0] - top2[:, 1]) > 4 * (lq - lo).abs().max()
        agree += int(((lq.argmax(-1) == lo.argmax(-1)) & margin_ok).sum())
        total += int(margin_ok.sum())
        assert torch.equal(lq.argmax(-1)[margin_ok], lo.argmax(-1)[margin_ok])
    assert total > 0 and agree == total


def test_int8_on_the_fly_reward_scoring():
    cfg = ModelArgs.from_name("tiny-test")
    rm = RewardModel(cfg, head_rows=2)
    init_random_(rm, seed=7, std=0.05)
    rm = rm.to(device=DEV, dtype=torch.bfloat16).eval()
    e2h.WeightOnlyInt8QuantHandler(rm).convert_for_runtime_on_the_fly()
    assert isinstance(rm.backbone.output, e2h.WeightOnlyInt8Linear) and rm.backbone.output.out_features == 2
    oracle = _oracle_copy(rm, "int8", None)
    ids = torch.randint(0, cfg.vocab_size, (3, 40), generator=torch.Generator().manual_seed(1)).to(DEV)
    r = model_score(rm, ids)
    r_ref = model_score(oracle, ids)
    assert r.shape == (3, 40)
    assert qo.normwise_rel_err(r.float().cpu().numpy(), r_ref.float().cpu().numpy()) <= 2e-2


def test_graph_replays_match_eager_every_time():
    model = _tiny()
    e2h.WeightOnlyInt4QuantHandler(model, groupsize=32).convert_for_runtime
    sd = e2h.WeightOnlyInt4QuantHandler(model, groupsize=32).create_quantized_state_dict()
    e2h.WeightOnlyInt4QuantHandler(model, groupsize=32).convert_for_runtime()
    model.load_state_dict(sd, assign=True)
    model = model.to(device=DEV, dtype=torch.bfloat16).eval()
    bsz = 2
    model.setup_caches(bsz, 32)
    prompt = torch.randint(0, 512, (bsz, 8), generator=torch.Generator().manual_seed(3)).to(DEV)
    cur = prefill(model, prompt, torch.arange(0, 8, device=DEV))
    stepper = GraphedDecodeStep(model, bsz, DEV)
    prefill(model, prompt, torch.arange(0, 8, device=DEV))  # restore the cache rows the capture warm-up touched
    for i in range(6):
        pos = torch.tensor([8 + i], device=DEV)
        eager = decode_one_token(model, cur, pos)
        torch.cuda.synchronize()
        replay = stepper.step(cur, pos).clone()
        torch.cuda.synchronize()
        assert torch.equal(eager, replay), i
        cur = eager


@pytest.mark.parametrize("mode,g,label,expect", [("int8", 128, "", "modelint8.pth"), ("int4", 64, "_x_", "model_x_int4.g64.pth")])
def test_quantize_writer_names_keys_and_reload(tmp_path, mode, g, label, expect):
    """quantize() (reference models/quantize.py:669-754): output file name convention (:707, :718), state-dict keys
    and dtypes of the two weight-only modes, and that the file loads into a converted model."""
    ckpt_dir = tmp_path / "tiny-test"
    ckpt_dir.mkdir()
    model = _tiny()
    torch.save(model.to(torch.bfloat16).state_dict(), ckpt_dir / "model.pth")
    out = e2h.quantize(ckpt_dir / "model.pth", mode, g, label)
    assert out == ckpt_dir / expect and out.is_file()
    sd = torch.load(out, weights_only=True)
    lin = "layers.0.attention.wqkv"
    with torch.device("meta"):
        rt = Transformer.from_name("tiny-test")
    n, k = model.layers[0].attention.wqkv.weight.shape
    if mode == "int8":
        assert sd[lin + ".weight"].dtype == torch.int8 and sd[lin + ".scales"].dtype == torch.bfloat16
        assert tuple(sd[lin + ".weight"].shape) == (n, k) and tuple(sd[lin + ".scales"].shape) == (n,)
        e2h.WeightOnlyInt8QuantHandler(rt).convert_for_runtime()
    else:
        assert sd[lin + ".weight"].dtype == torch.int32 and tuple(sd[lin + ".weight"].shape) == (n // 8, k // 128, 32, 4)
        assert sd[lin + ".scales_and_zeros"].dtype == torch.bfloat16 and tuple(sd[lin + ".scales_and_zeros"].shape) == (k // g, n, 2)
        e2h.WeightOnlyInt4QuantHandler(rt, g).convert_for_runtime()
    assert sd["tok_embeddings.weight"].dtype == torch.bfloat16  # non-linear entries pass through untouched
    rt.load_state_dict(sd, assign=True)
    rt = rt.to(device=DEV, dtype=torch.bfloat16).eval()
    rt.setup_caches(2, 7)
    ids = torch.randint(0, 512, (2, 7), generator=torch.Generator().manual_seed(3)).to(DEV)
    with torch.no_grad():
        logits = rt(ids, torch.arange(7, device=DEV))
    assert logits.shape == (2, 7, 512) and torch.isfinite(logits.float()).all()


@pytest.mark.parametrize("name", ["tiny-test", "tiny-gqa-test"])
def test_int8_fused_decode_step_equals_unfused_calls_and_graph_replay(name):
    """int8 model: the gated and the RoPE-projection launches form each linear's output with the reference's two roundings
    before their epilogue, so switching them off (separate linears + silu_mul + rope_kv_write) changes no bit of the
    logits; the HIP-graph replay reproduces eager decoding."""
    import easy_to_hard_amd.model as model_mod

    model = _tiny(name).to(device=DEV, dtype=torch.bfloat16).eval()
    e2h.WeightOnlyInt8QuantHandler(model).convert_for_runtime_on_the_fly()
    bsz, t = 3, 9
    model.setup_caches(bsz, 32)
    prompt = torch.randint(0, model.config.vocab_size, (bsz, t), generator=torch.Generator().manual_seed(5)).to(DEV)
    pos = torch.arange(0, t, device=DEV)
    cur = prefill(model, prompt, pos)
    step_pos = torch.tensor([t], device=DEV)
    logits_fused = model(cur, step_pos).clone()
    model_mod.FUSE_GATE = model_mod.FUSE_ROPE_PROJECTION = False
    try:
        prefill(model, prompt, pos)
        logits_plain = model(cur, step_pos).clone()
    finally:
        model_mod.FUSE_GATE = model_mod.FUSE_ROPE_PROJECTION = True
    assert torch.equal(logits_fused, logits_plain)
    seq_eager = generate(model, prompt, 6, use_graph=False)
    seq_graph = generate(model, prompt, 6, use_graph=True)
    assert torch.equal(seq_eager, seq_graph)

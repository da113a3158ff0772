"""GPU checks of the drop-in boundary: tracing under torch.compile(fullgraph=True) (the way the reference calls the
modules in decode, inference_generate.py:346-349), the reference's int32 position tensor, per-stream split-K scratch,
and the checkpoint writer -> file -> loader round trip (models/quantize.py:669-754, inference_generate.py:224-259)."""

import pytest
import torch

import easy_to_hard_amd as e2h
from easy_to_hard_amd import ops
from easy_to_hard_amd.generate import GraphedDecodeStep, decode_one_token, generate, load_model, load_reward_model, model_score, prefill
from easy_to_hard_amd.model import Transformer, init_random_
from tests.helpers import randn_bf16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tiny_int4(name="tiny-test", g=32):
    model = Transformer.from_name(name)
    init_random_(model, seed=1234, std=0.05)
    sd = e2h.WeightOnlyInt4QuantHandler(model, groupsize=g).create_quantized_state_dict()
    e2h.WeightOnlyInt4QuantHandler(model, groupsize=g).convert_for_runtime()
    model.load_state_dict(sd, assign=True)
    return model.to(device=DEV, dtype=torch.bfloat16).eval()


def test_quantized_modules_trace_under_fullgraph_compile_and_match_eager():
    """backend "aot_eager" traces with fake tensors through the registered e2h::int4_mm / e2h::int8_mm ops and then runs
    the traced graph with the real kernels; fullgraph=True fails on any graph break."""
    lin4 = e2h.WeightOnlyInt4Linear(512, 48, bias=False, groupsize=64, inner_k_tiles=8, padding=False).to(DEV)
    w = randn_bf16((48, 512), std=0.02, seed=1).to(DEV)
    lin4.weight, lin4.scales_and_zeros = e2h.prepare_int4_weight_and_scales_and_zeros(w, 64, 8)
    lin8 = e2h.WeightOnlyInt8Linear(512, 48).to(DEV)
    q, scales, _ = e2h.dynamically_quantize_per_channel(w.float(), -128, 127, torch.int8)
    lin8.load_state_dict({"weight": q, "scales": scales})
    x = randn_bf16((3, 5, 512), seed=2).to(DEV)
    for lin in (lin4, lin8):
        compiled = torch.compile(lin, backend="aot_eager", fullgraph=True)
        with torch.no_grad():
            assert torch.equal(compiled(x), lin(x))
            assert torch.equal(compiled(x[:1, :1]), lin(x[:1, :1]))   # another shape retraces


def _compiled_step_equals_graphed_step(model, bsz, t):
    """The reference decodes through torch.compile(mode="reduce-overhead", fullgraph=True) (inference_generate.py:346-349).
    Here: the model under torch.compile(backend="aot_eager", fullgraph=True) -- a trace with fake tensors through the
    registered e2h:: ops, any graph break is an error -- must run the very kernels of the HIP-graph replayed step: same
    logits as the eager step and the same next token as GraphedDecodeStep, bit for bit."""
    model.setup_caches(bsz, 32)
    prompt = torch.randint(0, model.config.vocab_size, (bsz, t), generator=torch.Generator().manual_seed(5)).to(DEV)
    pos = torch.arange(0, t, device=DEV)
    step_pos = torch.tensor([t], device=DEV)
    with torch.no_grad():
        cur = prefill(model, prompt, pos)
        eager = model(cur, step_pos).clone()
        prefill(model, prompt, pos)
        compiled = torch.compile(model, backend="aot_eager", fullgraph=True)
        traced = compiled(cur, step_pos).clone()
        assert torch.equal(traced, eager)
        stepper = GraphedDecodeStep(model, bsz, DEV)
        prefill(model, prompt, pos)
        replay = stepper.step(cur, step_pos).clone()
        assert torch.equal(replay, torch.argmax(traced[:, -1].float(), dim=-1, keepdim=True))
        # a second traced step (the first one's token, next position) against the eager one, caches included
        nxt_pos = torch.tensor([t + 1], device=DEV)
        prefill(model, prompt, pos)
        model(cur, step_pos)
        want = model(replay, nxt_pos).clone()
        prefill(model, prompt, pos)
        compiled(cur, step_pos)
        assert torch.equal(compiled(replay, nxt_pos), want)


@pytest.mark.parametrize("name", ["tiny-test", "tiny-gqa-test"])
def test_fused_decode_step_under_fullgraph_compile_equals_the_graphed_step(name):
    _compiled_step_equals_graphed_step(_tiny_int4(name), 3, 9)


@pytest.mark.parametrize("mode", ["int4", "int8"])
def test_7b_shaped_decode_step_under_fullgraph_compile_equals_the_graphed_step(mode):
    """Two layers of the 7B shape at 32 rows: the int4 model takes the staged decode-batch kernels (asserted), the int8
    model the row-major fused kernels, traced exactly as they run eagerly."""
    from easy_to_hard_amd.model import ModelArgs, random_quantized_transformer

    cfg = ModelArgs.from_name("7B")
    cfg.n_layer = 2
    model = random_quantized_transformer(cfg, mode, 128, device=DEV, seed=7)
    model.setup_caches(32, 32)
    assert model.staged_step_supported(32) == (mode == "int4")
    _compiled_step_equals_graphed_step(model, 32, 7)


@pytest.mark.parametrize("name", ["tiny-test", "tiny-gqa-test"])
def test_int32_position_tensor_as_the_reference_passes_it(name):
    """The reference decodes with torch.tensor([T], dtype=torch.int) (inference_generate.py:205)."""
    model = _tiny_int4(name, g=64)
    bsz, t = 2, 8
    model.setup_caches(bsz, 32)
    prompt = torch.randint(0, model.config.vocab_size, (bsz, t), generator=torch.Generator().manual_seed(3)).to(DEV)
    pos = torch.arange(0, t, device=DEV)
    cur = prefill(model, prompt, pos)
    want = decode_one_token(model, cur, torch.tensor([t], device=DEV, dtype=torch.int64))
    prefill(model, prompt, pos)
    got = decode_one_token(model, cur, torch.tensor([t], device=DEV, dtype=torch.int))
    assert torch.equal(got, want)
    stepper = GraphedDecodeStep(model, bsz, DEV)
    prefill(model, prompt, pos)
    replay = stepper.step(cur, torch.tensor([t], device=DEV, dtype=torch.int)).clone()
    assert torch.equal(replay, want)


def test_two_streams_use_separate_split_k_scratch():
    """Shapes that split K over workgroups (4096 x 4096 at 32 rows) issued concurrently on two streams: each stream has its
    own tickets and partial tiles, and every result equals the single-stream one bit for bit."""
    n, k, g = 4096, 4096, 128
    w = randn_bf16((n, k), std=0.02, seed=9).to(DEV)
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(w, g, 8)
    q8, s8, _ = e2h.dynamically_quantize_per_channel(w.float(), -128, 127, torch.int8)
    s8 = s8.to(torch.bfloat16)
    xs = [randn_bf16((32, k), seed=20 + i).to(DEV) for i in range(2)]
    want4 = [ops.int4_mm_direct(x, packed, g, sz) for x in xs]
    want8 = [ops.int8_mm_direct(x, q8, s8) for x in xs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=DEV) for _ in range(2)]
    got4, got8 = [[], []], [[], []]
    for _ in range(40):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                got4[i].append(ops.int4_mm_direct(xs[i], packed, g, sz))
                got8[i].append(ops.int8_mm_direct(xs[i], q8, s8))
    torch.cuda.synchronize()
    for i in range(2):
        assert all(torch.equal(y, want4[i]) for y in got4[i])
        assert all(torch.equal(y, want8[i]) for y in got8[i])
    keys = [key for key in ops._workspaces if key[0] == 0]
    assert len({ops._workspaces[key].data_ptr() for key in keys}) >= 3   # default stream + the two side streams


@pytest.mark.parametrize("mode,g", [("int4", 64), ("int8", 128)])
def test_writer_file_loader_round_trip(tmp_path, mode, g):
    """quantize() writes model{label}int4.g{G}.pth / model{label}int8.pth next to model.pth; load_model() reads the mode and
    the group size off that name, builds the module tree from the directory name, and the loaded model decodes exactly
    like one converted in memory."""
    ckpt_dir = tmp_path / "tiny-gqa-test"
    ckpt_dir.mkdir()
    model = Transformer.from_name("tiny-gqa-test")
    init_random_(model, seed=1234, std=0.05)
    torch.save(model.state_dict(), ckpt_dir / "model.pth")
    out = e2h.quantize(ckpt_dir / "model.pth", mode, g, "_")
    assert out.name == ("model_int4.g64.pth" if mode == "int4" else "model_int8.pth")
    loaded = load_model(out, DEV, torch.bfloat16, use_tp=False)
    lin = loaded.layers[0].attention.wqkv
    if mode == "int4":
        assert isinstance(lin, e2h.WeightOnlyInt4Linear) and lin.groupsize == g and lin.weight.dtype == torch.int32 and lin.weight.is_cuda
        handler = e2h.WeightOnlyInt4QuantHandler(model, groupsize=g)
    else:
        assert isinstance(lin, e2h.WeightOnlyInt8Linear) and lin.weight.dtype == torch.int8 and lin.scales.dtype == torch.bfloat16
        handler = e2h.WeightOnlyInt8QuantHandler(model)
    assert loaded.tok_embeddings.weight.dtype == torch.bfloat16 and not loaded.training
    sd = handler.create_quantized_state_dict()
    handler.convert_for_runtime()
    model.load_state_dict(sd, assign=True)
    model = model.to(device=DEV, dtype=torch.bfloat16).eval()
    prompt = torch.randint(0, model.config.vocab_size, (2, 6), generator=torch.Generator().manual_seed(8)).to(DEV)
    assert torch.equal(generate(loaded, prompt, 5, use_graph=False), generate(model, prompt, 5, use_graph=False))


def test_loader_rejects_what_it_cannot_interpret(tmp_path):
    ckpt_dir = tmp_path / "tiny-test"
    ckpt_dir.mkdir()
    model = Transformer.from_name("tiny-test")
    init_random_(model, seed=1, std=0.05)
    torch.save(model.state_dict(), ckpt_dir / "model.pth")
    out = e2h.quantize(ckpt_dir / "model.pth", "int4", 64, "")
    bad = ckpt_dir / "modelint4.pth"          # no .g{G}. component
    out.rename(bad)
    with pytest.raises(ValueError):
        load_model(bad, DEV)
    wrong = ckpt_dir / "modelint4.g128.pth"   # group size in the name differs from the tensors' shapes
    bad.rename(wrong)
    with pytest.raises(ValueError):
        load_model(wrong, DEV)
    with pytest.raises(FileNotFoundError):
        load_model(ckpt_dir / "missing_int8.pth", DEV)
    with pytest.raises(NotImplementedError):
        load_model(wrong, DEV, use_tp=True)


def test_reward_model_loader_with_on_the_fly_int8(tmp_path):
    """load_reward_model(..., on_the_fly_8bit_quantization=True) = the reference's _load_reward_model followed by the
    quantization step of its main (inference_reward.py:94-118, :171-178): every linear, the two-row head included, becomes
    a WeightOnlyInt8Linear on the GPU; scores stay within the weights' int8 quantization error (about 1 / 127.5 of each row's
    largest weight per weight, through two layers) of the unquantized bfloat16 model's -- arithmetic parity of the int8
    scoring pass against its oracle twin is tests/test_gpu_model.py::test_int8_on_the_fly_reward_scoring."""
    ckpt_dir = tmp_path / "tiny-test"
    ckpt_dir.mkdir()
    lm = Transformer.from_name("tiny-test")
    init_random_(lm, seed=11, std=0.05)
    torch.save(lm.state_dict(), ckpt_dir / "model.pth")
    plain = load_reward_model(ckpt_dir / "model.pth", DEV, torch.bfloat16)
    head = randn_bf16((2, lm.config.dim), std=0.05, seed=12).to(DEV)
    plain.backbone.output.weight.data.copy_(head)
    quant = load_reward_model(ckpt_dir / "model.pth", DEV, torch.bfloat16)
    quant.backbone.output.weight.data.copy_(head)
    quant = e2h.WeightOnlyInt8QuantHandler(quant).convert_for_runtime_on_the_fly().eval()
    direct = load_reward_model(ckpt_dir / "model.pth", DEV, torch.bfloat16, on_the_fly_8bit_quantization=True)
    for mod in (quant, direct):
        assert isinstance(mod.backbone.output, e2h.WeightOnlyInt8Linear) and mod.backbone.output.out_features == 2
        assert isinstance(mod.backbone.layers[0].attention.wqkv, e2h.WeightOnlyInt8Linear)
        assert mod.backbone.layers[0].attention.wqkv.weight.is_cuda
    ids = torch.randint(0, lm.config.vocab_size, (3, 24), generator=torch.Generator().manual_seed(2)).to(DEV)
    assert int(model_score(direct, ids).count_nonzero()) == 0          # zero head, as loaded
    want, got = model_score(plain, ids).float(), model_score(quant, ids).float()
    assert got.shape == (3, 24)
    assert float((got - want).abs().max()) <= 1e-1 * float(want.abs().max())
    assert torch.equal(model_score(direct, ids), torch.zeros_like(got, dtype=torch.bfloat16))


@pytest.mark.parametrize("m,n,k,g", [(32, 4096, 4096, 128), (1, 4096, 4096, 128), (5, 4096, 11008, 128), (33, 1024, 2048, 64), (64, 8192, 8192, 64),
                                      (17, 264, 1024, 32), (32, 12288, 4096, 128)])
def test_partial_sums_handed_to_the_norm_equal_the_combined_matmul(m, n, k, g):
    """e2h_int4_mm_partials + e2h_add_rmsnorm_partials against e2h_int4_mm + e2h_add_rmsnorm on the same operands: the
    slices are added in slice order in both forms, so the residual stream and the normed output are equal bit for bit;
    the partial sums themselves add up (in float32, in order) to a value that rounds to the matmul's output."""
    w = randn_bf16((n, k), std=0.02, seed=n + k).to(DEV)
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(w, g, 8)
    lin = e2h.WeightOnlyInt4Linear(k, n, bias=False, groupsize=g, inner_k_tiles=8, padding=False).to(DEV)
    lin.weight, lin.scales_and_zeros = packed, sz
    x = randn_bf16((m, k), seed=m).to(DEV)
    resid = randn_bf16((m, n), seed=m + 1).to(DEV)
    gamma = (1 + 0.1 * torch.randn(n, generator=torch.Generator().manual_seed(3))).to(torch.bfloat16).to(DEV)
    slices = ops.int4_partial_slices(m, lin)
    assert slices >= 1
    parts = ops.int4_mm_partials(x, packed, g, sz, slices)
    assert parts.shape == (slices, m, n) and parts.dtype == torch.float32
    y = ops.int4_mm_direct(x, packed, g, sz)
    total = parts[0].clone()
    for s in range(1, slices):
        total += parts[s]
    assert torch.equal(total.to(torch.bfloat16), y)
    h1, n1 = ops.add_rmsnorm(resid, y, gamma, 1e-5)
    h2, n2 = ops.add_rmsnorm(resid, parts, gamma, 1e-5)
    assert torch.equal(h1, h2) and torch.equal(n1, n2)


@pytest.mark.parametrize("m,n,k", [(32, 4096, 4096), (1, 4096, 4096), (5, 4096, 11008), (64, 1024, 2048), (17, 264, 1024)])
def test_int8_partial_sums_handed_to_the_norm_equal_the_combined_matmul(m, n, k):
    """The int8 pair: unscaled K-slice sums + column scales into the norm against e2h_int8_mm + e2h_add_rmsnorm."""
    w = randn_bf16((n, k), std=0.02, seed=n + k + 1).to(DEV)
    q, scales, _ = e2h.dynamically_quantize_per_channel(w.float(), -128, 127, torch.int8)
    lin = e2h.WeightOnlyInt8Linear(k, n).to(DEV)
    lin.load_state_dict({"weight": q, "scales": scales})
    x = randn_bf16((m, k), seed=m + 7).to(DEV)
    resid = randn_bf16((m, n), seed=m + 8).to(DEV)
    gamma = (1 + 0.1 * torch.randn(n, generator=torch.Generator().manual_seed(5))).to(torch.bfloat16).to(DEV)
    slices = ops.int8_partial_slices(m, lin)
    assert slices >= 1
    parts = ops.int8_mm_partials(x, lin.weight, lin.scales, slices)
    assert parts.partials.shape == (slices, m, n)
    y = ops.int8_mm_direct(x, lin.weight, lin.scales)
    h1, n1 = ops.add_rmsnorm(resid, y, gamma, 1e-5)
    h2, n2 = ops.add_rmsnorm(resid, parts, gamma, 1e-5)
    assert torch.equal(h1, h2) and torch.equal(n1, n2)


def test_partial_sum_form_is_refused_where_it_does_not_apply():
    lin = e2h.WeightOnlyInt4Linear(1024, 64, bias=False, groupsize=128, inner_k_tiles=4, padding=False)
    assert ops.int4_partial_slices(8, lin) == 0                     # inner_k_tiles 4
    lin8 = e2h.WeightOnlyInt4Linear(1024, 64, bias=False, groupsize=128, inner_k_tiles=8, padding=False)
    assert ops.int4_partial_slices(65, lin8) == 0 and ops.int4_partial_slices(0, lin8) == 0
    assert ops.int4_partial_slices(8, lin8) >= 1
    from easy_to_hard_amd import _lib
    lib = _lib.load()
    assert lib.e2h_int4_mm_partial_slices(8, 64, 1024, 256, 8) < 0    # group size 256
    assert lib.e2h_int4_mm_partial_slices(8, 60, 1024, 128, 8) < 0    # N % 8
    x = randn_bf16((8, 1024), seed=1).to(DEV)
    w = randn_bf16((64, 1024), std=0.02, seed=2).to(DEV)
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(w, 128, 8)
    want = ops.int4_partial_slices(8, lin8)
    out = torch.empty((want + 1, 8, 64), dtype=torch.float32, device=DEV)
    rc = lib.e2h_int4_mm_partials(ops._ptr(x), ops._ptr(packed), ops._ptr(sz), ops._ptr(out), 8, 64, 1024, 128, 8, want + 1, ops._stream(x))
    assert rc < 0                                                   # a slice count other than the library's own


@pytest.mark.parametrize("mode", ["int4", "int8"])
@pytest.mark.parametrize("bsz", [32, 5])
def test_decode_step_with_deferred_slices_equals_the_step_without(bsz, mode, monkeypatch):
    """The fused decode step with wo / w2 handing partial sums to the norms (model.DEFER_SPLIT_K) against the same step with
    the matmuls combining their slices themselves, on two layers of the 7B shape (K = 4096 and 11008 are long enough for
    the library to split): identical logits, eagerly and from a HIP graph."""
    import easy_to_hard_amd.model as model_mod
    from easy_to_hard_amd.model import ModelArgs, random_quantized_transformer

    cfg = ModelArgs.from_name("7B")
    cfg.n_layer = 2
    model = random_quantized_transformer(cfg, mode, 128, device=DEV, seed=7)
    t = 7
    prompt = torch.randint(0, cfg.vocab_size, (bsz, t), generator=torch.Generator().manual_seed(4)).to(DEV)
    calls = []
    name = mode + "_mm_partials"
    real = getattr(ops, name)
    monkeypatch.setattr(ops, name, lambda *a, **k: (calls.append(a[-1]), real(*a, **k))[1])
    logits = {}
    monkeypatch.setattr(model_mod, "STAGED_DECODE", False)  # this test is about the row-major kernels' K-slice hand-over
    for defer in (False, True):
        model_mod.DEFER_SPLIT_K = defer
        try:
            model.max_seq_length = -1
            model.setup_caches(bsz, 32)
            cur = prefill(model, prompt, torch.arange(0, t, device=DEV))
            out = []
            for i in range(3):
                lg = model(cur, torch.tensor([t + i], device=DEV))
                out.append(lg[:, -1].clone())
                cur = torch.argmax(lg[:, -1].float(), dim=-1, keepdim=True)
            logits[defer] = torch.stack(out)
            if defer:
                assert calls and min(calls) > 1          # both projections of both layers took the partial-sum form
                stepper = GraphedDecodeStep(model, bsz, DEV)
                prefill(model, prompt, torch.arange(0, t, device=DEV))
                first = torch.argmax(logits[False][0].float(), dim=-1, keepdim=True)
                tok = stepper.step(first, torch.tensor([t + 1], device=DEV)).clone()
                assert torch.equal(tok, torch.argmax(logits[False][1].float(), dim=-1, keepdim=True))
            else:
                assert not calls
        finally:
            model_mod.DEFER_SPLIT_K = True
    assert torch.equal(logits[True], logits[False])


def test_staged_decode_step_agrees_with_the_row_major_fused_step(monkeypatch):
    """The single-token step on staged activations (model.STAGED_DECODE) against the same step on the row-major fused
    kernels, two layers of the 7B shape at 32 and 5 rows: same arithmetic up to the order of the float32 sums over K, so the
    logits agree to bfloat16 rounding noise; the staged step replayed from a HIP graph equals its eager run bit for bit."""
    import easy_to_hard_amd.model as model_mod
    from easy_to_hard_amd.model import ModelArgs, random_quantized_transformer

    cfg = ModelArgs.from_name("7B")
    cfg.n_layer = 2
    model = random_quantized_transformer(cfg, "int4", 128, device=DEV, seed=7)
    t = 7
    for bsz in (32, 5):
        prompt = torch.randint(0, cfg.vocab_size, (bsz, t), generator=torch.Generator().manual_seed(4)).to(DEV)
        logits = {}
        for staged in (False, True):
            monkeypatch.setattr(model_mod, "STAGED_DECODE", staged)
            model.max_seq_length = -1
            model.setup_caches(bsz, 32)
            assert model.staged_step_supported(bsz) == staged
            cur = prefill(model, prompt, torch.arange(0, t, device=DEV))
            out = []
            for i in range(3):
                lg = model(cur, torch.tensor([t + i], device=DEV))
                out.append(lg[:, -1].clone())
                cur = torch.argmax(lg[:, -1].float(), dim=-1, keepdim=True)
            logits[staged] = torch.stack(out).float()
        err = (logits[True] - logits[False]).abs().max() / logits[False].abs().max()
        assert err <= 2e-2, err
        stepper = GraphedDecodeStep(model, bsz, DEV)
        prefill(model, prompt, torch.arange(0, t, device=DEV))
        first = torch.argmax(logits[True][0], dim=-1, keepdim=True)
        tok = stepper.step(first, torch.tensor([t + 1], device=DEV)).clone()
        assert torch.equal(tok, torch.argmax(logits[True][1], dim=-1, keepdim=True))


@pytest.mark.gpu
def test_greedy_token_from_the_head_launch_equals_argmax_over_logits(monkeypatch):
    """decode_one_token on an int4 model: the head launch that reduces its own columns picks the tokens that argmax over
    the stored logits picks (FUSE_HEAD_ARGMAX off), eagerly and through the captured graph."""
    import easy_to_hard_amd.model as model_mod

    cfg = model_mod.ModelArgs.from_name("7B")  # two layers of the 7B shape: every launch of the step has a staged form
    cfg.n_layer = 2
    model = model_mod.random_quantized_transformer(cfg, "int4", 128, device=DEV, seed=11)
    bsz = 32
    with torch.no_grad():
        model.setup_caches(max_batch_size=bsz, max_seq_length=64)
        prompt = torch.randint(0, cfg.vocab_size, (bsz, 9), generator=torch.Generator().manual_seed(2)).to(DEV)
        stepper = GraphedDecodeStep(model, bsz, DEV)  # (its capture warm-up writes cache row 0: the prompt comes after it)
        cur = prefill(model, prompt, torch.arange(0, 9, device=DEV))
        pos = torch.tensor([9], device=DEV, dtype=torch.int64)
        assert model.staged_step_supported(bsz)
        fused = decode_one_token(model, cur, pos)
        graphed = stepper.step(cur, pos).clone()
        monkeypatch.setattr(model_mod, "FUSE_HEAD_ARGMAX", False)
        plain = decode_one_token(model, cur, pos)
        logits = model(cur, pos)
    assert fused.shape == (bsz, 1) and fused.dtype == torch.int64
    assert torch.equal(fused, plain) and torch.equal(graphed, plain)
    assert torch.equal(plain, torch.argmax(logits[:, -1].float(), dim=-1, keepdim=True))


@pytest.mark.gpu
def test_read_only_probe_accepts_and_rejects_as_declared():
    """e2h_stream_read_probe (the launch behind `bench.py --floor`): it writes nothing, so what can be checked is that
    the documented argument ranges are accepted (empty launch, private bytes only, private + shared) and that bad sizes,
    a missing pointer and a misaligned one come back as their status codes."""
    import ctypes

    from easy_to_hard_amd import _lib

    lib = _lib.load()
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    shared = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p, s = ctypes.c_void_p(buf.data_ptr()), ctypes.c_void_p(shared.data_ptr())
    assert lib.e2h_stream_read_probe(None, 0, None, 0, None, stream) == 0
    assert lib.e2h_stream_read_probe(p, buf.numel(), None, 0, None, stream) == 0
    assert lib.e2h_stream_read_probe(p, buf.numel(), s, shared.numel(), None, stream) == 0
    assert lib.e2h_stream_read_probe(p, 24, None, 0, None, stream) == -2          # not a multiple of 16
    assert lib.e2h_stream_read_probe(p, 1 << 31, None, 0, None, stream) == -2     # beyond the 2 GB a launch addresses
    assert lib.e2h_stream_read_probe(None, 16, None, 0, None, stream) == -1
    assert lib.e2h_stream_read_probe(p, 16, None, 16, None, stream) == -1
    assert lib.e2h_stream_read_probe(ctypes.c_void_p(buf.data_ptr() + 8), 16, None, 0, None, stream) == -5
    torch.cuda.synchronize()
    assert not buf.any() and not shared.any()

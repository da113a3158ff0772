"""GPU parity at the sizes of the benchmark configurations, through the C ABI:

* the tile-packed layout against PyTorch-ROCm's own packer (an independent library), nibble for nibble;
* the 7B int4 g128 model (32 layers, batch 32, prompt 256) teacher-forced against an oracle copy whose linears are the
  dequantized weights applied with float32 F.linear, and its 32000 x 4096 output head alone;
* every linear shape of the 34B g64 configuration at 64 rows (sampled columns against the numpy oracle), including the
  gated pair and the grouped-query q|k|v projection with RoPE and cache write;
* every linear shape of the int8 reward-scoring configuration at its 49152 rows.
"""

import numpy as np
import pytest
import torch
import torch.nn as nn

import easy_to_hard_amd as e2h
from easy_to_hard_amd import _lib, ops
from easy_to_hard_amd.generate import decode_one_token
from easy_to_hard_amd.model import ModelArgs, apply_rotary_emb, precompute_freqs_cis, random_quantized_transformer
from oracle import quant_oracle as qo
from tests.helpers import bf16_to_np, randn_bf16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2


# ---- the packed layout against an independent packer ---------------------------------------------------------------

@pytest.mark.parametrize("ikt", [2, 4, 8])
def test_tile_packed_words_equal_the_stock_rocm_packer_after_its_lane_permutation(ikt):
    """PyTorch-ROCm's aten._convert_weight_to_int4pack packs the same codes with the same bit formula inside a word
    (v0 | v2<<4 | v4<<8 | v6<<12 | v1<<16 | v3<<20 | v5<<24 | v7<<28, v0..v3 from one 16-wide k tile and v4..v7 from
    the next) but with the lane -> (row, k) map of a 16x16x16 MFMA operand: memory is [N/16][K/(16 ikt)][64][ikt/2],
    lane t holds row 16 by + (t & 15) and the four consecutive k values 4 (t >> 4) .. +3 of each k tile.  The checkpoint
    layout (PyTorch 2.2 CUDA) holds row 8 nTile + t/4 and k values 2j, 2j+1, 2j+8, 2j+9 (j = t & 3).  Every checkpoint
    word is therefore a fixed gather of nibbles from two of the stock packer's words; that gather is applied here to the
    stock packer's output and must reproduce e2h_int4_pack bit for bit.  This pins the nibble order inside a word and
    the pairing of two k tiles per word against a library; the lane map of the CUDA layout itself stays as recalled."""
    n, k = 64, 16 * ikt * 5
    gen = torch.Generator().manual_seed(100 + ikt)
    codes = torch.randint(0, 16, (n, k), generator=gen, dtype=torch.int32)
    ours = ops.int4_pack(codes.to(DEV), ikt).cpu().numpy().astype(np.uint32)          # [N/8][KT][32][ikt/2]
    two_per_byte = ((codes[:, ::2] << 4) | codes[:, 1::2]).to(torch.uint8).to(DEV)
    try:
        stock = torch.ops.aten._convert_weight_to_int4pack(two_per_byte, ikt)
        torch.cuda.synchronize()
    except (RuntimeError, NotImplementedError) as exc:
        pytest.skip(f"stock aten._convert_weight_to_int4pack unavailable here: {exc}")
    kt = k // (16 * ikt)
    assert tuple(stock.shape) == (n // 8, kt, 32, ikt // 2)
    stock = stock.cpu().numpy().astype(np.uint32).reshape(n // 16, kt, 64, ikt // 2)   # how its memory is indexed
    # stock word (by, kx, t, p): element e of k tile 0 is value v_e, of k tile 1 is v_{4+e}; value v_i sits at this shift
    shift = {0: 0, 2: 4, 4: 8, 6: 12, 1: 16, 3: 20, 5: 24, 7: 28}
    rebuilt = np.zeros_like(ours)
    for n_tile in range(n // 8):
        for t in range(32):
            row, j = 8 * n_tile + t // 4, t & 3
            by, c = row // 16, row % 16
            e = (2 * j) & 3                                     # position of k = 2j (and 2j+8) inside its group of four
            lo = stock[by, :, 16 * (j >> 1) + c, :]             # lane with kb = j/2: k = 2j, 2j+1
            hi = stock[by, :, 16 * (2 + (j >> 1)) + c, :]       # lane with kb = 2 + j/2: k = 2j+8, 2j+9
            v = [(lo >> shift[e]) & 15, (lo >> shift[e + 1]) & 15, (hi >> shift[e]) & 15, (hi >> shift[e + 1]) & 15,
                 (lo >> shift[4 + e]) & 15, (lo >> shift[5 + e]) & 15, (hi >> shift[4 + e]) & 15, (hi >> shift[5 + e]) & 15]
            word = np.zeros_like(lo)
            for i in range(8):
                word |= v[i] << shift[i]
            rebuilt[n_tile, :, t, :] = word
    np.testing.assert_array_equal(rebuilt, ours)
    # and the oracle's packer writes the same bytes
    np.testing.assert_array_equal(qo.int4_tile_pack(codes.numpy(), ikt).astype(np.uint32), ours)


# ---- helpers: oracle-side dequantization on the GPU (pure torch index arithmetic, checked against the numpy oracle) ----

def _torch_tile_unpack(packed, ikt):
    """[N/8, KT, 32, ikt/2] int32 -> codes int32 [N, K] with stock torch ops (the layout statement of the oracle's
    int4_tile_unpack, restated so that 7B-sized weights can be unpacked on the GPU)."""
    n8, kt, _, pairs = packed.shape
    nib = (packed.unsqueeze(-1) >> (4 * torch.arange(8, device=packed.device, dtype=torch.int32))) & 15   # [n8, kt, 32, P, 8]
    nib = nib.view(n8, kt, 8, 4, pairs, 8).permute(0, 2, 1, 4, 3, 5).reshape(n8, 8, kt, pairs, 32)        # (.., j * 8 + i)
    koff = torch.empty(32, dtype=torch.int64)
    for j in range(4):
        for i, off in enumerate([2 * j, 2 * j + 8, 16 + 2 * j, 24 + 2 * j, 2 * j + 1, 2 * j + 9, 17 + 2 * j, 25 + 2 * j]):
            koff[j * 8 + i] = off
    out = torch.empty_like(nib)
    out.index_copy_(4, koff.to(packed.device), nib)
    return out.reshape(n8 * 8, kt * pairs * 32)


def _torch_dequant_fp32(packed, sz, g, ikt=8):
    codes = _torch_tile_unpack(packed, ikt)
    s = sz[..., 0].t().float().repeat_interleave(g, dim=1)
    z = sz[..., 1].t().float().repeat_interleave(g, dim=1)
    return (codes - 8).float() * s + z


def test_torch_side_dequantizer_equals_the_numpy_oracle():
    for ikt, g in ((8, 128), (4, 64), (2, 32)):
        w = randn_bf16((40, 512), std=0.02, seed=ikt)
        codes, sz = qo.int4_group_quantize(bf16_to_np(w), 4, g)
        packed = torch.from_numpy(qo.int4_tile_pack(codes, ikt)).to(DEV)
        sz_d = torch.from_numpy(sz).to(torch.bfloat16).to(DEV)
        assert np.array_equal(_torch_tile_unpack(packed, ikt).cpu().numpy(), codes)
        assert np.array_equal(_torch_dequant_fp32(packed, sz_d, g, ikt).cpu().numpy(), qo.int4_dequantize_fp32(codes, sz, g))


class OracleLinear(nn.Module):
    """x @ W^T with the dequantized weight (dequantize-then-F.linear), result rounded to bfloat16.  float32 weight and
    arithmetic: the parity oracle.  bfloat16 weight (rounded once, as the reference's group_dequantize_tensor produces it)
    and torch's bfloat16 F.linear: the reference's own arithmetic, whose distance from the float32 oracle is the noise
    floor that any bfloat16 implementation of the model shows."""

    def __init__(self, w):
        super().__init__()
        self.register_buffer("w", w)

    def forward(self, x):
        return torch.nn.functional.linear(x.to(self.w.dtype), self.w).to(torch.bfloat16)


def _oracle_twin(model, dtype=torch.float32):
    """Same module tree, same non-linear parameters, every int4 linear replaced by dequantize-then-F.linear in `dtype`."""
    import copy

    twin = copy.deepcopy(model)
    for _, mod in list(twin.named_modules()):
        for child_name, child in list(mod.named_children()):
            if isinstance(child, e2h.WeightOnlyInt4Linear):
                w = _torch_dequant_fp32(child.weight, child.scales_and_zeros, child.groupsize)
                setattr(mod, child_name, OracleLinear(w.to(dtype)))
    return twin


# ---- the 7B int4 g128 decode configuration -----------------------------------------------------------------------

@pytest.mark.parametrize("m", [1, 32])
def test_output_head_32000x4096_g128(m):
    n, k, g = 32000, 4096, 128
    gen = torch.Generator(device=DEV).manual_seed(11)
    w = (torch.randn((n, k), generator=gen, device=DEV) * 0.02).to(torch.bfloat16)
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(w, g, 8)
    x = randn_bf16((m, k), seed=m)
    y = ops.int4_mm_direct(x.to(DEV), packed, g, sz)
    tiles = np.unique(np.concatenate([[0, 1, n // 8 - 1], np.random.default_rng(3).integers(0, n // 8, 125)]))
    cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    codes = qo.int4_tile_unpack(packed[torch.from_numpy(tiles).to(DEV)].cpu().numpy(), 8)
    sz_s = bf16_to_np(sz[:, torch.from_numpy(cols).to(DEV), :])
    y_ref = qo.int4_linear_fp32(bf16_to_np(x), codes, sz_s, g)
    got = bf16_to_np(y[:, torch.from_numpy(cols).to(DEV)])
    assert qo.normwise_rel_err(got, y_ref) <= TOL
    assert qo.elementwise_violations(got, y_ref) == 0.0


def _spread(first, last, count):
    return sorted({first + round(i * (last - first) / (count - 1)) for i in range(count)})


def _decode_against_the_oracle_model(cfg, g, bsz, t_prompt, n_new, steps, label):
    """Random-init model of shape `cfg` (weights from a CPU generator, seed 1234), int4 with group size g, batch bsz, prompt
    of t_prompt uniform token ids: prefill, then `steps` greedy decode steps (reference inference_generate.py:123-157, one
    token per sequence and step) at cache positions spread from the end of the prompt to the end of the cache
    (t_prompt + n_new - 1) -- the positions bench.py times -- every step compared with a float32 oracle twin that sees the
    same tokens and the same cache (teacher forcing; cache rows between the visited positions hold the same N(0, 1)
    stand-ins in every model, as in bench.py).

    Token identity: wherever the oracle's top-1 / top-2 logit margin exceeds twice the measured logit noise of the step
    (max |logit - oracle logit|), the greedy token must be the oracle's; the histogram of margin / noise and the agreement
    in every bucket are printed.  Random-init logits over a vocabulary of 32000 are near ties, so most rows sit below that
    margin; for those the agreement rate must not fall behind that of the reference's own arithmetic (bfloat16
    dequantized weights, torch's bfloat16 F.linear) by more than 5 % of the rows.  Logits: normwise error at most the
    larger of 2e-2 and 1.5 x the error of the reference's arithmetic against the same oracle (many layers of bfloat16
    activations amplify rounding differences).  Finally the HIP-graph replayed step must reproduce the eager step bit
    for bit at this size."""
    from easy_to_hard_amd.generate import GraphedDecodeStep

    model = random_quantized_transformer(cfg, "int4", g, device=DEV, seed=1234, seed_on="cpu")
    max_seq = t_prompt + n_new
    model.setup_caches(bsz, max_seq)
    oracle = _oracle_twin(model, torch.float32)
    ref_arith = _oracle_twin(model, torch.bfloat16)
    prompt = torch.randint(0, cfg.vocab_size, (bsz, t_prompt), generator=torch.Generator().manual_seed(1234)).to(DEV)
    pos = torch.arange(0, t_prompt, device=DEV)
    report = []
    edges = [0.0, 0.5, 1.0, 2.0, 4.0, float("inf")]
    hist = [[0, 0, 0] for _ in edges[:-1]]  # per bucket of margin / noise: rows, rows equal to the oracle, same for the reference arithmetic
    counts = {"rows": 0, "same": 0, "same_ref": 0, "decided": 0}

    def compare(lq, lr, lo, what):
        lq, lr, lo = lq[:, -1].float(), lr[:, -1].float(), lo[:, -1].float()
        noise, floor = (lq - lo).abs().max(), (lr - lo).abs().max()
        scale = lo.abs().max()
        report.append((what, round(float(noise / scale), 4), round(float(floor / scale), 4)))
        assert noise <= max(2e-2 * scale, 1.5 * floor), report[-1]
        top2 = lo.topk(2, dim=-1).values
        ratio = (top2[:, 0] - top2[:, 1]) / noise
        same = lq.argmax(-1) == lo.argmax(-1)
        same_ref = lr.argmax(-1) == lo.argmax(-1)
        decided = ratio > 2.0
        assert bool(same[decided].all()), (what, "a greedy token differs from the oracle's above the noise margin")
        for i in range(len(hist)):
            in_bucket = (ratio >= edges[i]) & (ratio < edges[i + 1])
            hist[i][0] += int(in_bucket.sum())
            hist[i][1] += int((in_bucket & same).sum())
            hist[i][2] += int((in_bucket & same_ref).sum())
        counts["rows"] += lq.shape[0]
        counts["same"] += int(same.sum())
        counts["same_ref"] += int(same_ref.sum())
        counts["decided"] += int(decided.sum())

    with torch.no_grad():
        lq = model(prompt, pos)
        compare(lq, ref_arith(prompt, pos), oracle(prompt, pos), "prefill")
        cur = lq[:, -1].float().argmax(-1, keepdim=True)
        # cache rows beyond the prompt: the same stand-ins in the three models
        gen_dev = torch.Generator(device=DEV).manual_seed(1234)
        for blk, blk_o, blk_r in zip(model.layers, oracle.layers, ref_arith.layers):
            for name in ("k_cache", "v_cache"):
                cache = getattr(blk.attention.kv_cache, name)
                fill = torch.randn(cache[:, :, t_prompt:].shape, generator=gen_dev, device=DEV, dtype=torch.float32).to(cache.dtype)
                for b_ in (blk, blk_o, blk_r):
                    getattr(b_.attention.kv_cache, name)[:, :, t_prompt:] = fill
        positions = _spread(t_prompt, max_seq - 2, steps)
        for p in positions:
            step_pos = torch.tensor([p], device=DEV, dtype=torch.int64)
            lq = model(cur, step_pos)
            compare(lq, ref_arith(cur, step_pos), oracle(cur, step_pos), f"position {p}")
            cur = lq[:, -1].float().argmax(-1, keepdim=True)
        print(f"{label}: (step, normwise logit error vs float32 oracle, same for the reference's bf16 arithmetic):", report)
        print("margin / noise bucket: rows, greedy token equal to the oracle's, same for the reference's bf16 arithmetic")
        for i in range(len(hist)):
            print(f"  [{edges[i]}, {edges[i + 1]}): {hist[i][0]}, {hist[i][1]}, {hist[i][2]}")
        total, same, same_ref = counts["rows"], counts["same"], counts["same_ref"]
        print(f"greedy tokens equal to the float32 oracle's: {same} of {total} ({counts['decided']} rows above the noise margin, all equal); "
              f"the reference's bf16 arithmetic: {same_ref} of {total}")
        assert len(positions) >= 32 and positions[-1] >= max_seq - 2
        assert same >= same_ref - total // 20 and same >= total * 2 // 3, (same, same_ref)
        del oracle, ref_arith
        # the graph-replayed step reproduces the eager step bit for bit at this size too
        step_pos = torch.tensor([max_seq - 1], device=DEV, dtype=torch.int64)
        eager = decode_one_token(model, cur, step_pos)
        row0 = [(blk.attention.kv_cache.k_cache[:, :, 0].clone(), blk.attention.kv_cache.v_cache[:, :, 0].clone()) for blk in model.layers]
        stepper = GraphedDecodeStep(model, bsz, DEV)   # its warm-up overwrites cache row 0 (and nothing else): put it back
        for blk, (k0, v0) in zip(model.layers, row0):
            blk.attention.kv_cache.k_cache[:, :, 0] = k0
            blk.attention.kv_cache.v_cache[:, :, 0] = v0
        replay = stepper.step(cur, step_pos).clone()
        assert torch.equal(eager, replay)


def test_7b_int4_g128_batch32_decode_against_the_oracle_model():
    """The 7B decode configuration at its full size: 32 layers, batch 32, prompt 256, 512 new tokens; 33 decode steps at
    cache positions 256 .. 766."""
    _decode_against_the_oracle_model(ModelArgs.from_name("7B"), 128, 32, 256, 512, 33, "7B int4 g128 bs32")


def test_34b_int4_g64_batch64_decode_against_the_oracle_model():
    """The 34B decode configuration (dim 8192, 64 query / 8 kv heads, FFN 22016, group size 64, batch 64, prompt 512, 256
    new tokens) at full width with the first 8 of its 48 layers: every kernel of the step runs at its real shape
    (32768-row prefill matmuls, two-slab 64-row decode launches, grouped-query attention on the matrix cores), and the
    float32 oracle twin of 8 layers fits next to it; 32 decode steps at cache positions 512 .. 766."""
    cfg = ModelArgs.from_name("34B")
    cfg.n_layer = 8
    _decode_against_the_oracle_model(cfg, 64, 64, 512, 256, 32, "34B (8 layers) int4 g64 bs64")


# ---- the 34B int4 g64 decode configuration: every linear shape at 64 rows ----------------------------------------

def _sampled_columns(n, count, seed):
    tiles = np.unique(np.concatenate([[0, 1, n // 8 - 1], np.random.default_rng(seed).integers(0, n // 8, count)]))
    cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    return torch.from_numpy(tiles).to(DEV), torch.from_numpy(cols).to(DEV)


def _big_int4_weight(n, k, g, seed):
    gen = torch.Generator(device=DEV).manual_seed(seed)
    w = (torch.randn((n, k), generator=gen, device=DEV) * 0.02).to(torch.bfloat16)
    return e2h.prepare_int4_weight_and_scales_and_zeros(w, g, 8)


def _oracle_columns(x, packed, sz, tiles, cols, g):
    codes = qo.int4_tile_unpack(packed[tiles].cpu().numpy(), 8)
    return qo.int4_linear_fp32(bf16_to_np(x), codes, bf16_to_np(sz[:, cols, :]), g)


@pytest.mark.parametrize("n,k", [(10240, 8192), (8192, 8192), (22016, 8192), (8192, 22016), (32000, 8192)])
@pytest.mark.parametrize("m", [64, 33, 1])
def test_34b_linear_shapes_g64(n, k, m):
    g = 64
    packed, sz = _big_int4_weight(n, k, g, seed=n + k)
    x = randn_bf16((m, k), seed=m + 5)
    y = ops.int4_mm_direct(x.to(DEV), packed, g, sz)
    tiles, cols = _sampled_columns(n, 61, seed=n)
    y_ref = _oracle_columns(x, packed, sz, tiles, cols, g)
    got = bf16_to_np(y[:, cols])
    assert qo.normwise_rel_err(got, y_ref) <= TOL
    assert qo.elementwise_violations(got, y_ref) == 0.0


def test_34b_prefill_rows_8192x22016_g64_in_one_launch():
    """The prefill of the 34B configuration gives every linear 64 x 512 = 32768 rows; with K = 22016 at group size 64 the
    group sums of x for that many rows do not fit the workspace, and a call that needs them is cut into slices of rows.
    The 256-row kernel needs none: the whole call must go to it in one piece (sampled rows and columns against the
    oracle; rows on both sides of where the slices would have been cut)."""
    n, k, g, m = 8192, 22016, 64, 32768
    packed, sz = _big_int4_weight(n, k, g, seed=77)
    gen = torch.Generator(device=DEV).manual_seed(78)
    x = torch.randn((m, k), generator=gen, device=DEV).to(torch.bfloat16)
    y = ops.int4_mm_direct(x, packed, g, sz)
    rows = torch.tensor([0, 1, 255, 256, 12345, 24319, 24320, 24321, 32000, 32767], device=DEV)
    tiles, cols = _sampled_columns(n, 29, seed=3)
    y_ref = _oracle_columns(x[rows].cpu(), packed, sz, tiles, cols, g)
    got = bf16_to_np(y[rows][:, cols])
    assert qo.normwise_rel_err(got, y_ref) <= TOL
    assert qo.elementwise_violations(got, y_ref) == 0.0
    # the same rows as a small call (the exact-product kernel): agreement to the bfloat16 rounding of the weights
    small = ops.int4_mm_direct(x[rows].contiguous(), packed, g, sz)
    assert (small.float() - y[rows].float()).abs().max().item() <= 2.0 ** -6 * small.float().abs().max().item()


@pytest.mark.parametrize("m", [64, 32])
def test_34b_gated_pair_2x22016x8192_g64(m):
    n, k, g = 22016, 8192, 64
    p1, s1 = _big_int4_weight(n, k, g, seed=1)
    p2, s2 = _big_int4_weight(n, k, g, seed=2)
    x = randn_bf16((m, k), seed=m)
    xd = x.to(DEV)
    y = ops.int4_mm_silu_gate(xd, p1, s1, p2, s2, g)
    tiles, cols = _sampled_columns(n, 61, seed=9)
    a = _oracle_columns(x, p1, s1, tiles, cols, g).astype(np.float64)
    b = _oracle_columns(x, p2, s2, tiles, cols, g).astype(np.float64)
    ref = a / (1.0 + np.exp(-a)) * b
    assert qo.normwise_rel_err(bf16_to_np(y[:, cols]), ref) <= TOL
    _lib.set_option("int4_k_slices", 1)
    try:
        ya, yb = ops.int4_mm_direct(xd, p1, g, s1), ops.int4_mm_direct(xd, p2, g, s2)
    finally:
        _lib.set_option("int4_k_slices", 0)
    assert torch.equal(y, ops.silu_mul(ya, yb))


@pytest.mark.parametrize("bsz,tiles_per_wave", [(64, 0), (64, 1), (33, 2), (32, 0), (32, 2)])
def test_34b_grouped_query_projection_with_rope_and_cache_write_g64(bsz, tiles_per_wave):
    """tiles_per_wave 0 = the library's own choice (two column tiles per wave at 33 .. 64 rows of this shape, one at 32),
    1 / 2 = that geometry forced for the fused launch."""
    n_head, n_kv, d, k, g = 64, 8, 128, 8192, 64
    n = (n_head + 2 * n_kv) * d
    s_max, pos = 96, 41
    packed, sz = _big_int4_weight(n, k, g, seed=3)
    x = randn_bf16((bsz, k), seed=4)
    xd = x.to(DEV)
    gen = torch.Generator().manual_seed(5)
    kc0 = torch.randn((bsz, n_kv, s_max, d), generator=gen).to(torch.bfloat16).to(DEV)
    vc0 = torch.randn((bsz, n_kv, s_max, d), generator=gen).to(torch.bfloat16).to(DEV)
    freqs = precompute_freqs_cis(s_max, d, 1000000, device=DEV)
    input_pos = torch.tensor([pos], device=DEV)
    kc, vc = kc0.clone(), vc0.clone()
    _lib.set_option("int4_rows_per_wave", 16 * tiles_per_wave)
    try:
        q = ops.int4_mm_rope_kv(xd, packed, sz, g, freqs, kc, vc, input_pos, n_head, n_kv, d)
    finally:
        _lib.set_option("int4_rows_per_wave", 0)
    _lib.set_option("int4_k_slices", 1)
    try:
        qkv = ops.int4_mm_direct(xd, packed, g, sz)
    finally:
        _lib.set_option("int4_k_slices", 0)
    kc2, vc2 = kc0.clone(), vc0.clone()
    q2 = ops.rope_kv_write(qkv, freqs, kc2, vc2, input_pos, n_head, n_kv, d)
    assert torch.equal(q, q2) and torch.equal(kc, kc2) and torch.equal(vc, vc2)
    # heads 0, 17 and 63 of q, kv heads 0 and 7 of k and v against stock ops on the oracle's projection
    heads = [0, 17, 63, n_head + 0, n_head + 7, n_head + n_kv + 0, n_head + n_kv + 7]
    cols = torch.cat([torch.arange(h * d, (h + 1) * d) for h in heads]).to(DEV)
    tiles = torch.unique(cols // 8)
    y_ref = torch.from_numpy(_oracle_columns(x, packed, sz, tiles, cols, g)).to(torch.bfloat16).to(DEV).view(bsz, 1, len(heads), d)
    fc = freqs[input_pos]
    rot = apply_rotary_emb(y_ref[:, :, :5], fc).squeeze(1)           # q and k heads are rotated, v heads are not
    scale = float(y_ref.float().abs().max())
    assert (q[:, [0, 17, 63]].float() - rot[:, :3].float()).abs().max() <= TOL * scale
    assert (kc[:, [0, 7], pos].float() - rot[:, 3:5].float()).abs().max() <= TOL * scale
    assert (vc[:, [0, 7], pos].float() - y_ref[:, 0, 5:].float()).abs().max() <= TOL * scale
    untouched = torch.ones(s_max, dtype=torch.bool, device=DEV)
    untouched[pos] = False
    assert torch.equal(kc[:, :, untouched], kc0[:, :, untouched]) and torch.equal(vc[:, :, untouched], vc0[:, :, untouched])


# ---- the int8 reward-scoring configuration: every linear shape at 64 x 768 = 49152 rows ----------------------------

@pytest.mark.parametrize("n,k", [(12288, 4096), (11008, 4096), (4096, 11008), (2, 4096), (1, 4096)])
def test_int8_reward_scoring_shapes_at_49152_rows(n, k):
    m = 49152
    w = randn_bf16((n, k), std=0.02, seed=n + k)
    q, s, _ = qo.int8_quantize_per_channel(w.float().numpy())
    s = qo.bf16_round(s)
    q_d, s_d = torch.from_numpy(q).to(DEV), torch.from_numpy(s).to(torch.bfloat16).to(DEV)
    gen = torch.Generator().manual_seed(n)
    x = torch.randn(4096, k, generator=gen).to(torch.bfloat16).repeat(m // 4096, 1)
    x[-3:] = torch.randint(-2, 3, (3, k), generator=gen).to(torch.bfloat16)
    x_d = x.to(DEV)
    y = ops.int8_mm_direct(x_d, q_d, s_d)
    assert y.shape == (m, n) and bool(torch.isfinite(y.float()).all())
    rows = [0, 1, 255, 256, 4095, 4096, 24575, 49151 - 3, 49151]
    y_ref = qo.int8_linear_fp32(bf16_to_np(x[rows]), q, s)
    assert qo.normwise_rel_err(bf16_to_np(y[rows].cpu()), y_ref) <= TOL
    assert torch.equal(y[:4096], y[4096:8192]) and torch.equal(y[:4096], y[4096 * 7:4096 * 8])
    y_int = qo.int8_linear_reference_rounding(bf16_to_np(x[-3:]), q, s)
    assert np.array_equal(bf16_to_np(y[-3:].cpu()), y_int)

"""GPU checks of the decode-step kernels around the linears (RMSNorm, SiLU*mul, RoPE + KV write, single-query
attention) against the stock torch ops the harness otherwise uses, through the C ABI."""

import pytest
import torch
import torch.nn.functional as F

import easy_to_hard_amd.model as model_mod
from easy_to_hard_amd import ops
from easy_to_hard_amd.generate import decode_one_token, prefill
from easy_to_hard_amd.model import Transformer, apply_rotary_emb, init_random_, precompute_freqs_cis
from tests.helpers import randn_bf16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rmsnorm_reference(x, w, eps):
    """RMSNorm with the reference's rounding points (models/model.py:363-377) on stock ops.  mean(x^2) depends on the
    summation order in its last float32 bit, and where x * rsqrt(..) sits next to a bfloat16 rounding boundary that bit
    flips the first rounding and, through the multiplication by w, up to two ulps of the result (a whole row of 4096
    can do so when rsqrt(..) happens to be close to a short binary fraction): hence two ulps of tolerance and an
    "almost everywhere identical" check rather than equality."""
    xf = x.float()
    return (xf * torch.rsqrt(torch.mean(xf * xf, dim=-1, keepdim=True) + eps)).to(torch.bfloat16) * w


def test_rmsnorm_matches_stock_ops():
    for rows, dim in [(32, 4096), (5, 256), (1, 8192), (70, 512), (2, 16384), (600, 4096), (3, 20480)]:
        x = randn_bf16((rows, dim), std=1.5, seed=rows).to(DEV)
        w = (1 + 0.1 * randn_bf16((dim,), seed=dim).float()).to(torch.bfloat16).to(DEV)
        ref = _rmsnorm_reference(x, w, 1e-5)
        y = ops.rmsnorm(x, w, 1e-5)
        assert torch.allclose(y.float(), ref.float(), rtol=2 ** -6, atol=1e-6)
        assert (y == ref).float().mean() > 0.99


def test_add_rmsnorm_matches_stock_ops():
    for rows, dim in [(32, 4096), (3, 256), (2, 16384), (600, 4096), (3, 20480)]:
        x = randn_bf16((rows, dim), std=1.5, seed=rows).to(DEV)
        d = randn_bf16((rows, dim), std=0.7, seed=rows + 1).to(DEV)
        w = (1 + 0.1 * randn_bf16((dim,), seed=dim).float()).to(torch.bfloat16).to(DEV)
        h_ref = x + d
        ref = _rmsnorm_reference(h_ref, w, 1e-5)
        h, y = ops.add_rmsnorm(x, d, w, 1e-5)
        assert torch.equal(h, h_ref)
        assert torch.allclose(y.float(), ref.float(), rtol=2 ** -6, atol=1e-6)
        assert (y == ref).float().mean() > 0.99


def test_silu_mul_matches_stock_ops():
    a = randn_bf16((32, 11008), std=2.0, seed=1).to(DEV)
    b = randn_bf16((32, 11008), std=1.0, seed=2).to(DEV)
    ref = F.silu(a) * b
    y = ops.silu_mul(a, b)
    assert torch.allclose(y.float(), ref.float(), rtol=2 ** -7, atol=1e-6)
    assert (y == ref).float().mean() > 0.99


@pytest.mark.parametrize("n_head,n_kv,d", [(32, 32, 128), (64, 8, 128), (4, 4, 64), (8, 2, 64)])
def test_rope_kv_write_and_attention_match_stock_ops(n_head, n_kv, d):
    bsz, s_max, pos = 3, 96, 41
    gen = torch.Generator().manual_seed(n_head + d)
    qkv = (torch.randn((bsz, (n_head + 2 * n_kv) * d), generator=gen)).to(torch.bfloat16).to(DEV)
    kc = (torch.randn((bsz + 1, n_kv, s_max, d), generator=gen)).to(torch.bfloat16).to(DEV)
    vc = (torch.randn((bsz + 1, n_kv, s_max, d), generator=gen)).to(torch.bfloat16).to(DEV)
    freqs = precompute_freqs_cis(s_max, d, 10000, device=DEV)
    input_pos = torch.tensor([pos], device=DEV)
    # stock path
    kc_ref, vc_ref = kc.clone(), vc.clone()
    q, k, v = qkv.view(bsz, 1, -1).split([n_head * d, n_kv * d, n_kv * d], dim=-1)
    fc = freqs[input_pos]
    q_ref = apply_rotary_emb(q.view(bsz, 1, n_head, d), fc).transpose(1, 2)
    k_rot = apply_rotary_emb(k.view(bsz, 1, n_kv, d), fc).transpose(1, 2)
    kc_ref[:bsz].index_copy_(2, input_pos, k_rot)
    vc_ref[:bsz].index_copy_(2, input_pos, v.view(bsz, 1, n_kv, d).transpose(1, 2))
    # fused kernel
    q_out = ops.rope_kv_write(qkv, freqs, kc, vc, input_pos, n_head, n_kv, d)
    assert torch.equal(q_out, q_ref.squeeze(2))
    assert torch.equal(kc, kc_ref) and torch.equal(vc, vc_ref)
    # attention over positions 0..pos, with and without a left-padding mask
    for left_pad in (None, torch.tensor([0, 7, 41], device=DEV)):
        mask = (torch.arange(s_max, device=DEV) <= pos)[None, None, None, :]
        if left_pad is not None:
            vis = torch.arange(s_max, device=DEV).view(1, -1) >= left_pad.view(-1, 1)
            mask = torch.logical_and(mask, vis[:, None, None, :])
            mask = torch.logical_or(mask, (torch.arange(s_max, device=DEV) == pos)[None, None, None, :])
        rep = n_head // n_kv
        kk = kc_ref[:bsz].repeat_interleave(rep, dim=1).float()
        vv = vc_ref[:bsz].repeat_interleave(rep, dim=1).float()
        ref = F.scaled_dot_product_attention(q_ref.float(), kk, vv, attn_mask=mask).squeeze(2)
        y = ops.decode_attention(q_out, kc, vc, input_pos, left_pad)
        assert y.shape == (bsz, n_head, d)
        err = (y.float() - ref).abs().max() / ref.abs().max()
        assert err < 1e-2, err


def test_fused_decode_step_matches_stock_decode_step():
    model = Transformer.from_name("tiny-gqa-test")
    init_random_(model, seed=5, std=0.05)
    model = model.to(device=DEV, dtype=torch.bfloat16).eval()
    bsz, t = 3, 9
    prompt = torch.randint(0, 512, (bsz, t), generator=torch.Generator().manual_seed(2)).to(DEV)
    logits = {}
    for fused in (False, True):
        model_mod.FUSED_DECODE = fused
        try:
            model.max_seq_length = -1
            model.setup_caches(bsz, 32)
            cur = prefill(model, prompt, torch.arange(0, t, device=DEV))
            out = []
            for i in range(4):
                pos = torch.tensor([t + i], device=DEV)
                lg = model(cur, pos)
                out.append(lg[:, -1].float())
                cur = torch.argmax(lg[:, -1].float(), dim=-1, keepdim=True)
            logits[fused] = torch.stack(out)
        finally:
            model_mod.FUSED_DECODE = True
    err = (logits[True] - logits[False]).abs().max() / logits[False].abs().max()
    assert err < 2e-2, err


@pytest.mark.parametrize("n_head,n_kv,d", [(4, 4, 64), (8, 2, 128)])
@pytest.mark.parametrize("by_token", [False, True])
def test_rope_kv_write_seq_matches_stock_ops(n_head, n_kv, d, by_token):
    """Many tokens per sequence: q comes back head-major and rotated, k / v land in the cache rows of their positions
    (or in token order for a cache-less pass) with exactly the bits of apply_rotary_emb + KVCache.update."""
    bsz, t, s_max = 2, 7, 24
    gen = torch.Generator().manual_seed(n_head * 3 + d)
    qkv = torch.randn((bsz, t, (n_head + 2 * n_kv) * d), generator=gen).to(torch.bfloat16).to(DEV)
    freqs = precompute_freqs_cis(s_max, d, 10000, device=DEV)
    input_pos = torch.arange(5, 5 + t, device=DEV)
    rows = t if by_token else s_max
    kc0 = torch.randn((bsz + 1, n_kv, rows, d), generator=gen).to(torch.bfloat16).to(DEV)
    vc0 = torch.randn((bsz + 1, n_kv, rows, d), generator=gen).to(torch.bfloat16).to(DEV)
    kc, vc = kc0.clone(), vc0.clone()
    q_out = ops.rope_kv_write_seq(qkv, freqs, kc, vc, input_pos, n_head, n_kv, d, rows_by_token=by_token)
    q, k, v = qkv.split([n_head * d, n_kv * d, n_kv * d], dim=-1)
    fc = freqs[input_pos]
    q_ref = apply_rotary_emb(q.view(bsz, t, n_head, d), fc).transpose(1, 2)
    k_ref = apply_rotary_emb(k.view(bsz, t, n_kv, d), fc).transpose(1, 2)
    v_ref = v.view(bsz, t, n_kv, d).transpose(1, 2)
    assert q_out.shape == (bsz, n_head, t, d) and torch.equal(q_out, q_ref)
    kc_ref, vc_ref = kc0.clone(), vc0.clone()
    dest = torch.arange(t, device=DEV) if by_token else input_pos
    kc_ref[:bsz].index_copy_(2, dest, k_ref)
    vc_ref[:bsz].index_copy_(2, dest, v_ref)
    assert torch.equal(kc, kc_ref) and torch.equal(vc, vc_ref)


@pytest.mark.parametrize("fully_causal", [False, True])
def test_fused_prefill_matches_stock_prefill(fully_causal):
    model = Transformer.from_name("tiny-gqa-test")
    init_random_(model, seed=6, std=0.05)
    model = model.to(device=DEV, dtype=torch.bfloat16).eval()
    bsz, t = 3, 11
    ids = torch.randint(0, 512, (bsz, t), generator=torch.Generator().manual_seed(4)).to(DEV)
    out = {}
    for fused in (False, True):
        model_mod.FUSED_DECODE = fused
        try:
            model.max_seq_length = -1
            model.setup_caches(bsz, 32, kv_cache=not fully_causal)
            with torch.no_grad():
                out[fused] = model(ids, torch.arange(0, t, device=DEV), fully_causal=fully_causal).float()
        finally:
            model_mod.FUSED_DECODE = True
    err = (out[True] - out[False]).abs().max() / out[False].abs().max()
    assert err < 2e-2, err


@pytest.mark.parametrize("n_head,n_kv", [(16, 4), (64, 8), (32, 2), (12, 2)])
@pytest.mark.parametrize("s_max,pos", [(96, 0), (96, 31), (96, 32), (96, 41), (640, 575), (300, 299)])
def test_grouped_query_attention_on_matrix_cores_matches_sdpa_and_vector_kernel(n_head, n_kv, s_max, pos):
    """4 .. 16 query heads per kv head at head_dim 128 take the MFMA kernel (both cache lengths: 4 and 8 waves): against
    stock SDPA on the same cache, with and without left padding, and against the float32 vector kernel (the two differ
    by the bfloat16 rounding of the softmax weights only)."""
    from easy_to_hard_amd import _lib

    d, bsz = 128, 3
    rep = n_head // n_kv
    gen = torch.Generator().manual_seed(n_head * 7 + pos)
    q = torch.randn((bsz, n_head, d), generator=gen).to(torch.bfloat16).to(DEV)
    kc = torch.randn((bsz, n_kv, s_max, d), generator=gen).to(torch.bfloat16).to(DEV)
    vc = torch.randn((bsz, n_kv, s_max, d), generator=gen).to(torch.bfloat16).to(DEV)
    input_pos = torch.tensor([pos], device=DEV)
    for left_pad in (None, torch.tensor([0, min(7, pos), pos], device=DEV)):
        mask = (torch.arange(s_max, device=DEV) <= pos)[None, None, None, :]
        if left_pad is not None:
            vis = torch.arange(s_max, device=DEV).view(1, -1) >= left_pad.view(-1, 1)
            mask = torch.logical_and(mask, vis[:, None, None, :])
            mask = torch.logical_or(mask, (torch.arange(s_max, device=DEV) == pos)[None, None, None, :])
        kk = kc.repeat_interleave(rep, dim=1).float()
        vv = vc.repeat_interleave(rep, dim=1).float()
        ref = F.scaled_dot_product_attention(q.float()[:, :, None, :], kk, vv, attn_mask=mask).squeeze(2)
        y = ops.decode_attention(q, kc, vc, input_pos, left_pad)
        scale = float(ref.abs().max())
        assert (y.float() - ref).abs().max() < 1e-2 * scale
        if rep in (4, 8):  # the vector kernel is instantiated for 1, 2, 4 and 8 heads per kv head
            _lib.set_option("attention_no_mfma", 1)
            try:
                y_vec = ops.decode_attention(q, kc, vc, input_pos, left_pad)
            finally:
                _lib.set_option("attention_no_mfma", 0)
            assert (y.float() - y_vec.float()).abs().max() < 1e-2 * scale

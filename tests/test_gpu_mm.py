"""GPU parity of the dequant GEMV / skinny GEMM kernels against the float32 dequantize-then-matmul
oracle, through the C ABI.  Gate: max|y - y_ref| / max|y_ref| <= 1e-2 (bf16 outputs)."""

import ctypes

import numpy as np
import pytest
import torch

import easy_to_hard_amd as e2h
from easy_to_hard_amd import _lib, ops
from oracle import quant_oracle as qo
from tests.helpers import bf16_to_np, randn_bf16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2


def _int4_case(n, k, g, ikt, seed=1234):
    w = randn_bf16((n, k), std=0.02, seed=seed)
    codes, sz = qo.int4_group_quantize(bf16_to_np(w), 4, g)
    packed = qo.int4_tile_pack(codes, ikt)
    return codes, sz, torch.from_numpy(packed).to(DEV), torch.from_numpy(sz).to(torch.bfloat16).to(DEV)


def _check_int4(x, codes, sz, packed_d, sz_d, g, tol=TOL):
    y = ops.int4_mm_direct(x.to(DEV), packed_d, g, sz_d)
    assert y.dtype == torch.bfloat16 and y.shape == (x.shape[0], codes.shape[0])
    y_ref = qo.int4_linear_fp32(bf16_to_np(x), codes, sz, g)
    err = qo.normwise_rel_err(bf16_to_np(y), y_ref)
    viol = qo.elementwise_violations(bf16_to_np(y), y_ref)
    assert err <= tol, (err, viol)
    assert viol == 0.0, viol
    return y, err


@pytest.mark.parametrize("g", [32, 64, 128, 256])
@pytest.mark.parametrize("ikt", [2, 4, 8])
def test_int4_mm_all_geometries(g, ikt):
    n, k = 48, 512
    codes, sz, packed_d, sz_d = _int4_case(n, k, g, ikt, seed=g * 10 + ikt)
    for m in (1, 3, 16, 17, 32, 33, 64, 100):
        x = randn_bf16((m, k), seed=m)
        _check_int4(x, codes, sz, packed_d, sz_d, g)


def test_int4_mm_minimum_shapes():
    for ikt in (2, 4, 8):
        for g in (32, 64, 128, 256):
            k = max(16 * ikt, g)
            codes, sz, packed_d, sz_d = _int4_case(8, k, g, ikt, seed=7)
            _check_int4(randn_bf16((1, k), seed=1), codes, sz, packed_d, sz_d, g)
            _check_int4(randn_bf16((5, k), seed=2), codes, sz, packed_d, sz_d, g)


@pytest.mark.parametrize("rows_per_wave", [16, 32, 64])
def test_int4_mm_every_tile_width(rows_per_wave):
    _lib.set_option("int4_rows_per_wave", rows_per_wave)
    try:
        for n in (8, 24, 72, 200):       # N % 16 == 8 and tile counts that do not divide evenly
            codes, sz, packed_d, sz_d = _int4_case(n, 1024, 128, 8, seed=n)
            for m in (1, 8, 32, 64):
                _check_int4(randn_bf16((m, 1024), seed=m + n), codes, sz, packed_d, sz_d, 128)
    finally:
        _lib.set_option("int4_rows_per_wave", 0)


def test_int4_mm_exact_small_integers():
    # x in {-1, 0, 1}, scale = 1, zero = 8  =>  w = q exactly, y is a small integer: any mistake in the
    # nibble order, the lane mapping or the group bookkeeping changes the result by >= 1
    n, k, g, ikt = 32, 512, 128, 8
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 16, size=(n, k), dtype=np.int32)
    sz = np.zeros((k // g, n, 2), dtype=np.float32)
    sz[..., 0] = 1.0
    sz[..., 1] = 8.0
    xs = np.zeros((7, k), dtype=np.float32)
    for i in range(7):
        idx = rng.choice(k, size=12, replace=False)       # 12 non-zeros: |y| <= 180 < 256
        xs[i, idx] = rng.choice([-1.0, 1.0], size=12)
    y = ops.int4_mm_direct(torch.from_numpy(xs).to(torch.bfloat16).to(DEV), torch.from_numpy(qo.int4_tile_pack(codes, ikt)).to(DEV),
                           g, torch.from_numpy(sz).to(torch.bfloat16).to(DEV))
    expect = xs.astype(np.int64) @ codes.T.astype(np.int64)
    assert np.abs(expect).max() < 256  # exactly representable in bf16
    np.testing.assert_array_equal(bf16_to_np(y).astype(np.int64), expect)


@pytest.mark.parametrize("shape", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_int4_mm_llama_shapes_g128(shape):
    n, k = shape
    codes, sz, packed_d, sz_d = _int4_case(n, k, 128, 8)
    worst = 0.0
    for m in (1, 4, 8, 16, 32):
        x = randn_bf16((m, k), seed=100 + m)
        y, err = _check_int4(x, codes, sz, packed_d, sz_d, 128)
        worst = max(worst, err)
        y2 = ops.int4_mm_direct(x.to(DEV), packed_d, 128, sz_d)
        assert torch.equal(y, y2), "run-to-run results must be bit identical"
    print(f"int4 g128 {n}x{k}: worst normwise rel err {worst:.3e}")


def test_int4_mm_large_m_and_linearity():
    n, k, g = 256, 1024, 64
    codes, sz, packed_d, sz_d = _int4_case(n, k, g, 8, seed=3)
    x = randn_bf16((1000, k), seed=9)
    y, _ = _check_int4(x, codes, sz, packed_d, sz_d, g)
    # rows are independent: permuting the rows of x permutes the rows of y bit for bit
    xs = x[:24]
    perm = torch.randperm(24, generator=torch.Generator().manual_seed(0))
    ya = ops.int4_mm_direct(xs.to(DEV), packed_d, g, sz_d)
    yb = ops.int4_mm_direct(xs[perm].to(DEV), packed_d, g, sz_d)
    assert torch.equal(ya[perm.to(DEV)], yb)
    # a row inside a large batch and the same row alone may use different K splits: equal up to rounding
    y1 = ops.int4_mm_direct(x[517:518].to(DEV), packed_d, g, sz_d)
    assert torch.allclose(y[517:518].float(), y1.float(), rtol=2 ** -7, atol=1e-3)
    # exact linearity in x for power-of-two scalings (same launch geometry, every rounding commutes)
    y4 = ops.int4_mm_direct((xs * 4).to(DEV), packed_d, g, sz_d)
    assert torch.equal(y4.float(), ya.float() * 4)


def test_int4_module_forward_and_error_paths():
    n, k, g = 64, 512, 128
    codes, sz, packed_d, sz_d = _int4_case(n, k, g, 8, seed=12)
    mod = e2h.WeightOnlyInt4Linear(k, n, bias=False, groupsize=g, inner_k_tiles=8, padding=False).to(DEV)
    mod.load_state_dict({"weight": packed_d, "scales_and_zeros": sz_d})
    x = randn_bf16((2, 3, k), seed=5)
    y = mod(x.to(DEV))
    assert y.shape == (2, 3, n)
    y_ref = qo.int4_linear_fp32(bf16_to_np(x).reshape(6, k), codes, sz, g).reshape(2, 3, n)
    assert qo.normwise_rel_err(bf16_to_np(y), y_ref) <= TOL
    # float32 input is cast to bf16 like the reference (:659)
    y32 = mod(x.float().to(DEV))
    assert torch.equal(y32, y)
    with pytest.raises(RuntimeError):
        ops.int4_mm_direct(x.reshape(6, k)[:, :256].contiguous().to(DEV), packed_d, g, sz_d)   # K mismatch
    with pytest.raises(RuntimeError):
        ops.int4_mm_direct(x.reshape(6, k).to(DEV), packed_d, 96, sz_d)                      # bad groupsize


def test_int4_padded_module():
    # in_features 200 is padded to 1024 (reference :623-627, :660-663): weight columns >= 200 are zero weights
    k0, n, g = 200, 16, 128
    w = randn_bf16((n, k0), std=0.02, seed=31)
    wp = torch.nn.functional.pad(w, (0, 1024 - k0))
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(wp.to(DEV), g, 8)
    mod = e2h.WeightOnlyInt4Linear(k0, n, bias=False, groupsize=g, inner_k_tiles=8, padding=True).to(DEV)
    mod.load_state_dict({"weight": packed, "scales_and_zeros": sz})
    x = randn_bf16((4, k0), seed=32)
    y = mod(x.to(DEV))
    codes, sz_ref = qo.int4_group_quantize(bf16_to_np(wp), 4, g)
    xp = np.pad(bf16_to_np(x), ((0, 0), (0, 1024 - k0)))
    assert qo.normwise_rel_err(bf16_to_np(y), qo.int4_linear_fp32(xp, codes, sz_ref, g)) <= TOL


# ------------------------------------------------------------------------------------------------
# int8
# ------------------------------------------------------------------------------------------------


def _int8_case(n, k, seed=1234):
    w = randn_bf16((n, k), std=0.02, seed=seed)
    q, s, _ = qo.int8_quantize_per_channel(w.float().numpy())
    s_bf16 = qo.bf16_round(s)
    return q, s_bf16, torch.from_numpy(q).to(DEV), torch.from_numpy(s_bf16).to(torch.bfloat16).to(DEV)


def _check_int8(x, q, s, q_d, s_d):
    y = ops.int8_mm_direct(x.to(DEV), q_d, s_d)
    y_ref = qo.int8_linear_fp32(bf16_to_np(x), q, s)
    err = qo.normwise_rel_err(bf16_to_np(y), y_ref)
    assert err <= TOL, err
    assert qo.elementwise_violations(bf16_to_np(y), y_ref) == 0.0
    return y, err


def test_int8_mm_config1():
    # benchmark configuration 1: 4096x4096 weight ~N(0, 0.02), x [8, 4096] ~N(0, 1), seed 1234
    q, s, q_d, s_d = _int8_case(4096, 4096)
    x = randn_bf16((8, 4096), seed=1235)
    y, err = _check_int8(x, q, s, q_d, s_d)
    # against the reference's own double rounding only the accumulation order differs: a flip of the first
    # rounding moves the result by at most one bf16 ulp of the intermediate (2^-7 relative) and the second
    # rounding can add one more
    y_rr = qo.int8_linear_reference_rounding(bf16_to_np(x), q, s)
    diff = np.abs(bf16_to_np(y) - y_rr)
    assert np.all(diff <= np.abs(y_rr) * 2.0 ** -6 + 1e-6)
    assert np.mean(diff == 0) > 0.95
    print(f"int8 4096x4096 M=8: normwise rel err {err:.3e}, bit-identical to reference rounding: {np.mean(diff == 0):.4f}")


@pytest.mark.parametrize("shape", [(2, 4096), (1, 64), (24, 200), (17, 1000), (130, 72), (11008, 4096), (4096, 11008)])
def test_int8_mm_shapes(shape):
    n, k = shape
    q, s, q_d, s_d = _int8_case(n, k, seed=n + k)
    for m in (1, 5, 16, 32, 64, 77):
        _check_int8(randn_bf16((m, k), seed=m), q, s, q_d, s_d)


def test_int8_mm_exact_small_integers():
    n, k = 40, 320
    rng = np.random.default_rng(1)
    q = rng.integers(-128, 128, size=(n, k), dtype=np.int8)
    q[0, :] = -128
    q[1, :] = 127
    xs = np.zeros((9, k), dtype=np.float32)
    for i in range(9):
        idx = rng.choice(k, size=2, replace=False)
        xs[i, idx] = rng.choice([-1.0, 1.0], size=2)
    s = np.ones(n, dtype=np.float32)
    y = ops.int8_mm_direct(torch.from_numpy(xs).to(torch.bfloat16).to(DEV), torch.from_numpy(q).to(DEV), torch.from_numpy(s).to(torch.bfloat16).to(DEV))
    expect = xs.astype(np.int64) @ q.T.astype(np.int64)
    np.testing.assert_array_equal(bf16_to_np(y).astype(np.int64), expect)


def test_int8_module_and_on_the_fly_handler_with_hooks():
    torch.manual_seed(0)
    lin = torch.nn.Linear(256, 48, bias=False).to(torch.bfloat16)
    lin.weight.data = randn_bf16((48, 256), std=0.02, seed=77)
    calls = []
    lin.register_forward_hook(lambda m, i, o: calls.append("post"))
    lin.register_forward_pre_hook(lambda m, i: calls.append("pre"))
    model = torch.nn.Sequential(lin).to(DEV)
    e2h.WeightOnlyInt8QuantHandler(model).convert_for_runtime_on_the_fly()
    assert isinstance(model[0], e2h.WeightOnlyInt8Linear) and model[0].weight.is_cuda
    x = randn_bf16((3, 5, 256), seed=78)
    y = model(x.to(DEV))
    assert calls == ["pre", "post"] and y.shape == (3, 5, 48)
    q, s, _ = qo.int8_quantize_per_channel(lin.weight.detach().float().cpu().numpy())
    np.testing.assert_array_equal(model[0].weight.cpu().numpy(), q)
    np.testing.assert_array_equal(bf16_to_np(model[0].scales), qo.bf16_round(s))
    y_ref = qo.int8_linear_fp32(bf16_to_np(x).reshape(15, 256), q, qo.bf16_round(s)).reshape(3, 5, 48)
    assert qo.normwise_rel_err(bf16_to_np(y), y_ref) <= TOL
    # float32 / float16 activations run the reference's own two ops (reference :428-429) with its dtype promotion
    for dt in (torch.float32, torch.float16):
        xf = x.to(dt).to(DEV)
        yf = model[0](xf)
        expect = torch.nn.functional.linear(xf, model[0].weight.to(dt)) * model[0].scales
        assert yf.dtype == torch.float32 and torch.equal(yf, expect)


# ---- gated feed-forward front half: silu(w1 x) * w3 x in one launch (reference models/model.py:343-344) ----

@pytest.mark.parametrize("m", [1, 5, 16, 17, 32, 33, 64])
@pytest.mark.parametrize("n,k,g", [(48, 512, 128), (688, 1024, 64), (200, 256, 32), (11008, 4096, 128)])
def test_int4_gate_matches_oracle_and_unfused_path(m, n, k, g):
    codes1, sz1, p1, s1 = _int4_case(n, k, g, 8, seed=n + m)
    codes2, sz2, p2, s2 = _int4_case(n, k, g, 8, seed=n + m + 7)
    x = randn_bf16((m, k), std=1.0, seed=m * 31 + g)
    xd = x.to(DEV)
    y = ops.int4_mm_silu_gate(xd, p1, s1, p2, s2, g)
    assert y.dtype == torch.bfloat16 and y.shape == (m, n)
    # float oracle of the unrounded expression
    a = qo.int4_linear_fp32(bf16_to_np(x), codes1, sz1, g).astype(np.float64)
    b = qo.int4_linear_fp32(bf16_to_np(x), codes2, sz2, g).astype(np.float64)
    ref = a / (1.0 + np.exp(-a)) * b
    # three bf16 roundings (2^-9 each) on top of the matmul gate
    assert qo.normwise_rel_err(bf16_to_np(y), ref) <= TOL
    # same accumulation order as the single-matrix kernel with one K slice: identical bits
    _lib.set_option("int4_k_slices", 1)
    try:
        ya = ops.int4_mm_direct(xd, p1, g, s1)
        yb = ops.int4_mm_direct(xd, p2, g, s2)
    finally:
        _lib.set_option("int4_k_slices", 0)
    assert torch.equal(y, ops.silu_mul(ya, yb))


def test_int4_gate_rejects_what_it_does_not_cover():
    codes, sz, p, s = _int4_case(48, 512, 128, 8)
    x = randn_bf16((65, 512), seed=3).to(DEV)
    with pytest.raises(RuntimeError):
        ops.int4_mm_silu_gate(x, p, s, p, s, 128)           # m > 64
    _, _, p4, s4 = _int4_case(48, 512, 128, 4)
    with pytest.raises(RuntimeError):
        ops.int4_mm_silu_gate(x[:4], p4, s4, p4, s4, 128)   # inner_k_tiles != 8


# ---- fused q|k|v projection + RoPE + KV-cache write (reference models/model.py:283-296, :400-412, :94-104) ----

@pytest.mark.parametrize("bsz", [1, 3, 16, 32, 40, 64])
@pytest.mark.parametrize("n_head,n_kv,d,k,g", [(4, 4, 64, 256, 32), (8, 2, 64, 512, 64), (32, 32, 128, 4096, 128), (6, 3, 128, 384, 128)])
def test_int4_rope_kv_matches_two_kernel_path_and_stock_ops(bsz, n_head, n_kv, d, k, g):
    from easy_to_hard_amd.model import apply_rotary_emb, precompute_freqs_cis

    n = (n_head + 2 * n_kv) * d
    s_max, pos = 80, 37
    codes, sz, packed_d, sz_d = _int4_case(n, k, g, 8, seed=n + bsz)
    x = randn_bf16((bsz, k), std=1.0, seed=bsz * 17 + g).to(DEV)
    gen = torch.Generator().manual_seed(n_head + d)
    kc0 = torch.randn((bsz + 1, n_kv, s_max, d), generator=gen).to(torch.bfloat16).to(DEV)
    vc0 = torch.randn((bsz + 1, n_kv, s_max, d), generator=gen).to(torch.bfloat16).to(DEV)
    freqs = precompute_freqs_cis(s_max, d, 10000, device=DEV)
    input_pos = torch.tensor([pos], device=DEV)

    kc, vc = kc0.clone(), vc0.clone()
    q = ops.int4_mm_rope_kv(x, packed_d, sz_d, g, freqs, kc, vc, input_pos, n_head, n_kv, d)

    # two-kernel path with the same accumulation order (one K slice): identical bits
    _lib.set_option("int4_k_slices", 1)
    try:
        qkv = ops.int4_mm_direct(x, packed_d, g, sz_d)
    finally:
        _lib.set_option("int4_k_slices", 0)
    kc2, vc2 = kc0.clone(), vc0.clone()
    q2 = ops.rope_kv_write(qkv, freqs, kc2, vc2, input_pos, n_head, n_kv, d)
    assert torch.equal(q, q2) and torch.equal(kc, kc2) and torch.equal(vc, vc2)
    # only position `pos` of the first bsz sequences changed
    untouched = torch.ones(s_max, dtype=torch.bool, device=DEV)
    untouched[pos] = False
    assert torch.equal(kc[:, :, untouched], kc0[:, :, untouched]) and torch.equal(kc[bsz], kc0[bsz])
    assert torch.equal(vc[:, :, untouched], vc0[:, :, untouched]) and torch.equal(vc[bsz], vc0[bsz])

    # stock ops on the oracle's projection (float32 oracle rounded to bf16 may differ from the kernel's in the last
    # bit, so the comparison is by tolerance)
    y_ref = torch.from_numpy(qo.int4_linear_fp32(bf16_to_np(x.cpu()), codes, sz, g)).to(torch.bfloat16).to(DEV)
    qr, kr, vr = y_ref.view(bsz, 1, -1).split([n_head * d, n_kv * d, n_kv * d], dim=-1)
    fc = freqs[input_pos]
    q_ref = apply_rotary_emb(qr.view(bsz, 1, n_head, d), fc).squeeze(1)
    k_ref = apply_rotary_emb(kr.view(bsz, 1, n_kv, d), fc).squeeze(1)
    scale = float(y_ref.float().abs().max())
    assert (q.float() - q_ref.float()).abs().max() <= TOL * scale
    assert (kc[:bsz, :, pos].float() - k_ref.float()).abs().max() <= TOL * scale
    assert (vc[:bsz, :, pos].float() - vr.view(bsz, n_kv, d).float()).abs().max() <= TOL * scale


def test_int4_rope_kv_ignores_out_of_range_position():
    n_head, n_kv, d, k, g, bsz, s_max = 4, 4, 64, 256, 32, 2, 16
    _, _, packed_d, sz_d = _int4_case((n_head + 2 * n_kv) * d, k, g, 8)
    from easy_to_hard_amd.model import precompute_freqs_cis

    x = randn_bf16((bsz, k), seed=1).to(DEV)
    kc0 = torch.zeros((bsz, n_kv, s_max, d), dtype=torch.bfloat16, device=DEV)
    kc, vc = kc0.clone(), kc0.clone()
    freqs = precompute_freqs_cis(s_max, d, 10000, device=DEV)
    ops.int4_mm_rope_kv(x, packed_d, sz_d, g, freqs, kc, vc, torch.tensor([s_max], device=DEV), n_head, n_kv, d)
    torch.cuda.synchronize()
    assert torch.equal(kc, kc0) and torch.equal(vc, kc0)


def test_nan_and_inf_activations_propagate_to_their_rows_only():
    """A NaN / inf in one row of x must show up as NaN / inf in that row's outputs (torch semantics) and nowhere else."""
    codes, sz, packed_d, sz_d = _int4_case(64, 512, 128, 8)
    x = randn_bf16((8, 512), seed=9)
    x[2, 100] = float("nan")
    x[5, 7] = float("inf")
    y = ops.int4_mm_direct(x.to(DEV), packed_d, 128, sz_d).float().cpu()
    assert torch.isnan(y[2]).all()
    assert not torch.isfinite(y[5]).any()
    keep = [0, 1, 3, 4, 6, 7]
    assert torch.isfinite(y[keep]).all()
    q = torch.randint(-128, 128, (64, 512), dtype=torch.int8).to(DEV)
    s = torch.ones(64, dtype=torch.bfloat16, device=DEV)
    y8 = ops.int8_mm_direct(x.to(DEV), q, s).float().cpu()
    assert torch.isnan(y8[2]).all() and not torch.isfinite(y8[5]).any() and torch.isfinite(y8[keep]).all()


@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("m", [65, 130, 257])
def test_int4_many_rows_group_sum_prepass_matches_in_kernel_sums(m, g):
    """Calls with more than 64 rows take the group sums of x from a pre-pass; the in-kernel form (option
    int4_no_xsum) must agree to float32 summation-order noise, and both with the oracle."""
    n, k = 272, 1024
    codes, sz, packed_d, sz_d = _int4_case(n, k, g, 8, seed=m + g)
    x = randn_bf16((m, k), std=1.0, seed=m)
    y, _ = _check_int4(x, codes, sz, packed_d, sz_d, g)
    _lib.set_option("int4_no_xsum", 1)
    try:
        y2, _ = _check_int4(x, codes, sz, packed_d, sz_d, g)
    finally:
        _lib.set_option("int4_no_xsum", 0)
    diff = (y.float() - y2.float()).abs().max().item()
    assert diff <= 2.0 ** -7 * y2.float().abs().max().item()  # at most one bf16 step of the largest output


@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("m,n,k", [(65, 8, 128), (130, 272, 1024), (257, 136, 384), (512, 4096, 4096)])
def test_int4_gemm32_tiles_match_oracle_and_16x16_kernel(m, n, k, g):
    """The 32x32-tile kernel (many rows) against the oracle and against the 16x16-tile kernel on the same inputs:
    ragged M and N (not multiples of 128 / 32), a single chunk, odd numbers of groups."""
    if k == 4096 and g != 128:
        pytest.skip("large shape: one group size only")
    codes, sz, packed_d, sz_d = _int4_case(n, k, g, 8, seed=m + n + g)
    x = randn_bf16((m, k), std=1.0, seed=m + 1)
    _lib.set_option("int4_gemm32_min_rows", 65)
    try:
        y, _ = _check_int4(x, codes, sz, packed_d, sz_d, g)
        # exact small-integer case: x in {-1, 0, 1}, every partial sum is an integer well inside float32
        xi = torch.randint(-1, 2, (m, k), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
        yi = ops.int4_mm_direct(xi.to(DEV), packed_d, g, sz_d)
    finally:
        _lib.set_option("int4_gemm32_min_rows", 0)
    _lib.set_option("int4_no_gemm32", 1)
    try:
        y2, _ = _check_int4(x, codes, sz, packed_d, sz_d, g)
        yi2 = ops.int4_mm_direct(xi.to(DEV), packed_d, g, sz_d)
    finally:
        _lib.set_option("int4_no_gemm32", 0)
    assert (y.float() - y2.float()).abs().max().item() <= 2.0 ** -7 * y2.float().abs().max().item()
    assert (yi.float() - yi2.float()).abs().max().item() <= 2.0 ** -7 * yi2.float().abs().max().item()


@pytest.mark.parametrize("tile,waves,wave_cols", [(128, 0, 0), (256, 0, 0), (256, 8, 0), (256, 4, 2), (256, 4, 4)])
@pytest.mark.parametrize("m,n,k", [(65, 1, 128), (130, 272, 1024), (257, 136, 384), (512, 4096, 4096), (300, 2, 4096), (700, 520, 640)])
def test_int8_gemm32_tiles_match_oracle_and_16x16_kernel(m, n, k, tile, waves, wave_cols):
    """The 32x32-tile int8 kernels (many rows; 128 x 256 and 256 x 256 outputs per workgroup, the latter with eight or four waves) against the oracle, the
    reference's two-rounding form and the 16x16-tile kernel: ragged M and N (incl. the 2-row reward head), a single
    chunk, odd chunk counts, and rows with extreme codes (-128 / 127) so that the +128 offset and its correction are
    exercised at both ends."""
    q, s, q_d, s_d = _int8_case(n, k, seed=m + n)
    q = q.copy()
    q[0, :4] = (-128, 127, -128, 127)
    q[-1, -4:] = (127, -128, -127, 126)
    q_d = torch.from_numpy(q).to(DEV)
    x = randn_bf16((m, k), std=1.0, seed=m + 2)
    _lib.set_option("int4_gemm32_min_rows", 65)
    _lib.set_option("int8_gemm_tile", tile)
    _lib.set_option("int8_gemm_waves", waves)
    _lib.set_option("int8_gemm_wave_cols", wave_cols)
    try:
        y, _ = _check_int8(x, q, s, q_d, s_d)
        xi = torch.randint(-1, 2, (m, k), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
        yi = ops.int8_mm_direct(xi.to(DEV), q_d, s_d)
    finally:
        _lib.set_option("int4_gemm32_min_rows", 0)
        _lib.set_option("int8_gemm_tile", 0)
        _lib.set_option("int8_gemm_waves", 0)
        _lib.set_option("int8_gemm_wave_cols", 0)
    _lib.set_option("int4_no_gemm32", 1)
    try:
        y2, _ = _check_int8(x, q, s, q_d, s_d)
        yi2 = ops.int8_mm_direct(xi.to(DEV), q_d, s_d)
    finally:
        _lib.set_option("int4_no_gemm32", 0)
    assert (y.float() - y2.float()).abs().max().item() <= 2.0 ** -6 * y2.float().abs().max().item()
    # integer activations: every partial sum is an exact integer below 2^24, both kernels must agree bit for bit
    assert torch.equal(yi, yi2)
    y_rr = qo.int8_linear_reference_rounding(bf16_to_np(xi), q, s)
    assert np.array_equal(bf16_to_np(yi), y_rr)


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(2304, 8448, 128), (2304, 8448, 256), (4100, 4104, 384)])
def test_int8_many_row_kernel_walks_several_tiles_per_workgroup(m, n, k):
    """More 256 x 256 tiles than CUs, so that workgroups of the default many-row int8 kernel take a second tile while the
    chunk pipeline runs on: the shortest K (two and four 64-wide chunks: the loads aimed two chunks ahead are already in
    the next tile when a tile starts), a column-block count that leaves some XCDs a slot without a tile (33 and 17
    blocks over 8 XCDs), ragged M and N.  Integer activations: every partial sum is an exact integer, so the result
    must equal the reference's two-rounding form bit for bit and the 16x16-tile kernel's."""
    q, s, q_d, s_d = _int8_case(n, k, seed=m + k)
    xi = torch.randint(-2, 3, (m, k), generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    _lib.set_option("int8_gemm_tile", 256)
    try:
        yi = ops.int8_mm_direct(xi.to(DEV), q_d, s_d)
    finally:
        _lib.set_option("int8_gemm_tile", 0)
    _lib.set_option("int4_no_gemm32", 1)
    try:
        yi2 = ops.int8_mm_direct(xi.to(DEV), q_d, s_d)
    finally:
        _lib.set_option("int4_no_gemm32", 0)
    assert torch.equal(yi, yi2)
    rows = np.r_[0:64, 255:258, m - 70:m]
    y_rr = qo.int8_linear_reference_rounding(bf16_to_np(xi)[rows], q, s)
    assert np.array_equal(bf16_to_np(yi)[rows], y_rr)


@pytest.mark.gpu
def test_int8_many_rows_at_the_reward_scoring_size():
    """One linear of the scoring configuration at its full row count (64 x 768 = 49152 rows, 4096 x 4096 weight):
    sampled rows against the oracle, row-permutation equivariance (a row's result does not depend on where in the
    batch it sits: bit for bit), and rows of small integers against the exact integer product."""
    m, n, k = 49152, 4096, 4096
    q, s, q_d, s_d = _int8_case(n, k, seed=77)
    gen = torch.Generator().manual_seed(78)
    x = (torch.randn(4096, k, generator=gen) * 1.0).to(torch.bfloat16)
    x = x.repeat(m // 4096, 1)                          # 12 copies of 4096 distinct rows
    x[-3:] = torch.randint(-2, 3, (3, k), generator=gen).to(torch.bfloat16)   # exact rows at the very end
    x_d = x.to(DEV)
    y = ops.int8_mm_direct(x_d, q_d, s_d)
    assert y.shape == (m, n) and bool(torch.isfinite(y.float()).all())
    rows = [0, 1, 255, 256, 4095, 4096, 24575, 49151 - 3, 49151]
    y_ref = qo.int8_linear_fp32(bf16_to_np(x[rows]), q, s)
    assert qo.normwise_rel_err(bf16_to_np(y[rows].cpu()), y_ref) <= TOL
    # copies of the same input row give the same output row wherever they sit
    assert torch.equal(y[:4096], y[4096:8192]) and torch.equal(y[:4096], y[4096 * 5:4096 * 6])
    perm = torch.randperm(m, generator=gen).to(DEV)
    assert torch.equal(ops.int8_mm_direct(x_d[perm], q_d, s_d), y[perm])
    y_int = qo.int8_linear_reference_rounding(bf16_to_np(x[-3:]), q, s)
    assert np.array_equal(bf16_to_np(y[-3:].cpu()), y_int)

@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("m,n,k", [(300, 264, 512), (1000, 520, 256), (257, 136, 768), (257, 136, 384), (512, 4096, 4096)])
def test_int4_gemm128_dequantizing_kernel_matches_oracle_and_32x32_tile_kernel(m, n, k, g):
    """The 256 x 256-output kernel (weights dequantized to bfloat16 on the way into the matrix cores, the reference
    kernel's arithmetic) against the oracle and against the 128-row kernel (exact products, scale applied in float32):
    ragged M and N, one and several trips of its two-block loop, every group size; K = 384 is not a multiple of 256 and
    stays on the 128-row kernel.  The two kernels differ by the bfloat16 rounding of each weight (2^-9 relative, random
    sign) on top of the output rounding."""
    if k == 4096 and g != 128:
        pytest.skip("large shape: one group size only")
    codes, sz, packed_d, sz_d = _int4_case(n, k, g, 8, seed=m + n + g)
    x = randn_bf16((m, k), std=1.0, seed=m + 2)
    _lib.set_option("int4_gemm32_min_rows", 65)
    try:
        _lib.set_option("int4_gemm_tile", 256)
        y, _ = _check_int4(x, codes, sz, packed_d, sz_d, g)
        _lib.set_option("int4_gemm_tile", 128)
        y2, _ = _check_int4(x, codes, sz, packed_d, sz_d, g)
    finally:
        _lib.set_option("int4_gemm_tile", 0)
        _lib.set_option("int4_gemm32_min_rows", 0)
    bound = 2.0 ** -6 * y2.float().abs().max().item()
    assert (y.float() - y2.float()).abs().max().item() <= bound
    if k % 256:
        assert torch.equal(y, y2)


def test_int4_gemm128_with_weights_that_dequantize_exactly():
    """Scales that are powers of two and zeros that are small multiples of them make every s * (q - 8) + z a bfloat16
    value, and x in {-1, 0, 1} makes every product and partial sum exact: the dequantizing kernel must then return
    bfloat16(exact sum) for every element, whatever the order of its additions."""
    m, n, k, g = 300, 264, 512, 64
    gen = torch.Generator().manual_seed(21)
    codes = torch.randint(0, 16, (n, k), generator=gen, dtype=torch.int32)
    scales = torch.pow(2.0, torch.randint(-6, -2, (k // g, n), generator=gen).float())
    zeros = scales * torch.randint(-8, 9, (k // g, n), generator=gen).float()
    sz = torch.stack([scales, zeros], dim=-1).to(torch.bfloat16)
    x = torch.randint(-1, 2, (m, k), generator=gen).to(torch.bfloat16)
    w = (codes.float() - 8) * scales.t().repeat_interleave(g, 1) + zeros.t().repeat_interleave(g, 1)
    want = (x.double() @ w.double().t()).to(torch.bfloat16)
    packed_d = ops.int4_pack(codes.to(DEV), 8)
    _lib.set_option("int4_gemm_tile", 256)
    try:
        got = ops.int4_mm_direct(x.to(DEV), packed_d, g, sz.to(DEV))
    finally:
        _lib.set_option("int4_gemm_tile", 0)
    assert torch.equal(got.cpu(), want)


def _two_fma_weights(codes, sz, g):
    """The dequantizing kernel's conversion restated in numpy: c = float32(z - 136 s), w = bf16(float32((128 + q) s + c)).
    Each float32 FMA is formed in float64 (exact for bfloat16 s, z of these magnitudes: products of two 8-bit
    significands, sums whose exponents lie within 2^29 of each other) and rounded once to float32."""
    s = np.repeat(sz[..., 0].astype(np.float64).T, g, axis=1)  # [n, k]
    z = np.repeat(sz[..., 1].astype(np.float64).T, g, axis=1)
    c = (z - 136.0 * s).astype(np.float32)
    w = ((128.0 + codes.astype(np.float64)) * s + c.astype(np.float64)).astype(np.float32)
    return qo.bf16_round(w), c


@pytest.mark.parametrize("g", [32, 64, 128])
def test_int4_gemm128_converted_weights_read_back_through_identity_activations(g):
    """x = identity makes y[m][n] the kernel's own bfloat16 weight (one product 1 * w, every other term zero).  With
    random bfloat16 (scale, zero) pairs -- not the benign ones a quantizer emits -- the weights must equal the two-FMA
    conversion bit for bit, lie within one bfloat16 ulp of the single-rounded bf16(s (q - 8) + z), and equal it
    wherever z - 136 s is a float32 value."""
    n, k = 264, 256
    gen = torch.Generator().manual_seed(77 + g)
    codes = torch.randint(0, 16, (n, k), generator=gen, dtype=torch.int32)
    scales = (torch.rand((k // g, n), generator=gen) * 0.02 + 1e-4).to(torch.bfloat16)
    zeros = (torch.randn((k // g, n), generator=gen) * 0.05).to(torch.bfloat16)
    sz = torch.stack([scales, zeros], dim=-1)
    x = torch.eye(k, dtype=torch.bfloat16)
    packed_d = ops.int4_pack(codes.to(DEV), 8)
    _lib.set_option("int4_gemm_tile", 256)
    try:
        got = ops.int4_mm_direct(x.to(DEV), packed_d, g, sz.to(DEV))
    finally:
        _lib.set_option("int4_gemm_tile", 0)
    got = bf16_to_np(got.cpu()).T.astype(np.float64)  # [n, k]
    want, c = _two_fma_weights(codes.numpy(), bf16_to_np(sz), g)
    assert np.array_equal(got, want.astype(np.float64))
    s64 = np.repeat(bf16_to_np(sz)[..., 0].astype(np.float64).T, g, axis=1)
    z64 = np.repeat(bf16_to_np(sz)[..., 1].astype(np.float64).T, g, axis=1)
    exact = s64 * (codes.numpy().astype(np.float64) - 8.0) + z64  # exact in float64 at these magnitudes
    single = _bf16_round_f64(exact)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 1e-300))) - 7)
    c_mag = 136.0 * np.abs(s64) + np.abs(z64)
    # half a bfloat16 ulp of the exact value from the final rounding, and the two float32 roundings (of z - 136 s, of
    # the FMA's result) in front of it, each at most 2^-24 of a value no larger than |z| + 136 |s| + 143 |s|
    assert np.all(np.abs(got - exact) <= 0.5 * ulp + 2.0 ** -22 * c_mag)
    differs = got != single
    assert differs.mean() < 0.01  # near-ties of the last rounding and nearly cancelling weights only
    ordinary = np.abs(exact) >= 2.0 ** -6 * c_mag
    assert np.all(np.abs(got - single)[ordinary] <= ulp[ordinary] * (1 + 2.0 ** -7))


def _bf16_round_f64(x):
    """float64 -> nearest bfloat16 value (ties to even), as float64, in one rounding (normal magnitudes only)."""
    u = np.ascontiguousarray(x, dtype=np.float64).view(np.uint64)
    drop = np.uint64(52 - 7)
    lsb = (u >> drop) & np.uint64(1)
    r = ((u + ((np.uint64(1) << (drop - np.uint64(1))) - np.uint64(1)) + lsb) >> drop) << drop
    return r.view(np.float64)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["int8", "int4"])
def test_many_row_kernels_with_an_output_that_is_only_2_byte_aligned(mode):
    """The 32x32-tile kernels write 16-byte pieces of output rows; the C ABI only promises a 2-byte aligned y, so an
    output that starts 2 bytes into an allocation must take the element-wise stores and give the very same values."""
    m, n, k, g = 300, 264, 512, 128
    x = randn_bf16((m, k), std=1.0, seed=5).to(DEV)
    buf = torch.zeros(m * n + 8, dtype=torch.bfloat16, device=DEV)
    ws = ops._workspace(x.device)
    lib = ops._lib_for(x)
    _lib.set_option("int4_gemm32_min_rows", 65)
    try:
        if mode == "int8":
            q, s, q_d, s_d = _int8_case(n, k, seed=11)
            y_ref = ops.int8_mm_direct(x, q_d, s_d)
            for tile in (128, 256):
                _lib.set_option("int8_gemm_tile", tile)
                buf.zero_()
                rc = lib.e2h_int8_mm(ops._ptr(x), ops._ptr(q_d), ops._ptr(s_d), ctypes.c_void_p(buf.data_ptr() + 2), m, n, k, ops._ptr(ws), ws.numel(), ops._stream(x))
                _lib.check(rc, "e2h_int8_mm")
                assert torch.equal(buf[1:1 + m * n].view(m, n), y_ref)
                assert buf[0].item() == 0 and buf[1 + m * n:].abs().max().item() == 0
        else:
            codes, sz, packed_d, sz_d = _int4_case(n, k, g, 8, seed=12)
            for tile in (128, 256):
                _lib.set_option("int4_gemm_tile", tile)
                buf.zero_()
                y_ref = ops.int4_mm_direct(x, packed_d, g, sz_d)
                rc = lib.e2h_int4_mm(ops._ptr(x), ops._ptr(packed_d), ops._ptr(sz_d), ctypes.c_void_p(buf.data_ptr() + 2), m, n, k, g, 8, ops._ptr(ws),
                                     ws.numel(), ops._stream(x))
                _lib.check(rc, "e2h_int4_mm")
                assert torch.equal(buf[1:1 + m * n].view(m, n), y_ref)
                assert buf[0].item() == 0 and buf[1 + m * n:].abs().max().item() == 0
    finally:
        _lib.set_option("int4_gemm32_min_rows", 0)
        _lib.set_option("int8_gemm_tile", 0)
        _lib.set_option("int4_gemm_tile", 0)


@pytest.mark.gpu
@pytest.mark.parametrize("m", [1, 32])
def test_int4_mm_matches_the_stock_rocm_op_on_identical_codes(m):
    """PyTorch-ROCm ships its own aten._weight_int4pack_mm (another packed layout, same arithmetic: the op the reference
    calls at models/quantize.py:448-450).  Fed the same codes and (scale, zero) pairs it must agree with this library to
    bfloat16 rounding; skipped where the installed build has no kernel for this GPU."""
    dev = "cuda:0"
    gen = torch.Generator().manual_seed(99)
    n, k, g, ikt = 512, 1024, 128, 8
    w = (torch.randn((n, k), generator=gen) * 0.02).to(torch.bfloat16).to(dev)
    x = torch.randn((m, k), generator=gen).to(torch.bfloat16).to(dev)
    packed, sz = e2h.prepare_int4_weight_and_scales_and_zeros(w, g, ikt)
    codes = ops.int4_unpack(packed)
    two_per_byte = ((codes[:, ::2] << 4) | codes[:, 1::2]).to(torch.uint8)
    try:
        stock_packed = torch.ops.aten._convert_weight_to_int4pack(two_per_byte, ikt)
        y_stock = torch.ops.aten._weight_int4pack_mm(x, stock_packed, g, sz).float()
        torch.cuda.synchronize()
    except (RuntimeError, NotImplementedError) as exc:
        pytest.skip(f"stock aten._weight_int4pack_mm unavailable here: {exc}")
    y = ops.int4_mm_direct(x, packed, g, sz).float()
    assert float((y - y_stock).abs().max() / y_stock.abs().max()) <= 1e-2


# ---- int8 forms of the two fused decode-step launches ----

@pytest.mark.parametrize("m", [1, 5, 16, 17, 32, 33, 64])
@pytest.mark.parametrize("n,k", [(48, 512), (690, 1024), (11008, 4096)])
def test_int8_gate_matches_oracle_and_unfused_path(m, n, k):
    q1, s1, q1_d, s1_d = _int8_case(n, k, seed=n + m)
    q2, s2, q2_d, s2_d = _int8_case(n, k, seed=n + m + 7)
    x = randn_bf16((m, k), std=1.0, seed=m * 31)
    xd = x.to(DEV)
    y = ops.int8_mm_silu_gate(xd, q1_d, s1_d, q2_d, s2_d)
    assert y.dtype == torch.bfloat16 and y.shape == (m, n)
    a = qo.int8_linear_fp32(bf16_to_np(x), q1, s1).astype(np.float64)
    b = qo.int8_linear_fp32(bf16_to_np(x), q2, s2).astype(np.float64)
    assert qo.normwise_rel_err(bf16_to_np(y), a / (1.0 + np.exp(-a)) * b) <= TOL
    # same accumulation order as the single-matrix kernel with one K slice: identical bits
    _lib.set_option("int8_k_slices", 1)
    try:
        ya = ops.int8_mm_direct(xd, q1_d, s1_d)
        yb = ops.int8_mm_direct(xd, q2_d, s2_d)
    finally:
        _lib.set_option("int8_k_slices", 0)
    assert torch.equal(y, ops.silu_mul(ya, yb) if (m * n) % 8 == 0 else torch.nn.functional.silu(ya) * yb)
    with pytest.raises(RuntimeError):
        ops.int8_mm_silu_gate(randn_bf16((65, k), seed=3).to(DEV), q1_d, s1_d, q2_d, s2_d)  # more than 64 rows


@pytest.mark.parametrize("bsz", [1, 3, 16, 32, 40, 64])
@pytest.mark.parametrize("n_head,n_kv,d,k", [(4, 4, 64, 256), (8, 2, 64, 512), (32, 32, 128, 4096), (6, 3, 128, 384)])
def test_int8_rope_kv_matches_two_kernel_path(bsz, n_head, n_kv, d, k):
    from easy_to_hard_amd.model import precompute_freqs_cis

    n = (n_head + 2 * n_kv) * d
    s_max, pos = 80, 37
    _, _, q_d, s_d = _int8_case(n, k, seed=n + bsz)
    x = randn_bf16((bsz, k), std=1.0, seed=bsz * 17).to(DEV)
    gen = torch.Generator().manual_seed(n_head + d)
    kc0 = torch.randn((bsz + 1, n_kv, s_max, d), generator=gen).to(torch.bfloat16).to(DEV)
    vc0 = torch.randn((bsz + 1, n_kv, s_max, d), generator=gen).to(torch.bfloat16).to(DEV)
    freqs = precompute_freqs_cis(s_max, d, 10000, device=DEV)
    input_pos = torch.tensor([pos], device=DEV)
    kc, vc = kc0.clone(), vc0.clone()
    q = ops.int8_mm_rope_kv(x, q_d, s_d, freqs, kc, vc, input_pos, n_head, n_kv, d)
    _lib.set_option("int8_k_slices", 1)
    try:
        qkv = ops.int8_mm_direct(x, q_d, s_d)
    finally:
        _lib.set_option("int8_k_slices", 0)
    kc2, vc2 = kc0.clone(), vc0.clone()
    q2 = ops.rope_kv_write(qkv, freqs, kc2, vc2, input_pos, n_head, n_kv, d)
    assert torch.equal(q, q2) and torch.equal(kc, kc2) and torch.equal(vc, vc2)
    # a position outside the cache writes nothing
    kc3, vc3 = kc0.clone(), vc0.clone()
    ops.int8_mm_rope_kv(x, q_d, s_d, freqs, kc3, vc3, torch.tensor([s_max], device=DEV), n_head, n_kv, d)
    assert torch.equal(kc3, kc0) and torch.equal(vc3, vc0)

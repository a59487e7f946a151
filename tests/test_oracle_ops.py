"""Pins oracle/ops.py against closed forms, brute force and invariants (CPU only)."""

import math

import numpy as np
import torch

from oracle import fp8, ops
from oracle.inputs import attn_case, ffn_case, gemm_case

BF16 = torch.bfloat16


def _codes(vals):
    """e4m3fn tensor holding exactly ``vals`` (all representable)."""
    t = torch.tensor(vals, dtype=torch.float32)
    w8 = t.to(torch.float8_e4m3fn)
    assert torch.equal(w8.float(), t)
    return w8


# ------------------------------------------------------------------ linear / FFN
def test_lin_by_hand():
    x = torch.tensor([[1.0, 2.0]], dtype=BF16)
    w8 = _codes([[1.0, 0.5], [2.0, -1.0], [448.0, 0.0]])
    s = torch.tensor([0.5, 2.0, 0.25])
    y = ops.lin_fp8w(x, w8, s)
    assert y.dtype == BF16 and y.tolist() == [[1.0, 0.0, 112.0]]


def test_lin_scale_is_applied_to_the_accumulator_not_the_weight():
    # with scale 1/3 the two orders differ in fp32; the oracle must follow acc * s
    x, w8, _ = gemm_case(4, 64, 32, seed=3)
    s = torch.full((32,), 1.0 / 3.0)
    acc = x.float() @ w8.float().t()
    assert torch.equal(ops.lin_fp8w(x, w8, s), (acc * s).to(BF16))


def test_lin_against_float64_and_linearity():
    x, w8, s = gemm_case(50, 720, 96)
    y = ops.lin_fp8w(x, w8, s).double()
    ref = ops.lin_fp8w_f64(x, w8, s)
    # one bf16 rounding (2^-9 relative) plus fp32 accumulation noise
    assert float(((y - ref).abs() / (ref.abs() + 1e-3)).max()) < 2.0**-8
    # exact linearity in power-of-two scalings of x and of the scale
    assert torch.equal(ops.lin_fp8w(x * 2, w8, s), (ops.lin_fp8w(x, w8, s).float() * 2).to(BF16))
    assert torch.equal(ops.lin_fp8w(x, w8, s * 4), (ops.lin_fp8w(x, w8, s).float() * 4).to(BF16))
    # permuting output channels permutes columns
    perm = torch.randperm(96, generator=torch.Generator().manual_seed(0))
    assert torch.equal(ops.lin_fp8w(x, w8[perm], s[perm]), ops.lin_fp8w(x, w8, s)[:, perm])


def test_activation_closed_forms():
    z = torch.linspace(-6, 6, 101, dtype=torch.float64)
    silu = z / (1 + torch.exp(-z))
    gelu = 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z**3)))
    assert torch.allclose(ops.act_fn("silu", z), silu, atol=1e-12)
    assert torch.allclose(ops.act_fn("gelu_tanh", z), gelu, atol=1e-12)


def test_gated_ffn_by_hand_and_against_float64():
    # by hand: K=2, I=2; gate = [1, -1], up = [2, 3], h = silu(g)*u, y = h . Wd
    x = torch.tensor([[1.0, 0.0]], dtype=BF16)
    wg = _codes([[1.0, 0.0], [-1.0, 0.0]])
    wu = _codes([[2.0, 0.0], [3.0, 0.0]])
    wd = _codes([[1.0, 1.0], [1.0, -1.0]])
    one = torch.ones(2)
    y = ops.gated_ffn(x, wg, one, wu, one, wd, one, "silu")
    sg = torch.tensor([1.0, -1.0])
    h = (torch.nn.functional.silu(sg).to(BF16) * torch.tensor([2.0, 3.0], dtype=BF16)).float()
    assert torch.equal(y.float(), torch.stack([h.sum(), h[0] - h[1]]).to(BF16).float()[None])
    # config-1 shape against a float64 evaluation of the same formula
    for act in ("silu", "gelu_tanh"):
        xx, wg8, sg_, wu8, su_, wd8, sd_ = ffn_case(m=8, k=720, i=2048, seed=0)
        yy = ops.gated_ffn(xx, wg8, sg_, wu8, su_, wd8, sd_, act).double()
        g64 = ops.lin_fp8w_f64(xx, wg8, sg_)
        u64 = ops.lin_fp8w_f64(xx, wu8, su_)
        h64 = ops.act_fn(act, g64) * u64
        y64 = h64 @ fp8.dequantize_rows(wd8, sd_).double().t()
        assert float((yy - y64).abs().max()) < 2e-2 * float(y64.abs().max()) + 1e-3


# ------------------------------------------------------------------ norms
def test_rms_norm_llama_closed_form_and_dtypes():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 720, generator=g)
    w = (torch.rand(720, generator=g) + 0.5).to(BF16)
    ref = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5) * w.double()
    out32 = ops.rms_norm_llama(x, w, 1e-5)
    assert out32.dtype == torch.float32  # bf16 weight * fp32 activations promotes
    assert torch.allclose(out32.double(), ref, rtol=1e-5, atol=1e-6)
    out16 = ops.rms_norm_llama(x.to(BF16), w, 1e-5)
    assert out16.dtype == BF16
    # bf16 path rounds the normalised value first, then multiplies in bf16
    xb = x.to(BF16).float()
    n = (xb * torch.rsqrt(xb.pow(2).mean(-1, keepdim=True) + 1e-5)).to(BF16)
    assert torch.equal(out16, w * n)


def test_gemma_rms_norm_plain_and_adaptive():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, 6, 1024, generator=g).to(BF16)
    w = torch.randn(1024, generator=g) * 0.1
    base = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-6)
    out, gate = ops.gemma_rms_norm(x, 1e-6, weight=w)
    assert gate is None and out.dtype == BF16
    assert torch.allclose(out.double(), base * (1 + w.double()), rtol=2**-7, atol=1e-3)
    mod = torch.randn(1, 3 * 1024, generator=g) * 0.1
    out, gate = ops.gemma_rms_norm(x, 1e-6, modulation=mod)
    sc, sh, gt = mod.double().chunk(3, dim=-1)
    assert torch.allclose(out.double(), base * (1 + sc[:, None]) + sh[:, None], rtol=2**-7, atol=1e-2)
    assert gate.dtype == BF16 and torch.equal(gate, gt.to(BF16)[:, None])
    out2, gate2 = ops.gemma_rms_norm(x, 1e-6, modulation=mod[:, : 2 * 1024])
    assert gate2 is None and torch.equal(out2, out)


# ------------------------------------------------------------------ rotary
def test_rope_half_split_properties():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, 7, 3, 64, generator=g)
    pos = torch.tensor([[0, 1, 2, 5, 100, 241, 290]])
    y = ops.rope_half_split(x, pos)
    assert torch.equal(y[:, 0], x[:, 0])  # position 0 is the identity
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)  # rotations preserve norms
    # one-hot in slot i rotates into (i, i + D/2) by pos / base**(2i/D)
    for i in (0, 5, 31):
        e = torch.zeros(1, 1, 1, 64)
        e[..., i] = 1.0
        r = ops.rope_half_split(e, torch.tensor([[7]]))[0, 0, 0]
        ang = 7.0 / (10000.0 ** (2 * i / 64))
        assert abs(float(r[i]) - math.cos(ang)) < 1e-6 and abs(float(r[i + 32]) - math.sin(ang)) < 1e-6
        assert float(r.abs().sum()) - abs(float(r[i])) - abs(float(r[i + 32])) < 1e-7
    # relative-position property of the q.k score
    q = torch.randn(1, 1, 1, 64, generator=g)
    k = torch.randn(1, 1, 1, 64, generator=g)
    s1 = (ops.rope_half_split(q, torch.tensor([[10]])) * ops.rope_half_split(k, torch.tensor([[4]]))).sum()
    s2 = (ops.rope_half_split(q, torch.tensor([[16]])) * ops.rope_half_split(k, torch.tensor([[10]]))).sum()
    assert abs(float(s1 - s2)) < 1e-4
    assert ops.rope_half_split(x.to(BF16), pos).dtype == BF16


def test_gemma_rope_uses_bf16_rounded_frequencies():
    pos = torch.tensor([[0, 1, 37]])
    cos, sin = ops.gemma_rope_cos_sin(256, pos, torch.float32)
    assert cos.shape == (1, 3, 256)
    for i in (1, 17, 127):
        inv = torch.tensor(1.0 / (10000.0 ** (2 * i / 256))).to(BF16).float()
        assert abs(float(cos[0, 2, i]) - math.cos(37 * float(inv))) < 1e-6
        assert float(cos[0, 2, i]) == float(cos[0, 2, i + 128])  # emb = cat(freqs, freqs)
        assert abs(float(sin[0, 1, i]) - math.sin(float(inv))) < 1e-6
    x = torch.randn(1, 2, 3, 256, generator=torch.Generator().manual_seed(0))
    y = ops.gemma_apply_rope(x, cos, sin)
    assert torch.equal(y[:, :, 0], x[:, :, 0])
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)
    # pairs (i, i + D/2): y_i = x_i cos - x_{i+h} sin
    i = 9
    exp = x[0, 0, 2, i] * cos[0, 2, i] - x[0, 0, 2, i + 128] * sin[0, 2, i]
    assert abs(float(y[0, 0, 2, i] - exp)) < 1e-6


# ------------------------------------------------------------------ masks / time
def test_make_att_2d_masks_brute_force():
    pad = torch.tensor([[1, 1, 0, 1, 1, 1]], dtype=torch.bool)
    att = torch.tensor([[0, 0, 0, 1, 0, 1]])
    got = ops.make_att_2d_masks(pad, att)[0]
    c = np.cumsum(att[0].numpy())
    for i in range(6):
        for j in range(6):
            want = bool(c[j] <= c[i]) and bool(pad[0, i]) and bool(pad[0, j])
            assert bool(got[i, j]) == want


def test_suffix_mask_matches_the_two_policies():
    pad = torch.tensor([1, 0, 1, 1], dtype=torch.bool)
    for att_suf, mode in (([1] * 5, ops.MASK_CAUSAL), ([1, 0, 0, 0, 0], ops.MASK_BIDIR)):
        suf2d = ops.make_att_2d_masks(torch.ones(1, 5, dtype=torch.bool), torch.tensor([att_suf]))
        full = torch.cat([pad[None, None, :].expand(1, 5, 4), suf2d], dim=2)
        assert torch.equal(ops.suffix_mask(pad, 5, 5, mode), full)
    assert torch.equal(ops.suffix_mask(pad, 5, 0, ops.MASK_NONE), pad[None, None].expand(1, 5, 4))


def test_sinusoidal_embedding_closed_form():
    emb = ops.sinusoidal_time_embedding(torch.tensor([1.0, 0.3]), 720, 4e-3, 4.0)
    assert emb.shape == (2, 720) and emb.dtype == torch.float64
    t = float(torch.tensor(0.3))  # the fp32 timestep value enters the fp64 product as is
    # first / last periods are min_period / max_period
    assert abs(float(emb[1, 0]) - math.sin(2 * math.pi * t / 4e-3)) < 1e-9
    assert abs(float(emb[1, 359]) - math.sin(2 * math.pi * t / 4.0)) < 1e-12
    assert abs(float(emb[1, 360 + 359]) - math.cos(2 * math.pi * t / 4.0)) < 1e-12
    assert torch.allclose(emb[:, :360] ** 2 + emb[:, 360:] ** 2, torch.ones(2, 360, dtype=torch.float64))


# ------------------------------------------------------------------ attention
def test_eager_attention_against_float64_brute_force():
    q, k_pre, v_pre, k_suf, v_suf = attn_case(m=9, p=21, h=6, g_heads=2, d=64, seed=4)
    pad = torch.ones(21, dtype=torch.bool)
    pad[[3, 11]] = False
    for mode in (ops.MASK_BIDIR, ops.MASK_CAUSAL):
        out = ops.expert_attention(q, k_pre, v_pre, k_suf, v_suf, pad, mode)
        mask = ops.suffix_mask(pad, 9, 9, mode)[0]
        ref = ops.attention_f64(q, torch.cat([k_pre, k_suf]), torch.cat([v_pre, v_suf]), mask)
        assert out.dtype == BF16 and out.shape == (9, 6 * 64)
        assert float((out.double() - ref).abs().max()) < 2e-2


def test_attention_invariants():
    q, k_pre, v_pre, k_suf, v_suf = attn_case(m=5, p=12, h=6, g_heads=2, d=64, seed=5)
    pad = torch.ones(12, dtype=torch.bool)
    base = ops.expert_attention(q, k_pre, v_pre, k_suf, v_suf, pad, ops.MASK_CAUSAL)
    # GQA: kv head 1 only feeds q heads 3..5
    k2 = k_pre.clone()
    k2[:, 1] += 1.0
    out = ops.expert_attention(q, k2, v_pre, k_suf, v_suf, pad, ops.MASK_CAUSAL)
    assert torch.equal(out[:, : 3 * 64], base[:, : 3 * 64]) and not torch.equal(out[:, 3 * 64 :], base[:, 3 * 64 :])
    # causal: query 0 never sees suffix keys 1..4
    k3, v3 = k_suf.clone(), v_suf.clone()
    k3[1:] += 3.0
    v3[1:] -= 2.0
    out = ops.expert_attention(q, k_pre, v_pre, k3, v3, pad, ops.MASK_CAUSAL)
    assert torch.equal(out[0], base[0]) and not torch.equal(out[4], base[4])
    # permuting prefix keys (with their values and pad bits) changes nothing but summation order
    perm = torch.randperm(12, generator=torch.Generator().manual_seed(1))
    out = ops.expert_attention(q, k_pre[perm], v_pre[perm], k_suf, v_suf, pad[perm], ops.MASK_CAUSAL)
    assert float((out.float() - base.float()).abs().max()) < 2e-2
    # a fully masked row is uniform over ALL keys (finfo.min, not -inf)
    none = torch.zeros(12, dtype=torch.bool)
    out = ops.expert_attention(q, k_pre, v_pre, None, None, none, ops.MASK_NONE)
    mean_v = v_pre.float().mean(dim=0)  # [G, D]
    want = mean_v.repeat_interleave(3, dim=0).reshape(-1)
    assert float((out[0].float() - want).abs().max()) < 2e-2
    # constant V rows: output equals that constant whatever the scores
    vc = torch.ones_like(v_pre) * 0.5
    vs = torch.ones_like(v_suf) * 0.5
    out = ops.expert_attention(q, k_pre, vc, k_suf, vs, pad, ops.MASK_BIDIR)
    assert float((out.float() - 0.5).abs().max()) < 4e-3


def test_gemma_attention_core_matches_eager_within_bf16_noise():
    q, k_pre, v_pre, k_suf, v_suf = attn_case(m=7, p=40, h=8, g_heads=1, d=256, seed=6)
    pad = torch.ones(40, dtype=torch.bool)
    pad[5] = False
    a = ops.expert_attention(q, k_pre, v_pre, k_suf, v_suf, pad, ops.MASK_BIDIR, bf16_logits=False)
    b = ops.expert_attention(q, k_pre, v_pre, k_suf, v_suf, pad, ops.MASK_BIDIR, bf16_logits=True)
    assert a.shape == b.shape == (7, 8 * 256)
    assert float((a.float() - b.float()).abs().max()) < 5e-2


# --------------------------------------------------------------------------- #
# W8A8 tier: per-token activation quantisation and the fp8 x fp8 linear
# --------------------------------------------------------------------------- #
def test_activation_quantisation_closed_forms():
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(37, 96, generator=g) * torch.logspace(-3, 2, 37)[:, None]).to(BF16)
    x[5] = 0.0  # an all-zero token
    a8, sa = ops.quantize_activation_rows(x)
    amax = x.float().abs().amax(dim=-1)
    # the scale is amax / 448 exactly, the largest element of a row takes the largest code
    assert torch.equal(sa, amax / 448.0)
    vals = fp8.decode_e4m3fn(a8.view(torch.uint8))
    assert torch.equal(vals.abs().amax(dim=-1)[amax > 0], torch.full((36,), 448.0))
    assert sa[5] == 0 and (a8[5].view(torch.uint8) == 0).all()
    # the codes are the round-to-nearest-even of x / sa: an encoder written from the format's definition agrees
    live = amax > 0
    want = fp8.encode_e4m3fn_rne(x.float()[live] / sa[live, None]).reshape(-1, 96)
    assert torch.equal(a8[live].view(torch.uint8), want.to(torch.uint8))
    # ... so the dequantised value is within half a quantum of the input: |a8 * sa - x| <= sa * 2^(e-4),
    # e = exponent of the code's binade, 2^-9 * sa / 2 for the subnormal codes
    e = torch.floor(torch.log2(vals.abs().clamp(min=2.0**-6)))
    half_quantum = sa[:, None] * torch.exp2(e - 4.0)
    assert bool(((vals * sa[:, None] - x.float()).abs() <= half_quantum * (1 + 1e-6)).all())
    # scaling a token by a power of two scales its scale and keeps its codes (an exponent shift is exact)
    a8b, sab = ops.quantize_activation_rows((x.float() * 8.0).to(BF16))
    assert torch.equal(a8b.view(torch.uint8), a8.view(torch.uint8)) and torch.equal(sab, sa * 8.0)


def test_activation_quantisation_bf16_mode_rounds_scale_and_quotient():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(9, 64, generator=g).to(BF16) * 3.0
    a8, sa = ops.quantize_activation_rows(x, mode="bf16")
    # the scale is a bf16 value, within half a bf16 step of amax / 448
    assert torch.equal(sa, sa.to(BF16).float())
    exact = x.float().abs().amax(dim=-1) / 448.0
    assert bool(((sa - exact).abs() <= exact * 2.0**-8).all())
    # codes: fp8 of the bf16-rounded quotient by that scale
    want = (x.float() / sa[:, None]).to(BF16).to(ops.FP8)
    assert torch.equal(a8.view(torch.uint8), want.view(torch.uint8))
    # the two modes differ (double rounding, rounded scale): the fixture tells them apart
    a8f, _ = ops.quantize_activation_rows(x)
    assert not torch.equal(a8f.view(torch.uint8), a8.view(torch.uint8))


def test_w8a8_linear_against_float64_and_scale_placement():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(11, 128, generator=g).to(BF16)
    w8, sw = fp8.quantize_weight_rows(torch.randn(24, 128, generator=g) * 0.02)
    a8, sa = ops.quantize_activation_rows(x)
    got = ops.lin_w8a8(a8, sa, w8, sw)
    ref = (a8.double() @ w8.double().t()) * sa.double()[:, None] * sw.double()[None, :]
    assert got.dtype == BF16
    assert bool(((got.double() - ref).abs() <= ref.abs() * 2.0**-8 + 1e-30).all())  # one bf16 rounding of the exact value
    # both scales sit on the accumulator: doubling a token's scale doubles that output row only
    sa2 = sa.clone()
    sa2[3] *= 2.0
    got2 = ops.lin_w8a8(a8, sa2, w8, sw)
    assert torch.equal(got2[3].float(), got[3].float() * 2.0) and torch.equal(got2[:3], got[:3])
    # and the result is close to the unquantised product (e4m3 keeps 3-4 bits per factor)
    full = x.double() @ (w8.double() * sw.double()[:, None]).t()
    assert float((got.double() - full).abs().max()) <= 0.08 * float(full.abs().max())


def test_w8a8_ffn_composition():
    # gate and up share one quantised input; the intermediate is re-quantised per token before the down projection
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(13, 64, 96, seed=2)
    y = ops.gated_ffn_w8a8(x, wg8, sg, wu8, su, wd8, sd, "gelu_tanh")
    x8, sx = ops.quantize_activation_rows(x)
    h = ops.act_fn("gelu_tanh", ops.lin_w8a8(x8, sx, wg8, sg)) * ops.lin_w8a8(x8, sx, wu8, su)
    assert h.dtype == BF16
    h8, sh = ops.quantize_activation_rows(h)
    assert torch.equal(y, ops.lin_w8a8(h8, sh, wd8, sd))
    # within quantisation noise of the weight-only FFN
    wo = ops.gated_ffn(x, wg8, sg, wu8, su, wd8, sd, "gelu_tanh")
    assert float((y.float() - wo.float()).abs().max()) <= 0.1 * float(wo.float().abs().max()) + 1e-3

"""GPU parity of the fused expert-layer launches (norm + q|k|v + RoPE, o_proj + residual,
norm + gated FFN) against compositions of the CPU oracle's ops on seeded inputs.

Tolerance: rtol 2e-2 / atol 2e-2 on bf16 outputs, as for the other op tests.
"""

import pytest
import torch
import torch.nn.functional as F  # noqa: N812

from oracle import ops as oops
from oracle.inputs import ffn_case

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-2, 2e-2
BF16 = torch.bfloat16


def _close(got, want, what):
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - want).abs()
    worst = float((err - (ATOL + RTOL * want.abs())).max())
    assert worst <= 0, f"{what}: max|err|={float(err.max()):.4g}, exceeds atol+rtol*|ref| by {worst:.4g}"


@pytest.fixture(scope="module")
def tk():
    from tybok_amd import ops

    return ops


def _tables(tk, positions: int, d_half: int, base: float = 10_000.0):
    # the table the oracle's rope_half_split evaluates per call, for every position
    exponents = (2.0 / (d_half * 2)) * torch.arange(d_half, dtype=torch.float32)
    radians = torch.arange(positions, dtype=torch.float32)[:, None] / (base**exponents)[None, :]
    return tk.RopeTables(torch.cos(radians).cuda(), torch.sin(radians).cuda())


def _qkv_case(m, k, heads, kv_heads, d, x_dtype, seed):
    g = torch.Generator().manual_seed(seed)
    n = (heads + 2 * kv_heads) * d
    x = torch.randn(m, k, generator=g) * 1.7
    x = x.to(x_dtype)
    norm_w = (1.0 + 0.2 * torch.randn(k, generator=g)).to(BF16)
    w = (torch.randn(n, k, generator=g) * k**-0.5).to(BF16)
    pos = torch.randint(0, 400, (m,), generator=g, dtype=torch.int32)
    return x, norm_w, w, pos, n


def _qkv_oracle(x, norm_w, w, pos, heads, kv_heads, d, eps):
    m = x.shape[0]
    h = x if norm_w is None else oops.rms_norm_llama(x, norm_w, eps).to(BF16)
    y = F.linear(h, w)
    rc = (heads + kv_heads) * d
    qk = oops.rope_half_split(y[:, :rc].reshape(1, m, heads + kv_heads, d), pos[None].long())
    return torch.cat([qk.reshape(m, rc), y[:, rc:]], dim=1)


@pytest.mark.parametrize("x_dtype", [BF16, torch.float32])
@pytest.mark.parametrize(
    "m,k,heads,kv_heads,d",
    [
        (50, 720, 15, 5, 64),  # SmolVLA expert self-attention layer
        (50, 1024, 8, 1, 256),  # pi0.5 expert geometry
        (7, 48, 2, 1, 64),  # tiny, one ragged k tile
        (100, 720, 15, 5, 64),  # two row blocks
        (241, 960, 15, 5, 64),  # SmolVLA prefill, 3 cameras: 32-row blocks, every round requested up front
        (177, 960, 15, 5, 64),  # 2 cameras
        (40, 2048, 4, 2, 64),  # a K too long for the up-front prologue: statistics in a pass of their own
    ],
)
def test_norm_qkv_rope(tk, m, k, heads, kv_heads, d, x_dtype):
    eps = 1e-5
    x, norm_w, w, pos, n = _qkv_case(m, k, heads, kv_heads, d, x_dtype, seed=10)
    want = _qkv_oracle(x, norm_w, w, pos, heads, kv_heads, d, eps)
    pw = tk.pack_bf16_weight(w.cuda(), rope_half=d // 2)
    rope = _tables(tk, 512, d // 2)
    kw = dict(norm_w=norm_w.cuda(), eps=eps, rope=rope, rope_pos=pos.cuda(), rope_cols=(heads + kv_heads) * d)
    got = tk.bf16w_linear(x.cuda(), pw, **kw)
    again = tk.bf16w_linear(x.cuda(), pw, **kw)
    assert torch.equal(got, again), "two launches on the same input differ"
    _close(got, want, f"norm+qkv+rope M={m} K={k} D={d} x={x_dtype}")
    # the value columns also come out transposed (the attention kernel's suffix V^T operand)
    v0 = (heads + kv_heads) * d
    vt = torch.zeros(kv_heads * d, (m + 31) // 32 * 32, dtype=BF16, device="cuda")
    with_vt = tk.bf16w_linear(x.cuda(), pw, vt_out=vt, vt_col0=v0, **kw)
    assert torch.equal(with_vt, got)
    assert torch.equal(vt[:, :m], got[:, v0:].t()), "transposed value output differs from the value columns"
    assert not vt[:, m:].any(), "padding columns of V^T were written"


def test_qkv_rope_without_norm_and_query_only(tk):
    # cross layers project queries only (no k/v columns), positions 0..M-1
    m, k, heads, d = 50, 720, 15, 64
    x, _, w, _, _ = _qkv_case(m, k, heads, 0, d, BF16, seed=11)
    pos = torch.arange(m, dtype=torch.int32)
    want = _qkv_oracle(x, None, w, pos, heads, 0, d, 0.0)
    pw = tk.pack_bf16_weight(w.cuda(), rope_half=d // 2)
    got = tk.bf16w_linear(x.cuda(), pw, rope=_tables(tk, 64, d // 2), rope_pos=pos.cuda(), rope_cols=heads * d)
    _close(got, want, "q+rope")


def test_rope_positions_are_clamped_into_the_table(tk):
    m, k, heads, d = 8, 64, 1, 64
    x, _, w, _, _ = _qkv_case(m, k, heads, 0, d, BF16, seed=12)
    pos = torch.tensor([-5, 0, 3, 15, 16, 99, 7, 1], dtype=torch.int32)
    want = _qkv_oracle(x, None, w, pos.clamp(0, 15), heads, 0, d, 0.0)
    pw = tk.pack_bf16_weight(w.cuda(), rope_half=d // 2)
    got = tk.bf16w_linear(x.cuda(), pw, rope=_tables(tk, 16, d // 2), rope_pos=pos.cuda(), rope_cols=d)
    _close(got, want, "clamped positions")


@pytest.mark.parametrize("resid_dtype", [None, BF16, torch.float32])
@pytest.mark.parametrize("m,k,n", [(50, 960, 720), (50, 2048, 1024), (9, 80, 40), (130, 960, 720)])
def test_o_proj_residual(tk, m, k, n, resid_dtype):
    g = torch.Generator().manual_seed(13)
    x = torch.randn(m, k, generator=g).to(BF16)
    w = (torch.randn(n, k, generator=g) * k**-0.5).to(BF16)
    want = F.linear(x, w)
    resid = None
    if resid_dtype is not None:
        resid = torch.randn(m, n, generator=g).to(resid_dtype)
        want += resid  # in-place: an fp32 residual is added in fp32 and rounded to bf16 once
    pw = tk.pack_bf16_weight(w.cuda())
    got = tk.bf16w_linear(x.cuda(), pw, resid=None if resid is None else resid.cuda())
    _close(got, want, f"o_proj M={m} K={k} N={n} resid={resid_dtype}")
    for split in (1, 3):
        forced = tk.bf16w_linear(x.cuda(), pw, resid=None if resid is None else resid.cuda(), split_k=split)
        _close(forced, want, f"o_proj split_k={split}")


@pytest.mark.parametrize(
    "act,m,k,i",
    [("silu", 50, 720, 2048), ("gelu_tanh", 50, 1024, 4096), ("silu", 1, 720, 2048), ("silu", 241, 960, 2560), ("silu", 64, 720, 2048), ("silu", 33, 2048, 512)],
)
def test_norm_gated_ffn(tk, act, m, k, i):
    eps = 1e-5
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(m, k, i, seed=14)
    g = torch.Generator().manual_seed(15)
    x = (x.float() * 2.5).to(BF16)
    norm_w = (1.0 + 0.2 * torch.randn(k, generator=g)).to(BF16)
    resid = torch.randn(m, k, generator=g).to(BF16)
    want = oops.gated_ffn(oops.rms_norm_llama(x, norm_w, eps), wg8, sg, wu8, su, wd8, sd, act)
    want += resid
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    got = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, act, resid=resid.cuda(), norm_w=norm_w.cuda(), eps=eps)
    _close(got, want, f"norm+ffn {act} M={m}")
    # the fused norm must equal normalising first and calling the plain entry point, bit for bit
    # (same rounding points, same GEMM)
    h = oops.rms_norm_llama(x, norm_w, eps).cuda()
    two_step = tk.fp8w_gated_ffn(h, wgu, wd, act, resid=resid.cuda())
    mism = (got != two_step).float().mean().item()
    assert mism < 0.02, f"fused norm differs from norm-then-FFN on {mism:.1%} of the outputs"


@pytest.mark.parametrize("m,k,heads,kv_heads,d", [(50, 1024, 8, 1, 256), (19, 96, 2, 1, 64)])
def test_adarms_qkv_rope_bf16_arithmetic(tk, m, k, heads, kv_heads, d):
    # the pi0.5 expert projection: adaptive RMSNorm prologue, rotate-half RoPE in bf16 arithmetic
    eps = 1e-6
    x, _, w, pos, n = _qkv_case(m, k, heads, kv_heads, d, BF16, seed=16)
    g = torch.Generator().manual_seed(17)
    mod = 0.3 * torch.randn(1, 3 * k, generator=g)
    h, _ = oops.gemma_rms_norm(x[None], eps, modulation=mod)
    y = F.linear(h[0], w)
    rc = (heads + kv_heads) * d
    cos, sin = oops.gemma_rope_cos_sin(d, pos[None].long(), BF16)
    qk = oops.gemma_apply_rope(y[:, :rc].reshape(1, m, heads + kv_heads, d).transpose(1, 2), cos, sin)
    want = torch.cat([qk.transpose(1, 2).reshape(m, rc), y[:, rc:]], dim=1)
    cos_t, sin_t = oops.gemma_rope_cos_sin(d, torch.arange(512)[None], BF16)
    rope = tk.RopeTables(cos_t[0, :, : d // 2].float().contiguous().cuda(), sin_t[0, :, : d // 2].float().contiguous().cuda())
    scale, shift = mod[0, :k].contiguous().cuda(), mod[0, k : 2 * k].contiguous().cuda()
    pw = tk.pack_bf16_weight(w.cuda(), rope_half=d // 2)
    got = tk.bf16w_linear(x.cuda(), pw, ada=(scale, shift), eps=eps, rope=rope, rope_pos=pos.cuda(), rope_cols=rc, rope_bf16=True)
    _close(got, want, f"adarms+qkv+rope(bf16) M={m} K={k} D={d}")
    mism = (got.cpu() != want).float().mean().item()
    assert mism < 0.03, f"{mism:.1%} of the outputs differ from the eager composition (expected: rare 1-ulp flips)"


def test_gated_residual_o_proj_and_adarms_ffn(tk):
    m, k, n = 50, 2048, 1024
    g = torch.Generator().manual_seed(18)
    x = torch.randn(m, k, generator=g).to(BF16)
    w = (torch.randn(n, k, generator=g) * k**-0.5).to(BF16)
    gate = torch.randn(n, generator=g).to(BF16)
    resid = torch.randn(m, n, generator=g).to(BF16)
    want = resid + F.linear(x, w) * gate
    got = tk.bf16w_linear(x.cuda(), tk.pack_bf16_weight(w.cuda()), resid=resid.cuda(), gate=gate.cuda())
    _close(got, want, "o_proj gated residual")
    # adaptive norm + GeGLU FFN + gated residual
    eps = 1e-6
    xx, wg8, sg, wu8, su, wd8, sd = ffn_case(m, 1024, 4096, seed=19)
    mod = 0.3 * torch.randn(1, 3 * 1024, generator=g)
    h, gt = oops.gemma_rms_norm(xx[None], eps, modulation=mod)
    want = xx + oops.gated_ffn(h[0], wg8, sg, wu8, su, wd8, sd, "gelu_tanh") * gt[0]
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    scale, shift = mod[0, :1024].contiguous().cuda(), mod[0, 1024:2048].contiguous().cuda()
    got = tk.fp8w_gated_ffn(xx.cuda(), wgu, wd, "gelu_tanh", resid=xx.cuda(), gate=gt[0].contiguous().cuda(), ada=(scale, shift), eps=eps)
    _close(got, want, "adarms + GeGLU FFN + gated residual")


def test_fused_layer_argument_checks(tk):
    w = torch.zeros(128, 64, dtype=BF16, device="cuda")
    x = torch.zeros(4, 64, dtype=BF16, device="cuda")
    pw_rope = tk.pack_bf16_weight(w, rope_half=32)
    with pytest.raises(ValueError):
        tk.bf16w_linear(x, pw_rope)  # pair-ordered weight without the rotary epilogue
    with pytest.raises(TypeError):
        tk.bf16w_linear(x.float(), tk.pack_bf16_weight(w))  # fp32 input without a norm
    with pytest.raises(RuntimeError):
        tk.pack_bf16_weight(torch.zeros(96, 64, dtype=BF16, device="cuda"), rope_half=32)  # 64 does not divide 96
    rope = _tables(tk, 16, 32)
    with pytest.raises(RuntimeError):
        tk.bf16w_linear(x, pw_rope, rope=rope, rope_pos=torch.zeros(4, dtype=torch.int32, device="cuda"), rope_cols=32)


@pytest.mark.parametrize("adaptive", [False, True])
def test_step_tail_norm_projection_euler(tk, adaptive):
    m, k, n = 50, 720 if not adaptive else 1024, 32
    g = torch.Generator().manual_seed(20)
    x = (torch.randn(m, k, generator=g) * 2.0).to(BF16)
    w = torch.randn(n, k, generator=g) * k**-0.5
    b = torch.randn(n, generator=g)
    x_t = torch.randn(m, n, generator=g)
    dt = -0.1
    if adaptive:
        mod = 0.3 * torch.randn(1, 3 * k, generator=g)
        h, _ = oops.gemma_rms_norm(x[None], 1e-6, modulation=mod)
        h = h[0]
        kw = dict(ada=(mod[0, :k].contiguous().cuda(), mod[0, k : 2 * k].contiguous().cuda()), eps=1e-6)
    else:
        norm_w = (1.0 + 0.2 * torch.randn(k, generator=g)).to(BF16)
        h = oops.rms_norm_llama(x, norm_w, 1e-5)
        kw = dict(norm_w=norm_w.cuda(), eps=1e-5)
    v_want = F.linear(h.float(), w, b)
    x_want = x_t + dt * v_want
    v, x_new = tk.expert_tail(x.cuda(), w.cuda(), b.cuda(), x_t=x_t.cuda(), dt=dt, want_v=True, **kw)
    assert float((v.cpu() - v_want).abs().max()) < 2e-3, "velocity differs from norm + fp32 linear"
    assert float((x_new.cpu() - x_want).abs().max()) < 2e-4, "Euler update differs"
    v_only, none = tk.expert_tail(x.cuda(), w.cuda(), b.cuda(), **kw)
    assert none is None and torch.equal(v_only, v)


@pytest.mark.parametrize("model,m,k,j", [("smolvla", 50, 720, 720), ("pi05", 50, 1024, 1024), ("smolvla", 7, 96, 1100), ("pi05", 33, 2048, 40)])
def test_step_tail_with_the_next_steps_embedding(tk, model, m, k, j):
    # the tail launch also writes the first linear of the next step's suffix embedding from the updated x
    # (flow_matching.py:259-311 with the SiLU, fp32 out; pi05 flow_matching.py:464-502, cast to bf16): against the
    # torch expression on the tail's own x_new, and the tail's other outputs unchanged bit for bit
    n = 32
    g = torch.Generator().manual_seed(23)
    x = (torch.randn(m, k, generator=g) * 2.0).to(BF16).cuda()
    w = (torch.randn(n, k, generator=g) * k**-0.5).cuda()
    b = torch.randn(n, generator=g).cuda()
    x_t = torch.randn(m, n, generator=g).cuda()
    ew = (torch.randn(j, n, generator=g) * n**-0.5).cuda()
    eb = torch.randn(j, generator=g).cuda()
    if model == "pi05":
        mod = 0.3 * torch.randn(1, 3 * k, generator=g)
        kw = dict(ada=(mod[0, :k].contiguous().cuda(), mod[0, k : 2 * k].contiguous().cuda()), eps=1e-6)
        wide = torch.full((m, j + 8), 7.0, dtype=BF16, device="cuda")  # a row pitch wider than the rows
        out = wide[:, :j]
        act = "none"
    else:
        kw = dict(norm_w=(1.0 + 0.2 * torch.randn(k, generator=g)).to(BF16).cuda(), eps=1e-5)
        out = torch.empty(m, j, dtype=torch.float32, device="cuda")
        act = "silu"
    v0, x0 = tk.expert_tail(x, w, b, x_t=x_t, dt=-0.1, want_v=True, **kw)
    v1, x1 = tk.expert_tail(x, w, b, x_t=x_t, dt=-0.1, want_v=True, embed=(ew, eb, act, out), **kw)
    assert torch.equal(v0, v1) and torch.equal(x0, x1)
    want = F.linear(x1.cpu(), ew.cpu(), eb.cpu())
    if model == "pi05":
        # one rounding to bf16 of an fp32 sum: at most one bf16 step from the torch result where the sums differ in order
        got = out.float().cpu()
        assert float(((got - want.to(BF16).float()).abs() / want.abs().clamp_min(1.0)).max()) <= 2**-7
        assert float((got != want.to(BF16).float()).float().mean()) < 0.02
        assert torch.equal(wide[:, j:].float().cpu(), torch.full((m, 8), 7.0))
    else:
        want = F.silu(want)
        assert float((out.cpu() - want).abs().max()) < 2e-5
    # no bias
    out2 = torch.empty(m, j, dtype=torch.float32, device="cuda")
    tk.expert_tail(x, w, b, x_t=x_t, dt=-0.1, embed=(ew, None, "none", out2), **kw)
    assert float((out2.cpu() - F.linear(x1.cpu(), ew.cpu())).abs().max()) < 2e-5
    with pytest.raises(ValueError):
        tk.expert_tail(x, w, b, embed=(ew, eb, act, out), **kw)  # no x_t: nothing to embed


@pytest.mark.parametrize("m,p,k", [(50, 241, 720), (50, 177, 720), (7, 33, 96), (33, 256, 768)])
def test_cross_layer_in_one_launch(tk, m, p, k):
    # norm + q projection + RoPE inside the attention launch (SmolVLA cross layers: 15 / 5 heads of 64,
    # fp32 expert K/V as hi + lo planes, prefix pad mask) against projecting first and attending afterwards,
    # and against the CPU oracle's composition
    heads, kv_heads, d, eps = 15, 5, 64, 1e-5
    g = torch.Generator().manual_seed(51)
    x = (torch.randn(m, k, generator=g) * 1.7).to(BF16)
    norm_w = (1.0 + 0.2 * torch.randn(k, generator=g)).to(BF16)
    wq = (torch.randn(heads * d, k, generator=g) * k**-0.5).to(BF16)
    ek, ev = torch.randn(p, kv_heads, d, generator=g), torch.randn(p, kv_heads, d, generator=g)
    pad = torch.rand(p, generator=g) > 0.2
    pad[0] = True
    pos = torch.randint(0, 300, (m,), generator=g, dtype=torch.int32)
    rope = _tables(tk, 512, d // 2)
    pw = tk.pack_bf16_weight(wq.cuda(), rope_half=d // 2)
    cache = tk.prepare_prefix_kv(ek.cuda(), ev.cuda())
    fused = tk.cross_attn_fused(x.cuda(), pw, norm_w.cuda(), eps, rope, pos.cuda(), cache, pad.cuda())
    q = tk.bf16w_linear(x.cuda(), pw, norm_w=norm_w.cuda(), eps=eps, rope=rope, rope_pos=pos.cuda(), rope_cols=heads * d)
    two = tk.expert_attn(q.view(m, heads, d), cache, None, pad.cuda(), tk.MASK_NONE)
    _close(fused, two.cpu(), f"fused cross layer vs two launches M={m} P={p}")
    same = (fused == two).float().mean().item()
    assert same > 0.9, f"only {same:.1%} of the outputs agree bit for bit with the two-launch path"
    assert torch.equal(fused, tk.cross_attn_fused(x.cuda(), pw, norm_w.cuda(), eps, rope, pos.cuda(), cache, pad.cuda()))
    # oracle: RMSNorm -> q -> half-split RoPE -> eager attention over the fp32 K/V under the pad mask
    h = oops.rms_norm_llama(x, norm_w, eps)
    qo = oops.rope_half_split(F.linear(h, wq).view(1, m, heads, d), pos[None].long())
    want = oops.eager_attention(pad[None, None, :].expand(1, m, p), qo, ek[None], ev[None])[0]
    _close(fused, want, f"fused cross layer vs oracle M={m} P={p}")


def test_cross_layer_in_one_launch_rejects_what_it_cannot_run(tk):
    g = torch.Generator().manual_seed(52)
    rope = _tables(tk, 64, 32)
    x = torch.randn(8, 96, generator=g).to(BF16).cuda()
    nw = torch.ones(96, dtype=BF16, device="cuda")
    pw = tk.pack_bf16_weight(torch.randn(128, 96, generator=g).to(BF16).cuda(), rope_half=32)
    pos = torch.zeros(8, dtype=torch.int32, device="cuda")
    ok = tk.prepare_prefix_kv(torch.randn(40, 2, 64, generator=g).cuda(), torch.randn(40, 2, 64, generator=g).cuda())
    with pytest.raises(ValueError):  # bf16 K/V: no lo planes
        bf = tk.prepare_prefix_kv(torch.randn(40, 2, 64, generator=g).to(BF16).cuda(), torch.randn(40, 2, 64, generator=g).to(BF16).cuda())
        tk.cross_attn_fused(x, pw, nw, 1e-5, rope, pos, bf, None)
    with pytest.raises(RuntimeError, match="8 key tiles"):
        big = tk.prepare_prefix_kv(torch.randn(300, 2, 64, generator=g).cuda(), torch.randn(300, 2, 64, generator=g).cuda())
        tk.cross_attn_fused(x, pw, nw, 1e-5, rope, pos, big, None)
    assert tk.cross_attn_fused(x, pw, nw, 1e-5, rope, pos, ok, None).shape == (8, 128)


@pytest.mark.parametrize("bf16_math", [False, True])
@pytest.mark.parametrize("m,k,heads,kv_heads,d", [(300, 256, 4, 1, 64), (712, 2048, 8, 1, 256), (7, 96, 2, 2, 32)])
def test_norm_and_rotary_as_launches_of_their_own_equal_the_fused_projection(tk, m, k, heads, kv_heads, d, bf16_math):
    # many-row prefills run the q|k|v projection as a library GEMM between tk_rms_norm_rows and tk_rope_rows:
    # the two kernels must reproduce the fused projection's prologue / epilogue bit for bit on the same GEMM output
    g = torch.Generator().manual_seed(77)
    x = torch.randn(m, k, generator=g).to(BF16).cuda()
    scale = (0.3 * torch.randn(k, generator=g)).cuda()
    shift = (0.1 * torch.randn(k, generator=g)).cuda()
    w = torch.randn(k, generator=g).to(BF16).cuda()
    xf = x.float()
    rstd = torch.rsqrt(xf.square().mean(-1, keepdim=True) + 1e-6)
    want_ada = ((xf * rstd) * (1.0 + scale) + shift).to(BF16)
    want_llama = (w.float() * (xf * rstd).to(BF16).float()).to(BF16)
    got_ada = tk.rms_norm_rows(x, ada=(scale, shift), eps=1e-6)
    got_llama = tk.rms_norm_rows(x, norm_w=w, eps=1e-6)
    for got, want in ((got_ada, want_ada), (got_llama, want_llama)):
        diff = (got.float() - want.float()).abs()
        assert bool((diff <= want.float().abs().clamp_min(2.0**-6) * 2.0**-7).all())  # one bf16 step (rstd differs in its last bit)
        assert float((diff > 0).float().mean()) < 0.02
    # rotary: same table, same arithmetic as the projection epilogue -> compare on an identity-like path
    nq, nkv = heads * d, kv_heads * d
    half = d // 2
    pos = torch.randint(0, 60, (m,), generator=g).to(torch.int32).cuda()
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float32) / half))
    ang = torch.arange(64, dtype=torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos(), ang.sin()
    if bf16_math:
        cos, sin = cos.to(BF16).float(), sin.to(BF16).float()
    tables = tk.RopeTables(cos.contiguous().cuda(), sin.contiguous().cuda())
    y = torch.randn(m, nq + 2 * nkv, generator=g).to(BF16).cuda()
    ref = y.clone().float().cpu()
    c, s_ = cos[pos.cpu().long()], sin[pos.cpu().long()]  # [m, half]
    for h in range(heads + kv_heads):
        a, b = ref[:, h * d : h * d + half].clone(), ref[:, h * d + half : (h + 1) * d].clone()
        if bf16_math:
            r = lambda t: t.to(BF16).float()  # noqa: E731
            ref[:, h * d : h * d + half] = r(r(a * c) - r(b * s_))
            ref[:, h * d + half : (h + 1) * d] = r(r(b * c) + r(a * s_))
        else:
            ref[:, h * d : h * d + half] = (a * c - b * s_).to(BF16).float()
            ref[:, h * d + half : (h + 1) * d] = (b * c + a * s_).to(BF16).float()
    out = tk.rope_rows(y, tables, pos, nq + nkv, rope_bf16=bf16_math)
    assert out.data_ptr() == y.data_ptr()
    assert torch.equal(out.float().cpu(), ref), f"max diff {float((out.float().cpu() - ref).abs().max())}"
    with pytest.raises(RuntimeError):
        tk.rope_rows(y, tables, pos, nq + nkv + 8)

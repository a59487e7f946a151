"""bf16-weight many-row linear (bias / GELU / residual epilogues) against plain torch fp32 arithmetic on the same
bf16 operands, with the rounding points of ``F.linear`` / ``F.gelu`` on bf16 tensors.  GPU only."""

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


@pytest.fixture(scope="module")
def tk():
    from tybok_amd import ops

    return ops


def _case(m, k, n, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(BF16)
    w = (torch.randn(n, k, generator=g) / k**0.5).to(BF16)
    b = torch.randn(n, generator=g).to(BF16)
    return x, w, b


def _want(x, w, b, act=None, resid=None):
    y = (x.double() @ w.double().t() + (0 if b is None else b.double())).float()
    if act == "gelu_tanh":
        y = F.gelu(y.to(BF16).float(), approximate="tanh")
    elif act == "gelu_tanh_fp32":
        y = F.gelu(y, approximate="tanh")
    y = y.to(BF16)
    if resid is not None:
        y = (y.float() + resid.float()).to(BF16)
    return y


def _close(got, want, what, frac_exact=0.97):
    got, want = got.float().cpu(), want.float()
    err = (got - want).abs()
    tol = 1e-2 + 2**-7 * want.abs()  # one bf16 ulp of the result (the fp32 sum order differs) plus a floor near zero
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} / {bad.numel()} outside tolerance, max |err| {err.max():.4g}"
    same = (got == want).float().mean().item()
    assert same >= frac_exact, f"{what}: only {same:.1%} of the outputs equal the correctly rounded result"


TILES = [0, 42, 41, 32, 31, 22, 21, 12, 11]


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("m,k,n", [(768, 1152, 4608), (300, 4304, 1152), (3072, 768, 768), (257, 80, 40), (1, 64, 8), (130, 208, 264)])
def test_dense_matches_torch(tk, tile, m, k, n):
    x, w, b = _case(m, k, n)
    pw = tk.pack_bf16_weight(w.cuda())
    got = tk.bf16w_dense(x.cuda(), pw, b.cuda(), tile=tile)
    _close(got, _want(x, w, b), f"dense M={m} K={k} N={n} tile={tile}")
    got = tk.bf16w_dense(x.cuda(), pw, None, tile=tile)
    _close(got, _want(x, w, None), f"dense without bias M={m} K={k} N={n} tile={tile}")


@pytest.mark.parametrize("act", ["gelu_tanh", "gelu_tanh_fp32"])
@pytest.mark.parametrize("m,k,n", [(768, 1152, 4304), (3072, 768, 3072), (100, 64, 96)])
def test_dense_gelu(tk, act, m, k, n):
    x, w, b = _case(m, k, n, seed=1)
    got = tk.bf16w_dense(x.cuda(), tk.pack_bf16_weight(w.cuda()), b.cuda(), act)
    _close(got, _want(x, w, b, act), f"dense {act} M={m} K={k} N={n}", frac_exact=0.95)


@pytest.mark.parametrize("resid_dtype", [torch.float32, BF16])
@pytest.mark.parametrize("tile", [42, 31, 21, 11])
def test_dense_residual_tail_and_pitch(tk, resid_dtype, tile):
    # N % 8 == 4, output and residual are column slices of wider buffers; nothing past N may be written
    m, k, n = 385, 96, 260
    x, w, b = _case(m, k, n, seed=2)
    pitch = 272
    r = torch.randn(m, pitch, generator=torch.Generator().manual_seed(3)).to(resid_dtype)
    buf = torch.full((m, pitch), 7.0, dtype=BF16, device="cuda")
    tk.bf16w_dense(x.cuda(), tk.pack_bf16_weight(w.cuda()), b.cuda(), resid=r.cuda()[:, :n], out=buf[:, :n], tile=tile)
    _close(buf[:, :n], _want(x, w, b, resid=r[:, :n]), "dense + residual")
    assert bool((buf[:, n:] == 7.0).all()), "wrote past N"


@pytest.mark.parametrize("split", [2, 3, 5])
def test_dense_split_k_is_deterministic(tk, split):
    x, w, b = _case(300, 4304, 256, seed=4)
    pw = tk.pack_bf16_weight(w.cuda())
    xc, bc = x.cuda(), b.cuda()
    first = tk.bf16w_dense(xc, pw, bc, split_k=split)
    again = tk.bf16w_dense(xc, pw, bc, split_k=split)
    assert torch.equal(first, again)
    _close(first, _want(x, w, b), f"split {split}")


def test_dense_exact_on_small_integers(tk):
    # integer operands: every product and partial sum is exact in fp32 whatever the order, so a wrong pairing of k
    # between the two MFMA operands or a misplaced output column cannot hide behind a tolerance
    g = torch.Generator().manual_seed(5)
    m, k, n = 200, 144, 104
    x = torch.randint(-4, 5, (m, k), generator=g).to(BF16)
    w = torch.randint(-3, 4, (n, k), generator=g).to(BF16)
    b = torch.randint(-8, 9, (n,), generator=g).to(BF16)
    want = (x.float() @ w.float().t() + b.float()).to(BF16)
    for tile in TILES:
        got = tk.bf16w_dense(x.cuda(), tk.pack_bf16_weight(w.cuda()), b.cuda(), tile=tile)
        assert torch.equal(got.cpu(), want), f"tile {tile}"


def test_dense_rejects_bad_arguments(tk):
    x, w, b = _case(64, 64, 64)
    pw = tk.pack_bf16_weight(w.cuda())
    with pytest.raises(RuntimeError):
        tk.bf16w_dense(x.cuda(), pw, b.cuda(), tile=33)
    with pytest.raises(ValueError):
        tk.bf16w_dense(x.cuda()[:, :32], pw, b.cuda())


F16 = torch.float16


@pytest.mark.parametrize("tile", [0, 42, 31, 21, 11])
@pytest.mark.parametrize("m,k,n,act", [(512, 1152, 3456, None), (512, 1152, 4304, "gelu_tanh"), (512, 4304, 1152, None), (257, 80, 40, "gelu_tanh_fp32"), (130, 208, 264, None)])
def test_dense_fp16_flavour_matches_torch(tk, tile, m, k, n, act):
    # every 16-bit operand in fp16 (tk_f16w_dense): pi0.5's fp16 tower tiers.  Reference arithmetic: exact products
    # of the fp16 operands summed in float64, one rounding to fp16 (then the GELU on that value or on the fp32 one).
    g = torch.Generator().manual_seed(3)
    x = torch.randn(m, k, generator=g).to(F16)
    w = (torch.randn(n, k, generator=g) / k**0.5).to(F16)
    b = torch.randn(n, generator=g).to(F16)
    y = (x.double() @ w.double().t() + b.double()).float()
    if act == "gelu_tanh":
        y = F.gelu(y.to(F16).float(), approximate="tanh")
    elif act == "gelu_tanh_fp32":
        y = F.gelu(y, approximate="tanh")
    want = y.to(F16)
    got = tk.bf16w_dense(x.cuda(), tk.pack_bf16_weight(w.cuda()), b.cuda(), act, tile=tile)
    assert got.dtype == F16
    err = (got.float().cpu() - want.float()).abs()
    tol = 2e-3 + 2**-10 * want.float().abs()  # one fp16 ulp of the result plus a floor near zero
    assert not (err > tol).any(), f"fp16 dense M={m} K={k} N={n} tile={tile}: max |err| {err.max():.4g}"
    assert (got.cpu() == want).float().mean().item() >= 0.97
    # fp32 and fp16 residuals
    r32 = torch.randn(m, n, generator=g)
    got_r = tk.bf16w_dense(x.cuda(), tk.pack_bf16_weight(w.cuda()), b.cuda(), act, resid=r32.cuda(), tile=tile)
    assert torch.equal(got_r.cpu(), (got.float().cpu() + r32).to(F16))
    r16 = r32.to(F16)
    got_r = tk.bf16w_dense(x.cuda(), tk.pack_bf16_weight(w.cuda()), b.cuda(), act, resid=r16.cuda(), tile=tile)
    assert torch.equal(got_r.cpu(), (got.float().cpu() + r16.float()).to(F16))


def _rope_case(m, heads_rot, heads_v, d, positions=300, seed=3):
    g = torch.Generator().manual_seed(seed)
    half = d // 2
    ang = torch.rand(positions, half, generator=g) * 6.0
    pos = torch.randint(-3, positions + 5, (m,), generator=g).to(torch.int32)  # some outside the tables: clamped
    return ang.cos().contiguous(), ang.sin().contiguous(), pos, half, heads_rot * d, (heads_rot + heads_v) * d


@pytest.mark.parametrize("tile", [0, 42, 32, 22, 12])
@pytest.mark.parametrize("bf16_math", [True, False])
@pytest.mark.parametrize("m,k,d,heads_rot,heads_v", [(712, 2048, 256, 9, 1), (300, 960, 64, 20, 5), (257, 80, 64, 3, 2), (33, 64, 128, 1, 1)])
def test_dense_with_rotary_epilogue_gives_the_bits_of_the_three_launches(tk, tile, bf16_math, m, k, d, heads_rot, heads_v):
    # tk_bf16w_dense_rope (weights in rotary pair order, q | k rotated in the epilogue, V^T written beside V) against
    # tk_bf16w_dense on naturally packed weights + tk_rope_rows + tk_batched_transpose_v: the same arithmetic in the
    # same order, so the same bits -- and the rotated columns against plain torch on the GEMM's own output
    cos, sin, pos, half, rope_cols, n = _rope_case(m, heads_rot, heads_v, d)
    if bf16_math:
        cos, sin = cos.to(BF16).float(), sin.to(BF16).float()
    x, w, _ = _case(m, k, n, seed=4)
    tables = tk.RopeTables(cos.cuda(), sin.cuda())
    mp = (m + 31) // 32 * 32
    # reference path: three launches
    # (the summation order of an output depends on the K split alone: pinned to the same value on both paths --
    # none where a tile is forced, 2 for the automatic choice when K allows it)
    ks = 1 if tile or k < 128 else 2
    base = tk.bf16w_dense(x.cuda(), tk.pack_bf16_weight(w.cuda()), None, split_k=ks)
    plain = base.clone()
    tk.rope_rows(base, tables, pos.cuda(), rope_cols, rope_bf16=bf16_math)
    vt_want = torch.zeros(n - rope_cols, mp, dtype=BF16, device="cuda")
    vt_want[:, :m] = base[:, rope_cols:].t()
    # one launch; vt_out starts with a sentinel-free zero fill (rows past M must stay zero)
    vt = torch.zeros(n - rope_cols, mp, dtype=BF16, device="cuda")
    got = tk.bf16w_dense_rope(x.cuda(), tk.pack_bf16_weight(w.cuda(), rope_half=half), tables, pos.cuda(), rope_cols, rope_bf16=bf16_math,
                              vt_out=vt, vt_col0=rope_cols, tile=tile, split_k=ks)  # fmt: skip
    assert torch.equal(got, base), f"max |diff| {float((got.float() - base.float()).abs().max())}"
    assert torch.equal(vt, vt_want)
    # the rotation itself, in torch, on the linear's bf16 output
    p = pos.long().clamp(0, cos.shape[0] - 1)
    y = plain.float().cpu()[:, :rope_cols].view(m, heads_rot, 2, half)
    a, b = y[:, :, 0], y[:, :, 1]
    c, s = cos[p][:, None, :], sin[p][:, None, :]
    if bf16_math:
        r = lambda t: t.to(BF16).float()  # noqa: E731
        ra, rb = r(r(a * c) - r(b * s)), r(r(b * c) + r(a * s))
    else:
        ra, rb = (a * c - b * s).to(BF16).float(), (b * c + a * s).to(BF16).float()
    want = torch.stack([ra, rb], dim=2).reshape(m, rope_cols)
    err = (got.float().cpu()[:, :rope_cols] - want).abs()
    assert float(err.max()) <= (0.0 if bf16_math else 2**-6 * float(want.abs().max())), float(err.max())


def test_dense_rope_argument_rules(tk):
    cos, sin, pos, half, rope_cols, n = _rope_case(64, 2, 1, 64)
    x, w, _ = _case(64, 64, n)
    tables = tk.RopeTables(cos.cuda(), sin.cuda())
    with pytest.raises(ValueError, match="rotary pair order"):
        tk.bf16w_dense_rope(x.cuda(), tk.pack_bf16_weight(w.cuda()), tables, pos.cuda(), rope_cols)
    pw = tk.pack_bf16_weight(w.cuda(), rope_half=half)
    with pytest.raises(RuntimeError, match="whole heads"):
        tk.bf16w_dense_rope(x.cuda(), pw, tables, pos.cuda(), rope_cols + 32)
    with pytest.raises(RuntimeError, match="tile"):
        tk.bf16w_dense_rope(x.cuda(), pw, tables, pos.cuda(), rope_cols, tile=31)


@pytest.mark.parametrize("tile", [0, 42, 41, 32, 31, 22, 21, 12, 11])
@pytest.mark.parametrize("dt", [BF16, torch.float16])
@pytest.mark.parametrize("b,p,k,heads,d", [(3, 1024, 768, 12, 64), (2, 256, 1152, 16, 96), (1, 96, 64, 2, 64), (5, 32, 80, 1, 64)])
def test_dense_writes_the_transposed_values_of_a_packed_qkv_projection(tk, tile, dt, b, p, k, heads, d):
    # tk_bf16w_dense_vt: the projection's own output is unchanged and the value columns also arrive as
    # [B, G, D, P] -- the bits tk_batched_transpose_v makes of them
    n = 3 * heads * d
    x, w, bias = _case(b * p, k, n, seed=5)
    x, w, bias = x.to(dt), w.to(dt), bias.to(dt)
    pw = tk.pack_bf16_weight(w.cuda())
    want = tk.bf16w_dense(x.cuda(), pw, bias.cuda(), tile=tile, split_k=1)
    vt_want = tk.transpose_v(want.view(b, p, 3, heads, d)[:, :, 2])
    vt = torch.full((b, heads, d, p), 7.0, dtype=dt, device="cuda")
    got = tk.bf16w_dense(x.cuda(), pw, bias.cuda(), tile=tile, split_k=1, vt_out=vt, vt_col0=2 * heads * d)
    assert torch.equal(got, want)
    assert torch.equal(vt, vt_want[..., :p])


def test_dense_vt_argument_rules(tk):
    x, w, bias = _case(64, 64, 3 * 64)
    pw = tk.pack_bf16_weight(w.cuda())
    vt = torch.empty(2, 1, 64, 32, dtype=BF16, device="cuda")
    with pytest.raises(ValueError, match="no activation or residual"):
        tk.bf16w_dense(x.cuda(), pw, bias.cuda(), "gelu_tanh", vt_out=vt, vt_col0=128)
    with pytest.raises(ValueError, match="multiple of 32"):
        tk.bf16w_dense(x.cuda(), pw, bias.cuda(), vt_out=torch.empty(4, 1, 64, 16, dtype=BF16, device="cuda"), vt_col0=128)
    with pytest.raises(RuntimeError, match="multiple of 64"):
        tk.bf16w_dense(x.cuda(), pw, bias.cuda(), vt_out=torch.empty(2, 1, 96, 32, dtype=BF16, device="cuda"), vt_col0=96)

"""GPU parity of the HIP kernels (through the C ABI) against the CPU oracle on seeded inputs.

Tolerances are the ones the task states for bf16 op outputs: rtol 2e-2 / atol 2e-2.
"""

import pytest
import torch

from oracle import fp8 as ofp8
from oracle import ops as oops
from oracle.inputs import GEMM_MS, GEMM_SHAPES, attn_case, ffn_case, gemm_case

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-2, 2e-2


def _close(got: torch.Tensor, want: torch.Tensor, what: str):
    got = got.float().cpu()
    want = want.float().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - want).abs()
    bound = ATOL + RTOL * want.abs()
    worst = float((err - bound).max())
    assert worst <= 0, f"{what}: max|err|={float(err.max()):.4g}, exceeds atol+rtol*|ref| by {worst:.4g}"


@pytest.fixture(scope="module")
def tk():
    from tybok_amd import ops

    return ops


def test_device_decodes_ocp_e4m3fn(tk):
    got = tk.decode_fp8_table().cpu()
    want = torch.from_numpy(ofp8.e4m3fn_table())
    ok = ~torch.isnan(want)
    assert torch.equal(torch.isnan(got), torch.isnan(want)), "NaN codes differ: not the OCP e4m3fn flavour"
    assert torch.equal(got[ok], want[ok])
    assert torch.equal(torch.signbit(got[ok]), torch.signbit(want[ok]))


def test_pack_layout(tk):
    g = torch.Generator().manual_seed(0)
    n, k = 80, 48  # ragged in both directions (3 n-tiles, 2 k-tiles)
    codes = torch.randint(0, 256, (n, k), generator=g, dtype=torch.uint8)
    packed = tk.pack_fp8_weight(codes.cuda(), torch.ones(n)).data.cpu()
    kt_n = 2
    ref = torch.zeros(3 * kt_n * 1024, dtype=torch.uint8)
    for nt in range(3):
        for kt in range(kt_n):
            for lane in range(64):
                row = nt * 32 + lane % 32
                col = kt * 32 + 16 * (lane // 32)
                if row < n and col < k:
                    off = ((nt * kt_n + kt) * 64 + lane) * 16
                    ref[off : off + 16] = codes[row, col : col + 16]
    assert torch.equal(packed, ref)


@pytest.mark.parametrize("k,n", GEMM_SHAPES)
@pytest.mark.parametrize("m", GEMM_MS)
def test_gemm_sweep(tk, m, k, n):
    x, w8, s = gemm_case(m, k, n)
    want = oops.lin_fp8w(x, w8, s)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    got = tk.fp8w_gemm(x.cuda(), pw)
    torch.cuda.synchronize()
    _close(got, want, f"gemm M={m} K={k} N={n}")


@pytest.mark.parametrize("split", [1, 2, 5, 16])
def test_gemm_split_k_equals_no_split_within_tolerance_and_is_deterministic(tk, split):
    x, w8, s = gemm_case(50, 2048, 2048)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    xc = x.cuda()
    a = tk.fp8w_gemm(xc, pw, split_k=split)
    b = tk.fp8w_gemm(xc, pw, split_k=split)
    torch.cuda.synchronize()
    assert torch.equal(a, b), "same launch twice must give the same bits (fixed-order reduction)"
    _close(a, oops.lin_fp8w(x, w8, s), f"gemm split_k={split}")


@pytest.mark.parametrize("m,k,n", [(3, 16, 32), (5, 32, 37), (40, 96, 130), (33, 48, 40), (50, 720, 720), (64, 80, 96), (241, 960, 2560), (130, 2048, 320)])
def test_gemm_ragged_shapes(tk, m, k, n):
    x, w8, s = gemm_case(m, k, n)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    got = tk.fp8w_gemm(x.cuda(), pw)
    _close(got, oops.lin_fp8w(x, w8, s), f"gemm ragged M={m} K={k} N={n}")


def test_gemm_strided_input_and_residual(tk):
    x, w8, s = gemm_case(50, 720, 2048)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    wide = torch.zeros(50, 1440, dtype=torch.bfloat16, device="cuda")
    wide[:, :720] = x.cuda()
    g = torch.Generator().manual_seed(9)
    for rdt in (torch.bfloat16, torch.float32):
        resid = torch.randn(50, 2048, generator=g).to(rdt)
        got = tk.fp8w_gemm(wide[:, :720], pw, resid=resid.cuda())
        y = oops.lin_fp8w(x, w8, s)
        y += resid  # the reference's in-place add: fp32 math, bf16 result
        _close(got, y, f"gemm+resid {rdt}")


def test_gemm_linearity_at_full_size(tk):
    # size-independent property at the largest sweep shape: scaling x by 2 scales y by 2 bit-exactly
    x, w8, s = gemm_case(64, 16384, 2048)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    a = tk.fp8w_gemm(x.cuda(), pw)
    b = tk.fp8w_gemm((x * 2).cuda(), pw)
    assert torch.equal((a.float() * 2).to(torch.bfloat16), b)


def test_gemm_rejects_bad_arguments(tk):
    x, w8, s = gemm_case(4, 32, 32)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    with pytest.raises(TypeError):
        tk.fp8w_gemm(x.float().cuda(), pw)
    with pytest.raises(ValueError):
        tk.fp8w_gemm(x.cuda()[:, :16], pw)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        tk.pack_fp8_weight(torch.zeros(32, 24, dtype=torch.uint8, device="cuda"), torch.ones(32))


@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("m,k,i", [(50, 720, 2048), (50, 1024, 4096), (1, 720, 2048), (64, 960, 2560)])
def test_gated_ffn(tk, act, m, k, i):
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(m, k, i, seed=0)
    want = oops.gated_ffn(x, wg8, sg, wu8, su, wd8, sd, act)
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    got = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, act)
    again = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, act)
    assert torch.equal(got, again)
    _close(got, want, f"ffn {act} M={m} K={k} I={i}")


def test_gated_ffn_residual(tk):
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(50, 720, 2048, seed=1)
    resid = torch.randn(50, 720, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    want = oops.gated_ffn(x, wg8, sg, wu8, su, wd8, sd, "silu")
    want += resid
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    got = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, "silu", resid=resid.cuda())
    _close(got, want, "ffn+resid")


ATTN_CASES = [
    # m, p, h, g, d, mode, bf16_logits
    (50, 241, 15, 5, 64, oops.MASK_BIDIR, False),   # config 3
    (50, 241, 15, 5, 64, oops.MASK_CAUSAL, False),  # SmolVLA self layer, 3 cameras
    (50, 177, 15, 5, 64, oops.MASK_CAUSAL, False),  # 2 cameras
    (50, 712, 8, 1, 256, oops.MASK_BIDIR, True),    # pi0.5 expert
    (7, 5, 4, 2, 64, oops.MASK_CAUSAL, False),      # tiny, ragged
    (33, 95, 4, 4, 128, oops.MASK_BIDIR, False),
    # 256-wide heads take the kernel that cuts the two products along different axes (rounds of 8 key tiles)
    (50, 712, 8, 1, 256, oops.MASK_CAUSAL, False),  # 4 key splits, causal suffix, fp32 logits
    (7, 5, 4, 2, 256, oops.MASK_CAUSAL, True),      # one block of two key tiles: six idle waves
    (50, 230, 8, 1, 256, oops.MASK_BIDIR, True),    # 2 splits of 5 tiles
    (33, 1900, 2, 2, 256, oops.MASK_BIDIR, False),  # 8 splits (the most) of one round each
    (40, 2100, 2, 1, 256, oops.MASK_BIDIR, True),   # 8 splits of two rounds (8 + 1 tiles; the suffix in the last)
]


@pytest.mark.parametrize("m,p,h,g,d,mode,bl", ATTN_CASES)
def test_expert_attention(tk, m, p, h, g, d, mode, bl):
    q, k_pre, v_pre, k_suf, v_suf = attn_case(m, p, h, g, d, seed=0)
    pad = torch.ones(p, dtype=torch.bool)
    pad[torch.randperm(p, generator=torch.Generator().manual_seed(3))[: p // 7]] = False
    want = oops.expert_attention(q, k_pre, v_pre, k_suf, v_suf, pad, mode, bf16_logits=bl)
    got = tk.expert_attn_plain(q.cuda(), k_pre.cuda(), v_pre.cuda(), k_suf.cuda(), v_suf.cuda(), pad.cuda(), mode, logits_bf16=bl)
    again = tk.expert_attn_plain(q.cuda(), k_pre.cuda(), v_pre.cuda(), k_suf.cuda(), v_suf.cuda(), pad.cuda(), mode, logits_bf16=bl)
    assert torch.equal(got, again)
    _close(got, want, f"attn M={m} P={p} H={h} G={g} D={d} mode={mode}")


def test_cross_attention_fp32_kv(tk):
    # SmolVLA cross layers: fp32 expert K/V over the prefix only, fp32 P.V
    q, k_pre, v_pre, _, _ = attn_case(50, 241, 15, 5, 64, seed=1, kv_dtype=torch.float32)
    pad = torch.ones(241, dtype=torch.bool)
    pad[200:] = False
    want = oops.expert_attention(q, k_pre, v_pre, None, None, pad, oops.MASK_NONE)
    got = tk.expert_attn_plain(q.cuda(), k_pre.cuda(), v_pre.cuda(), None, None, pad.cuda(), oops.MASK_NONE)
    assert want.dtype == torch.float32
    _close(got, want.to(torch.bfloat16), "cross attn fp32 kv")


def test_attention_strided_kv_cache_views(tk):
    # K/V as slices of a [L, G, D] cache buffer (suffix right behind the prefix), and head-major prefix
    q, k_pre, v_pre, k_suf, v_suf = attn_case(50, 177, 15, 5, 64, seed=2)
    kbuf = torch.cat([k_pre, k_suf]).cuda()
    vbuf = torch.cat([v_pre, v_suf]).cuda()
    want = oops.expert_attention(q, k_pre, v_pre, k_suf, v_suf, torch.ones(177, dtype=torch.bool), oops.MASK_CAUSAL)
    got = tk.expert_attn_plain(q.cuda(), kbuf[:177], vbuf[:177], kbuf[177:], vbuf[177:], None, oops.MASK_CAUSAL)
    _close(got, want, "attn cache views")
    k_hm = k_pre.permute(1, 0, 2).contiguous().cuda().permute(1, 0, 2)  # [P, G, D] view of [G, P, D]
    v_hm = v_pre.permute(1, 0, 2).contiguous().cuda().permute(1, 0, 2)
    got = tk.expert_attn_plain(q.cuda(), k_hm, v_hm, k_suf.cuda(), v_suf.cuda(), None, oops.MASK_CAUSAL)
    _close(got, want, "attn head-major prefix")


@pytest.mark.parametrize("h,g,d", [(15, 5, 64), (8, 1, 256)])
def test_attention_fully_masked_prefix_is_uniform(tk, h, g, d):
    q, k_pre, v_pre, _, _ = attn_case(50, 64, h, g, d, seed=3)
    none = torch.zeros(64, dtype=torch.bool)
    want = oops.expert_attention(q, k_pre, v_pre, None, None, none, oops.MASK_NONE)
    got = tk.expert_attn_plain(q.cuda(), k_pre.cuda(), v_pre.cuda(), None, None, none.cuda(), oops.MASK_NONE)
    _close(got, want, "attn fully masked")


@pytest.mark.parametrize("p,h,g,d", [(241, 15, 5, 64), (177, 15, 5, 64), (100, 15, 5, 64), (384, 6, 2, 64), (385, 6, 2, 64), (40, 4, 2, 128), (1024, 12, 12, 64), (712, 8, 1, 256), (90, 4, 2, 256), (1000, 16, 2, 256)])
def test_prefill_attention_with_2d_mask(tk, p, h, g, d):
    # the VLM prefill: every token is a query, keys are the same tokens, visibility from the
    # block-causal 2-D mask (image/language tokens see each other, the state token sees all) & padding
    q, k, v, _, _ = attn_case(p, p, h, g, d, seed=4)
    gen = torch.Generator().manual_seed(5)
    pad = torch.rand(p, generator=gen) > 0.1
    att = torch.zeros(p, dtype=torch.bool)
    att[-1] = True
    mask = oops.make_att_2d_masks(pad[None], att[None])[0]
    want = oops.eager_attention(mask[None], q[None], k[None], v[None])[0]
    p_pad = (p + 31) // 32 * 32
    m2 = torch.zeros(p, p_pad, dtype=torch.uint8)
    m2[:, :p] = mask
    pre = tk.prepare_prefix_kv(k.cuda(), v.cuda())
    got = tk.expert_attn(q.cuda(), pre, None, None, oops.MASK_NONE, mask2d=m2.cuda())
    again = tk.expert_attn(q.cuda(), pre, None, None, oops.MASK_NONE, mask2d=m2.cuda())
    assert torch.equal(got, again)
    _close(got, want, f"prefill attention P={p} H={h} D={d}")


def test_batched_vision_attention(tk):
    # three images' self-attention in one launch, bf16-rounded logits as the torch bf16 matmul path gives
    b, m, h, d = 3, 256, 12, 64
    g = torch.Generator().manual_seed(6)
    qkv = torch.randn(b, m, 3, h, d, generator=g).to(torch.bfloat16)
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))  # [b, h, m, d]
    att = torch.softmax(torch.matmul(q, k.transpose(2, 3)).float() * d**-0.5, dim=-1).to(v.dtype)
    want = torch.matmul(att, v).transpose(1, 2).reshape(b, m, h * d)
    dev = qkv.cuda()
    vt = dev[:, :, 2].permute(0, 2, 3, 1).contiguous()
    got = tk.batched_attn(dev[:, :, 0], dev[:, :, 1], vt, logits_bf16=True)
    _close(got, want, "batched vision attention")


@pytest.mark.parametrize(
    "b,m,p,h,g,d",
    [(3, 1024, 1024, 12, 12, 64), (3, 1000, 1000, 12, 12, 64), (6, 520, 300, 12, 4, 64), (2, 1024, 640, 12, 12, 64), (2, 200, 200, 4, 4, 64),
     (1, 130, 300, 6, 2, 64), (2, 160, 160, 3, 3, 96), (1, 128, 129, 2, 1, 96), (5, 1024, 320, 16, 16, 96)],
)  # fmt: skip
def test_tower_attention_ragged_shapes(tk, b, m, p, h, g, d):
    # the many-query path (128 queries per block, keys in stages of 64): full SmolVLA tower shape, query and
    # key counts that end inside a tile / a stage, grouped heads, both head sizes; zero-padded V^T keys.  On a
    # 256-CU device the first two shapes take the five-tile blocks (288 four-tile blocks would double up on some
    # CUs, 252 five-tile blocks fit one per CU; the second ends inside a block, a tile and a stage), the third the
    # four-tile blocks two per CU (360 blocks), the fourth the four-tile blocks one per CU (192), the next four the
    # two-tile blocks (grids that would leave more than half of the CUs idle), the last the four-tile blocks at head size 96
    gen = torch.Generator().manual_seed(17)
    q = torch.randn(b, m, h, d, generator=gen).to(torch.bfloat16)
    k = torch.randn(b, p, g, d, generator=gen).to(torch.bfloat16)
    v = torch.randn(b, p, g, d, generator=gen).to(torch.bfloat16)
    rep = h // g
    kk, vv = k.repeat_interleave(rep, dim=2).float(), v.repeat_interleave(rep, dim=2).float()
    logits = torch.einsum("bmhd,bphd->bhmp", q.float(), kk).to(torch.bfloat16).float() * d**-0.5
    probs = torch.softmax(logits, dim=-1).to(torch.bfloat16).float()
    want = torch.einsum("bhmp,bphd->bmhd", probs, vv).to(torch.bfloat16).reshape(b, m, h * d)
    p_pad = (p + 31) // 32 * 32
    vt = torch.zeros(b, g, d, p_pad, dtype=torch.bfloat16)
    vt[..., :p] = v.permute(0, 2, 3, 1)
    got = tk.batched_attn(q.cuda(), k.cuda(), vt.cuda(), logits_bf16=True)
    again = tk.batched_attn(q.cuda(), k.cuda(), vt.cuda(), logits_bf16=True)
    assert torch.equal(got, again)
    _close(got, want, f"tower attention B={b} M={m} P={p} H={h} G={g} D={d}")


@pytest.mark.parametrize("b,p,g,d", [(3, 1024, 12, 64), (2, 256, 16, 96), (1, 200, 3, 64), (2, 33, 2, 96)])
def test_batched_value_transpose(tk, b, p, g, d):
    # V^T operand straight from a packed q|k|v buffer: exact copy, zero padding keys
    gen = torch.Generator().manual_seed(23)
    qkv = torch.randn(b, p, 3, g, d, generator=gen).to(torch.bfloat16).cuda()
    p_pad = (p + 31) // 32 * 32
    out = torch.full((b, g, d, p_pad + 8), 7.0, dtype=torch.bfloat16, device="cuda")[..., :p_pad]  # rows longer than the operand
    got = tk.transpose_v(qkv[:, :, 2], out=out)
    assert torch.equal(got[..., :p], qkv[:, :, 2].permute(0, 2, 3, 1))
    assert torch.count_nonzero(got[..., p:]) == 0
    assert torch.equal(tk.transpose_v(qkv[:, :, 2]), got)
    with pytest.raises(RuntimeError):
        tk.transpose_v(torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16, device="cuda"))


def test_batched_attention_padded_head_with_explicit_scale(tk):
    # SigLIP-So400m heads are 72 wide: run as 96-wide heads whose last 24 columns are zero, with the
    # logit scale of the true size; the padded output columns must come back as zeros
    b, length, heads, hd, hp = 2, 256, 16, 72, 96
    g = torch.Generator().manual_seed(31)
    q, k, v = (torch.randn(b, length, heads, hd, generator=g).to(torch.bfloat16) for _ in range(3))
    pad = lambda t: torch.nn.functional.pad(t, (0, hp - hd))  # noqa: E731
    vt = pad(v).permute(0, 2, 3, 1).contiguous()
    got = tk.batched_attn(pad(q).cuda(), pad(k).cuda(), vt.cuda(), scale=hd**-0.5).cpu().view(b, length, heads, hp)
    assert torch.count_nonzero(got[..., hd:]) == 0
    probs = torch.softmax(torch.einsum("blhd,bmhd->bhlm", q.float(), k.float()) * hd**-0.5, dim=-1).to(torch.bfloat16)
    want = torch.einsum("bhlm,bmhd->blhd", probs.float(), v.float()).to(torch.bfloat16)
    _close(got[..., :hd], want, "padded-head batched attention")


@pytest.mark.parametrize("layers,p,kv,n", [(8, 241, 320, 320), (16, 177, 320, 320), (3, 33, 208, 64), (1, 40, 96, 128)])
def test_kv_projection_of_several_layers_in_one_launch_gives_the_single_launches_bits(tk, layers, p, kv, n):
    # the cross layers' projections are independent: one launch over all of them must write, layer by layer, the
    # planes that one launch per layer writes (inputs strided like the per-layer q|k|v rows of the prefill)
    g = torch.Generator().manual_seed(43)
    wide = torch.randn(layers, p, 4 * kv, generator=g).to(torch.bfloat16).cuda()
    ks, vs = [wide[i, :, 2 * kv : 3 * kv] for i in range(layers)], [wide[i, :, 3 * kv :] for i in range(layers)]
    wks = [(torch.randn(n, kv, generator=g) * kv**-0.5).cuda() for _ in range(layers)]
    wvs = [(torch.randn(n, kv, generator=g) * kv**-0.5).cuda() for _ in range(layers)]
    got = tk.project_prefix_kv_layers(ks, vs, wks, wvs, 64)
    assert len(got) == layers
    for i in range(layers):
        one = tk.project_prefix_kv(ks[i], vs[i], wks[i], wvs[i], 64)
        for name in ("k", "k_lo", "vt", "vt_lo"):
            assert torch.equal(getattr(got[i], name), getattr(one, name)), (i, name)
    with pytest.raises(ValueError):
        tk.project_prefix_kv_layers(ks * 17, vs * 17, wks * 17, wvs * 17, 64)


@pytest.mark.parametrize("p,kv,n,d", [(241, 320, 320, 64), (177, 320, 320, 64), (40, 96, 128, 64), (33, 208, 64, 64)])
def test_expert_kv_projection_into_attention_planes(tk, p, kv, n, d):
    # float(K) @ Wk^T / float(V) @ Wv^T in fp32, delivered as the attention kernel's hi + lo planes:
    # hi + lo must reproduce the fp32 projection to ~2^-16, the padded V^T keys must be zero, and the
    # attention over the planes must equal the attention over the torch projection
    g = torch.Generator().manual_seed(41)
    wide = torch.randn(p, 4 * kv, generator=g).to(torch.bfloat16).cuda()  # rows strided like a q|k|v buffer
    k, v = wide[:, 2 * kv : 3 * kv], wide[:, 3 * kv :]
    wk, wv = (torch.randn(n, kv, generator=g) * kv**-0.5).cuda(), (torch.randn(n, kv, generator=g) * kv**-0.5).cuda()
    cache = tk.project_prefix_kv(k, v, wk, wv, d)
    ek = (k.float().cpu().double() @ wk.cpu().double().T).float()
    ev = (v.float().cpu().double() @ wv.cpu().double().T).float()
    got_k = (cache.k.float() + cache.k_lo.float()).cpu().reshape(p, n)
    got_vt = (cache.vt.float() + cache.vt_lo.float()).cpu()
    assert float((got_k - ek).abs().max()) <= 3e-5 * max(1.0, float(ek.abs().max()))
    assert float((got_vt[:, :, :p].reshape(n, p).T - ev).abs().max()) <= 3e-5 * max(1.0, float(ev.abs().max()))
    assert torch.count_nonzero(got_vt[:, :, p:]) == 0
    # same bits on a second call (fixed accumulation order)
    again = tk.project_prefix_kv(k, v, wk, wv, d)
    assert torch.equal(again.k, cache.k) and torch.equal(again.k_lo, cache.k_lo) and torch.equal(again.vt_lo, cache.vt_lo)
    heads = n // d
    q = torch.randn(50, heads * 3, d, generator=g).to(torch.bfloat16).cuda()
    ref_cache = tk.prepare_prefix_kv(ek.view(p, heads, d).cuda(), ev.view(p, heads, d).cuda())
    a = tk.expert_attn(q, cache, None, None, tk.MASK_NONE)
    b = tk.expert_attn(q, ref_cache, None, None, tk.MASK_NONE)
    _close(a, b.cpu(), "attention over projected planes")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,k", [(512, 1152), (3072, 768), (5, 8), (131, 2048)])
def test_layer_norm_with_folded_cast(tk, dtype, m, k):
    # F.layer_norm in fp32 statistics, result rounded once to bf16 -- for fp32 rows (pi0.5 tower, followed
    # by .to(bf16) in the reference's low-precision tiers) and bf16 rows (SmolVLA tower)
    g = torch.Generator().manual_seed(61)
    x = (torch.randn(m, k, generator=g) * 3.0 + 0.5).to(dtype)
    w, b = (1.0 + 0.3 * torch.randn(k, generator=g)).to(dtype), (0.2 * torch.randn(k, generator=g)).to(dtype)
    want = torch.nn.functional.layer_norm(x.float(), (k,), w.float(), b.float(), 1e-6).to(torch.bfloat16)
    got = tk.layer_norm(x.cuda(), w.cuda(), b.cuda(), 1e-6)
    assert got.dtype == torch.bfloat16 and got.shape == x.shape
    diff = (got.float().cpu() - want.float()).abs()
    ulp = want.float().abs().clamp_min(2.0**-6) * 2.0**-7  # one bf16 step at the value's magnitude
    assert bool((diff <= ulp).all()), f"max |err| {float(diff.max()):.4g}: more than one bf16 step from the fp32 LayerNorm"
    assert float((diff > 0).float().mean()) < 0.02, "more than 2% of the outputs differ from the fp32 LayerNorm rounded once"
    with pytest.raises(TypeError):
        tk.layer_norm(x.cuda(), w.float().cuda(), b.half().cuda(), 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,k", [(512, 1152), (3072, 768), (5, 8)])
def test_residual_add_and_layer_norm_in_one_launch(tk, dtype, m, k):
    # x += r (the sum in x's type: exact for fp32 rows, rounded once for bf16 rows), then the LayerNorm of the sum
    g = torch.Generator().manual_seed(62)
    x = (torch.randn(m, k, generator=g) * 2.0).to(dtype)
    r = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w, b = (1.0 + 0.3 * torch.randn(k, generator=g)).to(dtype), (0.2 * torch.randn(k, generator=g)).to(dtype)
    want_sum = x + r  # torch promotes bf16 to fp32 for fp32 x; bf16 + bf16 rounds once
    assert want_sum.dtype == dtype
    want = torch.nn.functional.layer_norm(want_sum.float(), (k,), w.float(), b.float(), 1e-6).to(torch.bfloat16)
    xd = x.cuda()
    got_x, got = tk.add_layer_norm(xd, r.cuda(), w.cuda(), b.cuda(), 1e-6)
    assert got_x.data_ptr() == xd.data_ptr() and torch.equal(got_x.cpu(), want_sum)
    diff = (got.float().cpu() - want.float()).abs()
    assert bool((diff <= want.float().abs().clamp_min(2.0**-6) * 2.0**-7).all())
    assert float((diff > 0).float().mean()) < 0.02
    assert torch.equal(got, tk.layer_norm(got_x, w.cuda(), b.cuda(), 1e-6))  # same kernel arithmetic after the add


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,k", [(3072, 768), (64, 1152), (5, 8)])
def test_residual_add_and_layer_norm_with_a_row_permutation(tk, dtype, m, k):
    # the normalised rows written in another order (the pixel shuffle behind a tower's closing LayerNorm): row i of
    # the plain launch must be row y_rows[i] here, bit for bit, and the in-place sum stays where it is
    g = torch.Generator().manual_seed(63)
    x = (torch.randn(m, k, generator=g) * 2.0).to(dtype).cuda()
    r = torch.randn(m, k, generator=g).to(torch.bfloat16).cuda()
    w, b = (1.0 + 0.3 * torch.randn(k, generator=g)).to(dtype).cuda(), (0.2 * torch.randn(k, generator=g)).to(dtype).cuda()
    rows = torch.randperm(m, generator=g).to(torch.int32).cuda()
    plain_x, plain = tk.add_layer_norm(x.clone(), r, w, b, 1e-6)
    got_x, got = tk.add_layer_norm(x.clone(), r, w, b, 1e-6, y_rows=rows)
    assert torch.equal(got_x, plain_x)
    assert torch.equal(got[rows.long()], plain)
    with pytest.raises(ValueError):
        tk.add_layer_norm(x.clone(), r, w, b, 1e-6, y_rows=rows.long())
    with pytest.raises(ValueError):
        tk.add_layer_norm(x.clone(), r, w, b, 1e-6, y_rows=rows[: m - 1])


def test_gated_residual_epilogue(tk):
    # pi0.5 AdaRMS gated residual: y = resid + bf16(ffn(x) * gate)
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(50, 1024, 4096, seed=3)
    g = torch.Generator().manual_seed(4)
    resid = torch.randn(50, 1024, generator=g).to(torch.bfloat16)
    gate = torch.randn(1024, generator=g).to(torch.bfloat16)
    want = resid + oops.gated_ffn(x, wg8, sg, wu8, su, wd8, sd, "gelu_tanh") * gate
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    got = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, "gelu_tanh", resid=resid.cuda(), gate=gate.cuda())
    _close(got, want, "ffn gated residual")
    pw = tk.pack_fp8_weight(wd8.cuda(), sd)
    h = torch.randn(50, 4096, generator=g).to(torch.bfloat16)
    want = resid + oops.lin_fp8w(h, wd8, sd) * gate
    got = tk.fp8w_gemm(h.cuda(), pw, resid=resid.cuda(), gate=gate.cuda())
    _close(got, want, "gemm gated residual")


@pytest.mark.parametrize("m,k,n", [(3072, 768, 3072), (512, 1152, 4304), (7, 64, 96)])
def test_linear_gelu_tanh_is_the_tanh_form_of_the_two_launch_op(tk, m, k, n):
    """The vision towers' fc1 + GELU as one library GEMM (activation in the epilogue) against the two-launch
    form of the reference (vision.py: ``gelu_pytorch_tanh(fc1(x))``) on the CPU, and -- on the rows where the
    tanh and the erf form differ most -- against both closed forms in fp64: it has to be the tanh one."""
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) * 1.5 * k**-0.5).to(torch.bfloat16)
    b = torch.randn(n, generator=g).to(torch.bfloat16)
    got = tk.linear_gelu_tanh(x.cuda(), w.cuda(), b.cuda())
    want = torch.nn.functional.gelu(torch.nn.functional.linear(x, w, b), approximate="tanh")
    _close(got, want, f"linear_gelu_tanh {m}x{k}->{n}")
    z = x.double() @ w.double().t() + b.double()
    sel = (z.abs() > 1.0) & (z.abs() < 3.0)
    if int(sel.sum()) > 100_000:
        err_tanh = (got.cpu().double() - torch.nn.functional.gelu(z, approximate="tanh"))[sel]
        err_erf = (got.cpu().double() - torch.nn.functional.gelu(z))[sel]
        # the two forms differ by 2.2e-5 on average over this range; rounding noise averages out
        assert abs(float(err_tanh.mean())) < 6e-6 < abs(float(err_erf.mean()))


@pytest.mark.parametrize("h,g,d,mode", [(15, 5, 64, oops.MASK_CAUSAL), (8, 1, 256, oops.MASK_BIDIR), (4, 2, 128, oops.MASK_CAUSAL)])
def test_attention_over_the_suffix_alone_and_with_whole_key_tiles_masked(tk, h, g, d, mode):
    # no prefix at all (the first tile is then a suffix tile), and a prefix whose pad mask removes two whole
    # 32-key tiles plus a ragged remainder: a masked tile must contribute exactly nothing
    q, k_pre, v_pre, k_suf, v_suf = attn_case(50, 200, h, g, d, seed=9)
    bl = d == 256
    want = oops.expert_attention(q, k_pre[:0], v_pre[:0], k_suf, v_suf, torch.ones(0, dtype=torch.bool), mode, bf16_logits=bl)
    got = tk.expert_attn_plain(q.cuda(), None, None, k_suf.cuda(), v_suf.cuda(), None, mode, logits_bf16=bl)
    _close(got, want, f"suffix-only attention D={d}")
    pad = torch.ones(200, dtype=torch.bool)
    pad[32:96] = False
    pad[190:] = False
    want = oops.expert_attention(q, k_pre, v_pre, k_suf, v_suf, pad, mode, bf16_logits=bl)
    got = tk.expert_attn_plain(q.cuda(), k_pre.cuda(), v_pre.cuda(), k_suf.cuda(), v_suf.cuda(), pad.cuda(), mode, logits_bf16=bl)
    _close(got, want, f"attention with whole key tiles masked D={d}")

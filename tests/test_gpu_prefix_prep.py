"""GPU parity of the per-request bookkeeping launches against the tensor operations they replace.

`tk_prefix_meta`: `make_att_2d_masks`, `cumsum(pad_masks) - 1` and `prefix_pad.sum(-1) + arange(S)`
(tybok/policies/smolvla/models/flow_matching.py:40-58,343-350,527-546; tybok/policies/pi05/models/flow_matching.py:
440-470 with no attention blocks) -- integer / byte results, compared exactly.
`tk_patchify_images`: `images * 2 - 1`, the cast to bf16 and the unfolding in front of the patch GEMM
(tybok/policies/smolvla/policy.py:117-163, tybok/policies/smolvla/models/vision.py:120-160) -- compared exactly.
`tk_prefix_rows`: the scaled image rows, the scaled embedding rows of the language tokens and the state row concatenated
in fp32, with their pad flags (tybok/policies/smolvla/models/flow_matching.py:160-257) -- compared exactly.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tk():
    from tybok_amd import ops

    return ops


def _meta_reference(pad, att, positions, s):
    c = torch.cumsum(att.long(), dim=0)
    mask = (c[None, :] <= c[:, None]) & (pad[None, :] & pad[:, None])
    pos = (torch.cumsum(pad.long(), dim=0) - 1).clamp(0, positions - 1).to(torch.int32)
    suf = (pad.long().sum() + torch.arange(s)).clamp(0, positions - 1).to(torch.int32)
    return mask.to(torch.uint8), pos, suf


@pytest.mark.parametrize("p_len,s", [(1, 1), (31, 7), (241, 50), (712, 50), (1000, 64), (2048, 3)])
@pytest.mark.parametrize("with_att", [False, True])
def test_prefix_meta_matches_the_tensor_operations(tk, p_len, s, with_att):
    g = torch.Generator().manual_seed(p_len * 7 + s)
    pad = torch.rand(p_len, generator=g) < 0.8
    att = (torch.rand(p_len, generator=g) < 0.05) if with_att else torch.zeros(p_len, dtype=torch.bool)
    want_mask, want_pos, want_suf = _meta_reference(pad, att, 16384, s)
    mask2d, pos32, suf = tk.prefix_meta(pad.cuda(), att.cuda() if with_att else None, 16384, s)
    p_pad = (p_len + 31) // 32 * 32
    assert mask2d.shape == (p_len, p_pad) and mask2d.dtype == torch.uint8
    assert torch.equal(mask2d[:, :p_len].cpu(), want_mask)
    assert not bool(mask2d[:, p_len:].any()), "the padding columns must be zero"
    assert torch.equal(pos32.cpu(), want_pos)
    assert torch.equal(suf.cpu(), want_suf)


def test_prefix_meta_edge_cases_and_clamping(tk):
    # nothing valid: positions clamp at 0, the mask is empty; everything valid with a short table: clamped at its end;
    # the SmolVLA prefix: one attention block that starts at the last token (the state), so no other row sees it
    pad = torch.zeros(100, dtype=torch.bool)
    m, p, sfx = tk.prefix_meta(pad.cuda(), None, 16384, 5)
    assert not bool(m.any()) and not bool(p.any()) and sfx.tolist() == [0, 1, 2, 3, 4]
    pad = torch.ones(100, dtype=torch.bool)
    m, p, sfx = tk.prefix_meta(pad.cuda(), None, 64, 5)
    assert p.tolist() == [min(i, 63) for i in range(100)] and sfx.tolist() == [63] * 5
    assert bool((m[:, :100] == 1).all())
    att = torch.zeros(100, dtype=torch.bool)
    att[-1] = True
    m, _, _ = tk.prefix_meta(pad.cuda(), att.cuda(), 16384, 0, want_mask=True)
    assert bool((m[:99, 99] == 0).all()) and bool((m[99, :100] == 1).all()) and bool((m[:99, :99] == 1).all())
    m, p, sfx = tk.prefix_meta(pad.cuda(), None, 16384, 0, want_mask=False)
    assert m is None and sfx is None and p.tolist() == list(range(100))


def test_prefix_meta_argument_rules(tk):
    with pytest.raises(TypeError):
        tk.prefix_meta(torch.ones(8, dtype=torch.uint8, device="cuda"), None, 16384)
    with pytest.raises(TypeError):
        tk.prefix_meta(torch.ones(8, dtype=torch.bool, device="cuda"), torch.ones(9, dtype=torch.bool, device="cuda"), 16384)
    with pytest.raises(RuntimeError, match="P="):
        tk.prefix_meta(torch.ones(2049, dtype=torch.bool, device="cuda"), None, 16384)


@pytest.mark.parametrize("n,h,w,ps", [(1, 32, 32, 16), (3, 512, 512, 16), (2, 64, 96, 8), (4, 48, 48, 24)])
def test_patchify_images_matches_scale_cast_unfold(tk, n, h, w, ps):
    g = torch.Generator().manual_seed(n * 100 + ps)
    images = [(torch.randint(0, 256, (1, 3, h, w), generator=g, dtype=torch.uint8).float() / 255.0) for _ in range(n)]
    x = torch.cat([img * 2.0 - 1.0 for img in images], dim=0).to(torch.bfloat16)
    want = x.view(n, 3, h // ps, ps, w // ps, ps).permute(0, 2, 4, 1, 3, 5).reshape(n, (h // ps) * (w // ps), 3 * ps * ps)
    got = tk.patchify_images([img.cuda() for img in images], ps, 2.0, -1.0)
    assert got.shape == want.shape and got.dtype == torch.bfloat16
    assert torch.equal(got.cpu(), want)
    # a scale that is not a power of two: product and sum must round one after the other, as the two tensor operations do
    want2 = torch.cat([img * 0.3 + 0.1 for img in images], dim=0).to(torch.bfloat16)
    want2 = want2.view(n, 3, h // ps, ps, w // ps, ps).permute(0, 2, 4, 1, 3, 5).reshape(want.shape)
    got2 = tk.patchify_images([img.cuda() for img in images], ps, 0.3, 0.1)
    assert torch.equal(got2.cpu(), want2)


@pytest.mark.parametrize("n,h,w,ps", [(2, 224, 224, 14), (1, 28, 42, 14), (4, 24, 24, 6), (3, 32, 32, 16)])
def test_patchify_images_in_fp32_with_any_even_patch(tk, n, h, w, ps):
    # the fp32 form (14 x 14 patches in front of an fp32 patch embedding): x * 2 - 1 and the unfolding, bit for bit
    g = torch.Generator().manual_seed(n * 100 + ps)
    images = [torch.rand(1, 3, h, w, generator=g) for _ in range(n)]
    for scale, shift in ((2.0, -1.0), (0.3, 0.1)):
        x = torch.cat([img * scale + shift for img in images], dim=0)
        want = x.view(n, 3, h // ps, ps, w // ps, ps).permute(0, 2, 4, 1, 3, 5).reshape(n, (h // ps) * (w // ps), 3 * ps * ps)
        got = tk.patchify_images([img.cuda() for img in images], ps, scale, shift, out_dtype=torch.float32)
        assert got.dtype == torch.float32 and got.shape == want.shape
        assert torch.equal(got.cpu(), want)
    with pytest.raises(RuntimeError, match="patch"):
        tk.patchify_images([torch.zeros(1, 3, 21, 21, device="cuda")], 7, out_dtype=torch.float32)  # odd patch size


def test_patchify_images_argument_rules(tk):
    img = torch.zeros(1, 3, 32, 32, device="cuda")
    with pytest.raises(ValueError):
        tk.patchify_images([], 16)
    with pytest.raises(TypeError):
        tk.patchify_images([img.half()], 16)
    with pytest.raises(RuntimeError, match="patch"):
        tk.patchify_images([img], 12)  # not a multiple of 8
    with pytest.raises(RuntimeError, match="patch"):
        tk.patchify_images([torch.zeros(1, 3, 40, 40, device="cuda")], 16)  # does not divide the image


@pytest.mark.parametrize("cams,per_cam,n_tok,h", [(3, 64, 48, 960), (1, 64, 48, 960), (4, 16, 7, 64), (2, 5, 1, 8)])
def test_prefix_rows_are_the_scaled_concatenation(tk, cams, per_cam, n_tok, h):
    # image rows times a bf16-rounded scale, gathered embedding rows times sqrt(H), the projected state row, all
    # widened to fp32, and the pad flags of those rows: bit for bit what the tensor operations build
    import math

    g = torch.Generator().manual_seed(70 + cams)
    img = torch.randn(cams, per_cam, h, generator=g).to(torch.bfloat16).cuda()
    table = torch.randn(300, h, generator=g).to(torch.bfloat16).cuda()
    tokens = torch.randint(0, 300, (n_tok,), generator=g).cuda()
    last = torch.randn(1, h, generator=g).cuda()
    scale = torch.tensor(h**0.5, dtype=torch.bfloat16)
    cam_flags = [torch.tensor([bool(i != 1)]).cuda() for i in range(cams)]
    tok_flags = (torch.rand(n_tok, generator=g) < 0.7).cuda()
    got, flags = tk.prefix_rows(img, float(scale), table, tokens, math.sqrt(h), last, cam_flags=cam_flags, tok_flags=tok_flags)
    lang = torch.nn.functional.embedding(tokens[None], table) * math.sqrt(h)
    want = torch.cat([(img * scale.cuda()).reshape(1, -1, h).float(), lang.float(), last[None]], dim=1)
    assert got.dtype == torch.float32 and torch.equal(got, want)
    want_flags = torch.cat([f[:, None].expand(1, per_cam) for f in cam_flags] + [tok_flags[None], torch.ones(1, 1, dtype=torch.bool).cuda()], dim=1)
    assert flags.dtype == torch.bool and torch.equal(flags, want_flags)
    plain, none = tk.prefix_rows(img, float(scale), table, tokens, math.sqrt(h), last)
    assert none is None and torch.equal(plain, want)
    with pytest.raises(TypeError):
        tk.prefix_rows(img.half(), float(scale), table, tokens, math.sqrt(h), last)
    with pytest.raises(ValueError):
        tk.prefix_rows(img, float(scale), table, tokens, math.sqrt(h), last, cam_flags=cam_flags[:-1] or [None, None], tok_flags=tok_flags)


@pytest.mark.parametrize("cams,per_cam,n_tok,h", [(2, 256, 200, 2048), (1, 256, 40, 2048), (3, 7, 5, 64)])
def test_prefix_rows_from_fp32_image_rows_in_bf16(tk, cams, per_cam, n_tok, h):
    # fp32 image rows as they are, embedding rows times a bf16-rounded scale, no closing rows, everything rounded to
    # bf16: the hidden rows a prefill takes from `cat(...).to(bfloat16)`, bit for bit; and the same in fp32
    g = torch.Generator().manual_seed(80 + cams)
    img = (torch.randn(cams, per_cam, h, generator=g) * 3.0).cuda()
    table = torch.randn(500, h, generator=g).to(torch.bfloat16).cuda()
    tokens = torch.randint(0, 500, (n_tok,), generator=g).cuda()
    scale = torch.tensor(h**0.5, dtype=torch.bfloat16)
    cam_flags = [torch.tensor([bool(i != 0)]).cuda() for i in range(cams)]
    tok_flags = (torch.rand(n_tok, generator=g) < 0.5).cuda()
    lang = torch.nn.functional.embedding(tokens[None], table) * scale.cuda()
    want = torch.cat([img.reshape(1, -1, h), lang], dim=1)
    assert want.dtype == torch.float32
    got, flags = tk.prefix_rows(img, 1.0, table, tokens, float(scale), None, cam_flags=cam_flags, tok_flags=tok_flags, out_dtype=torch.bfloat16)
    assert got.dtype == torch.bfloat16 and torch.equal(got, want.to(torch.bfloat16))
    assert torch.equal(flags, torch.cat([f[:, None].expand(1, per_cam) for f in cam_flags] + [tok_flags[None]], dim=1))
    got32, _ = tk.prefix_rows(img, 1.0, table, tokens, float(scale))
    assert torch.equal(got32, want)

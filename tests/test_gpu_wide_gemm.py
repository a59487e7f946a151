"""GPU parity of the many-row (M >= 256) fp8-weight GEMM / gated FFN: the VLM prefill shapes.

Reference path: the W8 prefill MLP of tybok/policies/pi05/models/triton_prefill_mlp.py:145-166 called
at M = prefix length; checked against the CPU oracle's weight-only composition at sizes it finishes
in seconds, and through size-independent properties at the full pi0.5 prefill size.
"""

import pytest
import torch

from oracle import ops as oops
from oracle.inputs import ffn_case, gemm_case

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _close(got, want, what):
    got = got.float().cpu()
    want = want.float().cpu()
    err = (got - want).abs()
    tol = 2e-2 + 2e-2 * want.abs()  # bf16 op outputs: rtol 2e-2 / atol 2e-2
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} / {bad.numel()} outside tolerance, max |err| {err.max():.4g}"


@pytest.fixture(scope="module")
def tk():
    from tybok_amd import ops

    return ops


@pytest.mark.parametrize("m,k,n", [(257, 64, 32), (256, 2048, 2048), (385, 96, 260), (300, 720, 2048), (300, 1024, 36), (712, 2048, 2048), (100, 64, 16384)])
def test_many_row_gemm(tk, m, k, n):
    x, w8, s = gemm_case(m, k, n)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    got = tk.fp8w_gemm(x.cuda(), pw)
    _close(got, oops.lin_fp8w(x, w8, s), f"gemm M={m} K={k} N={n}")


@pytest.mark.parametrize("resid_dtype", [None, torch.float32, BF16])
@pytest.mark.parametrize("m,k,n", [(385, 96, 260), (300, 256, 36), (257, 128, 1000)])
def test_many_row_gemm_row_segment_stores_respect_n_and_the_pitch(tk, m, k, n, resid_dtype):
    # output and residual are column slices of wider 16-byte aligned buffers (pitch % 8 == 0): the kernel stores
    # 16-byte row segments, the last one of a row cut to N; the columns past N must keep their sentinel
    x, w8, s = gemm_case(m, k, n)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    pitch = (n + 15) // 8 * 8
    buf = torch.full((m, pitch), 7.0, dtype=BF16, device="cuda")
    want = oops.lin_fp8w(x, w8, s)
    resid = None
    if resid_dtype is not None:
        r = torch.randn(m, pitch, generator=torch.Generator().manual_seed(3)).to(resid_dtype)
        want = (want.float() + r[:, :n].float()).to(BF16)
        resid = r.cuda()[:, :n]
    tk.fp8w_gemm(x.cuda(), pw, resid=resid, out=buf[:, :n])
    _close(buf[:, :n], want, f"gemm M={m} K={k} N={n} pitch={pitch}")
    assert bool((buf[:, n:] == 7.0).all()), "wrote past N"


def test_many_row_gemm_matches_skinny_kernel_rows(tk):
    # the same rows through the skinny kernel (M <= 64 per call) must give the same bits: both
    # kernels accumulate a row's k tiles in ascending order within a wave ... but split K over waves
    # differently, so compare within one bf16 ulp and require most outputs identical
    x, w8, s = gemm_case(320, 2048, 1024)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    xc = x.cuda()
    wide = tk.fp8w_gemm(xc, pw)
    skinny = torch.cat([tk.fp8w_gemm(xc[i : i + 64].contiguous(), pw) for i in range(0, 320, 64)])
    same = (wide == skinny).float().mean().item()
    assert same > 0.95, f"only {same:.1%} of the outputs agree bit for bit"
    _close(wide, skinny.cpu(), "wide vs skinny")


@pytest.mark.parametrize("m", [712, 1024])
def test_eight_wave_blocks_give_the_four_wave_kernels_bits(tk, m):
    # wide launches with enough column blocks run on eight-wave blocks of 192 (M=712) or 256 (M=1024) rows that stage
    # both operands through LDS; a 256-row slice of the same input stays on the four-wave kernel.  A row's k tiles are
    # accumulated in the same order in both, so the shared rows must agree bit for bit -- with and without a residual.
    k, n = 256, 32768
    x, w8, s = gemm_case(m, k, n)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    xc = x.cuda()
    r = torch.randn(m, n, generator=torch.Generator().manual_seed(5)).to(BF16).cuda()
    for resid in (None, r):
        full = tk.fp8w_gemm(xc, pw, resid=resid)
        for lo in (0, m - 256):
            part = tk.fp8w_gemm(xc[lo : lo + 256].contiguous(), pw, resid=None if resid is None else resid[lo : lo + 256].contiguous())
            assert torch.equal(full[lo : lo + 256], part), f"rows {lo}.. differ between the two kernels"
    _close(full[:64], (oops.lin_fp8w(x[:64], w8, s).float() + r[:64].float().cpu()).to(BF16), "eight-wave blocks vs oracle (first rows)")


@pytest.mark.parametrize("split", [1, 2, 5, 7])
def test_many_row_split_k_is_deterministic(tk, split):
    x, w8, s = gemm_case(300, 4096, 512)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    xc = x.cuda()
    a = tk.fp8w_gemm(xc, pw, split_k=split)
    b = tk.fp8w_gemm(xc, pw, split_k=split)
    assert torch.equal(a, b), "same launch twice must give the same bits (fixed-order reduction)"
    _close(a, oops.lin_fp8w(x, w8, s), f"many-row gemm split_k={split}")


@pytest.mark.parametrize("m,k,n", [(712, 4096, 2048), (300, 2048, 516), (257, 1024, 260)])
def test_many_row_split_k_reduction_launch_with_gate_and_residual(tk, m, k, n):
    # a K-split plain launch leaves fp32 partials and a second launch sums them in split order and runs the epilogue
    # (scale, per-column gate, bf16 / fp32 residual): ragged rows, N % 8 == 4, both residual types; the same
    # launch twice gives the same bits, and every split count agrees with the oracle
    x, w8, s = gemm_case(m, k, n)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    g = torch.Generator().manual_seed(7)
    gate = torch.randn(n, generator=g).to(BF16)
    base = oops.lin_fp8w(x, w8, s)
    for rdt in (BF16, torch.float32):
        resid = torch.randn(m, n, generator=g).to(rdt)
        want = ((base * gate).float() + resid.float()).to(BF16)
        for split in (2, 3, 4):
            a = tk.fp8w_gemm(x.cuda(), pw, resid=resid.cuda(), gate=gate.cuda(), split_k=split)
            b = tk.fp8w_gemm(x.cuda(), pw, resid=resid.cuda(), gate=gate.cuda(), split_k=split)
            assert torch.equal(a, b)
            _close(a, want, f"many-row split_k={split} + gate + resid {rdt} M={m} K={k} N={n}")


def test_many_row_gemm_residual_gate_and_strides(tk):
    m, k, n = 270, 720, 960
    x, w8, s = gemm_case(m, k, n)
    pw = tk.pack_fp8_weight(w8.cuda(), s.cuda())
    g = torch.Generator().manual_seed(3)
    padded = torch.zeros(m, 2 * k, dtype=BF16, device="cuda")
    padded[:, :k] = x.cuda()
    gate = torch.randn(n, generator=g).to(BF16)
    for rdt in (BF16, torch.float32):
        resid = torch.randn(m, n, generator=g).to(rdt)
        y = (oops.lin_fp8w(x, w8, s) * gate).float() + resid.float()
        got = tk.fp8w_gemm(padded[:, :k], pw, resid=resid.cuda(), gate=gate.cuda())
        _close(got, y.to(BF16), f"many-row gemm + gate + resid {rdt}")


@pytest.mark.parametrize("act,m,k,i", [("silu", 482, 960, 2560), ("gelu_tanh", 256, 1024, 4096), ("gelu_tanh", 712, 512, 1024)])
def test_many_row_gated_ffn(tk, act, m, k, i):
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(m, k, i, seed=4)
    resid = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).to(BF16)
    want = oops.gated_ffn(x, wg8, sg, wu8, su, wd8, sd, act)
    want += resid
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    got = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, act, resid=resid.cuda())
    again = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, act, resid=resid.cuda())
    assert torch.equal(got, again)
    _close(got, want, f"many-row ffn {act} M={m} K={k} I={i}")


@pytest.mark.parametrize("adaptive", [False, True])
def test_many_row_norm_gated_ffn(tk, adaptive):
    m, k, i = 300, 960, 2560
    eps = 1e-6 if adaptive else 1e-5
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(m, k, i, seed=6)
    g = torch.Generator().manual_seed(7)
    x = (x.float() * 2.5).to(BF16)
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    if adaptive:
        mod = 0.3 * torch.randn(1, 3 * k, generator=g)
        h, _ = oops.gemma_rms_norm(x[None], eps, modulation=mod)
        h = h[0]
        kw = dict(ada=(mod[0, :k].contiguous().cuda(), mod[0, k : 2 * k].contiguous().cuda()))
    else:
        norm_w = (1.0 + 0.2 * torch.randn(k, generator=g)).to(BF16)
        h = oops.rms_norm_llama(x, norm_w, eps)
        kw = dict(norm_w=norm_w.cuda())
    want = oops.gated_ffn(h, wg8, sg, wu8, su, wd8, sd, "gelu_tanh" if adaptive else "silu")
    want += x
    got = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, "gelu_tanh" if adaptive else "silu", resid=x.cuda(), eps=eps, **kw)
    _close(got, want, f"many-row norm + ffn adaptive={adaptive}")
    # normalising first and calling the plain entry point: same rounding points
    two_step = tk.fp8w_gated_ffn(h.cuda(), wgu, wd, "gelu_tanh" if adaptive else "silu", resid=x.cuda())
    mism = (got != two_step).float().mean().item()
    assert mism < 0.02, f"fused norm differs from norm-then-FFN on {mism:.1%} of the outputs"


def test_prefill_size_ffn_matches_oracle_and_rows_are_independent(tk):
    # pi0.5 prefill size (M=712, K=2048, I=16384; `make_fp8_mlp_forward`,
    # tybok/policies/pi05/models/triton_prefill_mlp.py:145-166) against the CPU oracle at full size, plus
    # what the mathematics fixes: an output row depends on its own input row only (shuffling the rows
    # shuffles the result bit-exactly, whatever block / wave / tile a row lands in).
    m, k, i = 712, 2048, 16384
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(m, k, i, seed=8)
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    xc = x.cuda()
    y = tk.fp8w_gated_ffn(xc, wgu, wd, "gelu_tanh")
    want = oops.gated_ffn(x, wg8, sg, wu8, su, wd8, sd, "gelu_tanh")
    _close(y, want, "prefill-size ffn (712, 2048, 16384) vs oracle")
    # the two linears on their own at this size (`w8a8_gemm` shapes, weight-only semantics)
    g = tk.fp8w_gemm(xc, tk.pack_fp8_weight(wg8.cuda(), sg))
    _close(g, oops.lin_fp8w(x, wg8, sg), "prefill-size gate projection (712, 2048 -> 16384) vs oracle")
    h = (oops.act_fn("gelu_tanh", oops.lin_fp8w(x, wg8, sg)) * oops.lin_fp8w(x, wu8, su)).to(BF16)
    d = tk.fp8w_gemm(h.cuda(), wd)
    _close(d, oops.lin_fp8w(h, wd8, sd), "prefill-size down projection (712, 16384 -> 2048) vs oracle")
    perm = torch.randperm(m, generator=torch.Generator().manual_seed(9)).cuda()
    yp = tk.fp8w_gated_ffn(xc[perm].contiguous(), wgu, wd, "gelu_tanh")
    assert torch.equal(yp, y[perm]), "rows must not depend on their position in the batch"
    skinny = tk.fp8w_gated_ffn(xc[:64].contiguous(), wgu, wd, "gelu_tanh")
    _close(y[:64], skinny.cpu(), "prefill-size ffn vs skinny kernel rows")

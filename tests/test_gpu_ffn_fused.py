"""The action chunk's gated FFN as ONE launch (down blocks wait for the gate/up blocks inside the kernel) against the
two-launch form, through the library's public entry points.

Reference seams: `triton_norm_gate_up` + down projection (tybok/policies/smolvla/models/triton_mlp.py:30-144) and
`triton_mlp_fp8_chain` (tybok/policies/pi05/models/triton_expert_mlp_fp8.py:438-469).  Same arithmetic and summation
order in both forms, so the outputs must agree to the last bit; parity against the oracle is covered by the FFN
cases of tests/test_gpu_ops.py and tests/test_gpu_fused_layer.py (two-launch form, the default: the single-launch
form measures slower on MI355X and is opt-in) and, for the two shapes the benchmark names, here.
"""

import pytest
import torch

from oracle import ops as oops
from oracle.inputs import ffn_case
from tybok_amd import ops as tk

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _case(m, k, i, seed, form):
    x, wg8, sg, wu8, su, wd8, sd = ffn_case(m, k, i, seed=seed)
    g = torch.Generator().manual_seed(seed + 77)
    kw = {}
    if form == "smolvla":  # RMSNorm prologue, bf16 residual
        kw = dict(norm_w=(1.0 + 0.1 * torch.randn(k, generator=g)).to(BF16).cuda(), eps=1e-5, resid=x.cuda())
    elif form == "pi05":  # per-column gate and residual on the down projection (the adaptive norm is a launch of its own)
        kw = dict(gate=torch.randn(k, generator=g).to(BF16).cuda(), resid=torch.randn(m, k, generator=g).to(BF16).cuda())
    wgu = tk.pack_fp8_gate_up(wg8.cuda(), sg, wu8.cuda(), su)
    wd = tk.pack_fp8_weight(wd8.cuda(), sd)
    return x, (wg8, sg, wu8, su, wd8, sd), wgu, wd, kw


@pytest.fixture(autouse=True)
def single_launch_form():
    """The single-launch form is opt-in: every test here runs with it on and restores the setting."""
    prev = tk.set_ffn_fusion(True)
    yield
    tk.set_ffn_fusion(prev)


CASES = [
    (50, 720, 2048, "silu", "plain"),
    (50, 720, 2048, "silu", "smolvla"),
    (50, 1024, 4096, "gelu_tanh", "plain"),
    (50, 1024, 4096, "gelu_tanh", "pi05"),
    (64, 720, 2048, "silu", "smolvla"),
    (33, 1024, 4096, "gelu_tanh", "pi05"),
    (17, 720, 2048, "silu", "smolvla"),
    (1, 1024, 4096, "gelu_tanh", "plain"),
]


@pytest.mark.parametrize("m,k,i,act,form", CASES)
def test_single_launch_ffn_gives_the_two_launch_bits(m, k, i, act, form):
    x, raw, wgu, wd, kw = _case(m, k, i, 3, form)
    ws = tk.Workspace("cuda")
    prev = tk.set_ffn_fusion(False)
    try:
        want = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, act, ws=ws, **kw)
    finally:
        tk.set_ffn_fusion(prev)
    tk.set_ffn_fusion(True)
    # several calls in a row on one workspace: the arrival counters must come back to zero every time
    for _ in range(4):
        got = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, act, ws=ws, **kw)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
    assert not ws.handoff_error()
    if form == "plain":  # and the oracle, at the two shapes the benchmark names
        _ = raw
        ref = oops.gated_ffn(x, *raw, act)
        err = (got.float().cpu() - ref.float()).abs()
        assert not (err > 2e-2 + 2e-2 * ref.float().abs()).any()


def test_single_launch_ffn_reads_this_launch_s_intermediate_not_an_older_one():
    # consecutive launches write DIFFERENT intermediates to the same workspace addresses (as consecutive layers do):
    # a down block that picked up a stale copy of a slice from its cache would show here
    m, k, i = 50, 720, 2048
    ws = tk.Workspace("cuda")
    cases = [_case(m, k, i, seed, "smolvla") for seed in (11, 12, 13)]
    prev = tk.set_ffn_fusion(False)
    try:
        wants = [tk.fp8w_gated_ffn(x.cuda(), wgu, wd, "silu", ws=ws, **kw) for x, _, wgu, wd, kw in cases]
    finally:
        tk.set_ffn_fusion(prev)
    tk.set_ffn_fusion(True)
    try:
        xs = [c[0].cuda() for c in cases]
        outs = [torch.empty_like(w) for w in wants]
        for _ in range(20):  # back to back, no synchronisation in between
            for j, (_, _, wgu, wd, kw) in enumerate(cases):
                tk.fp8w_gated_ffn(xs[j], wgu, wd, "silu", ws=ws, out=outs[j], **kw)
        torch.cuda.synchronize()
        for got, want in zip(outs, wants):
            assert torch.equal(got, want)
        # and under graph replay, where the launches follow each other most closely
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.inference_mode(), torch.cuda.graph(graph, stream=stream):
            for _ in range(4):
                for j, (_, _, wgu, wd, kw) in enumerate(cases):
                    tk.fp8w_gated_ffn(xs[j], wgu, wd, "silu", ws=ws, out=outs[j], **kw)
        for _ in range(5):
            for o in outs:
                o.zero_()
            graph.replay()
            torch.cuda.synchronize()
            for got, want in zip(outs, wants):
                assert torch.equal(got, want)
        assert not ws.handoff_error()
    finally:
        tk.set_ffn_fusion(prev)


def test_single_launch_ffn_replays_in_a_graph():
    x, _, wgu, wd, kw = _case(50, 720, 2048, 5, "smolvla")
    ws = tk.Workspace("cuda")
    xg = x.cuda()
    eager = tk.fp8w_gated_ffn(xg, wgu, wd, "silu", ws=ws, **kw)
    out = torch.zeros_like(eager)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.inference_mode(), torch.cuda.graph(graph, stream=stream):
        for _ in range(3):  # three dependent FFNs back to back, as consecutive layers launch them
            tk.fp8w_gated_ffn(xg, wgu, wd, "silu", ws=ws, out=out, **kw)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        assert torch.equal(tk.fp8w_gated_ffn(xg, wgu, wd, "silu", ws=ws, **kw), eager)  # eager work between the replays
    assert not ws.handoff_error()


def test_a_wait_that_gives_up_ends_the_launch_and_says_so():
    # Failure handling, forced from the host: with a bound of zero polls a down block does not wait at all.  Every
    # block still runs to its end (nothing here can hang); the launch's output is undefined, the workspace carries
    # the error word, and after a reset the next call is right again.
    x, _, wgu, wd, kw = _case(50, 1024, 4096, 7, "pi05")
    ws = tk.Workspace("cuda")
    want = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, "gelu_tanh", ws=ws, **kw)
    prev = tk.set_handoff_spin(0)
    try:
        tk.fp8w_gated_ffn(x.cuda(), wgu, wd, "gelu_tanh", ws=ws, **kw)
        torch.cuda.synchronize()
        assert ws.handoff_error()
    finally:
        tk.set_handoff_spin(prev)
    ws.reset()
    assert not ws.handoff_error()
    got = tk.fp8w_gated_ffn(x.cuda(), wgu, wd, "gelu_tanh", ws=ws, **kw)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and not ws.handoff_error()

"""tk_fp8w_gemm_static -- the entry point that allocates nothing -- against tk_fp8w_gemm, through the C ABI.

Same kernels, same split rule, so the outputs must agree to the last bit.  Two calls in a row share the
library's static scratch; the second uses a smaller input and must not see what the first left there.
"""

import pytest
import torch

from oracle.inputs import gemm_case
from tybok_amd import native
from tybok_amd import ops as tk

pytestmark = pytest.mark.gpu


def _both(x, w, split_k, resid=None):
    lib = native.lib()
    m, k = x.shape
    ws = tk.default_workspace(x.device)
    st = torch.cuda.current_stream().cuda_stream
    want = torch.empty(m, w.n, dtype=torch.bfloat16, device=x.device)
    got = torch.full_like(want, float("nan"))
    rp = resid.data_ptr() if resid is not None else None
    ldr = resid.stride(0) if resid is not None else 0
    args = (x.data_ptr(), x.stride(0), w.data.data_ptr(), w.scale.data_ptr())
    native.check(lib.tk_fp8w_gemm(*args, want.data_ptr(), w.n, rp, ldr, 0, None, m, w.n, k, split_k, ws.ptr, ws.nbytes, st), "tk_fp8w_gemm")
    # torch's allocator makes no allocation during the call (the cumulative count: a collection of earlier tests'
    # garbage between the two reads may free memory, it cannot allocate)
    before = torch.cuda.memory_stats().get("allocation.all.allocated", 0)
    native.check(lib.tk_fp8w_gemm_static(*args, got.data_ptr(), w.n, rp, ldr, 0, None, m, w.n, k, split_k, st), "tk_fp8w_gemm_static")
    assert torch.cuda.memory_stats().get("allocation.all.allocated", 0) == before
    torch.cuda.synchronize()
    return got, want


def test_static_scratch_matches_workspace_entry_point_on_two_calls_in_a_row():
    lib = native.lib()
    assert lib.tk_static_scratch_bytes() == (64 << 10) + (8 << 20)
    # first call: the pi0.5 expert's down projection (M=50, 4096 -> 1024), K split chosen by the library
    x, w8, s = gemm_case(50, 4096, 1024)
    w = tk.pack_fp8_weight(w8.cuda(), s)
    resid = torch.randn(50, 1024, generator=torch.Generator().manual_seed(5)).bfloat16().cuda()
    got, want = _both(x.cuda(), w, 0, resid)
    assert torch.equal(got, want)
    # second call, smaller input, explicit split: reuses the scratch the first call wrote
    x2, w82, s2 = gemm_case(16, 2048, 2048)
    w2 = tk.pack_fp8_weight(w82.cuda(), s2)
    got2, want2 = _both(x2.cuda(), w2, 4)
    assert torch.equal(got2, want2)
    # and the first shape again after the smaller one: with the split forced, then as in the first call
    got3, want3 = _both(x.cuda(), w, 8, resid)
    assert torch.equal(got3, want3)
    got4, _ = _both(x.cuda(), w, 0, resid)
    assert torch.equal(got4, got)


def test_static_scratch_rejects_what_it_cannot_hold():
    lib = native.lib()
    x, w8, s = gemm_case(16, 2048, 16384)
    w = tk.pack_fp8_weight(w8.cuda(), s)
    xg = x.cuda()
    y = torch.empty(16, 16384, dtype=torch.bfloat16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    # 256 two-tile strips x 16 splits x 8 KiB of partials = 32 MiB: more than the 8 MiB of partial space
    rc = lib.tk_fp8w_gemm_static(xg.data_ptr(), 2048, w.data.data_ptr(), w.scale.data_ptr(), y.data_ptr(), 16384, None, 0, 0, None, 16, 16384, 2048, 16, st)
    assert rc == -2 and b"workspace too small" in lib.tk_last_error()
    # more rows than the entry point is built for
    rc = lib.tk_fp8w_gemm_static(xg.data_ptr(), 2048, w.data.data_ptr(), w.scale.data_ptr(), y.data_ptr(), 16384, None, 0, 0, None, 65, 16384, 2048, 0, st)
    assert rc == -1 and b"exceeds the 64 rows" in lib.tk_last_error()
    # the automatic choice stays inside the scratch and matches the workspace entry point
    got, want = _both(xg, w, 0)
    assert torch.equal(got, want)


def test_static_scratch_split_launch_replays_in_a_graph():
    # a K-split launch of the static entry point captured into a graph (the address lookup happened in the calls
    # above or in tk_static_scratch_bytes(); the counters are cleared by a fill kernel, which a graph may hold):
    # every replay gives the eager bits, with eager launches that reuse the scratch between the replays
    lib = native.lib()
    lib.tk_static_scratch_bytes()
    x, w8, s = gemm_case(50, 4096, 1024)
    w = tk.pack_fp8_weight(w8.cuda(), s)
    xg = x.cuda()
    eager, _ = _both(xg, w, 8)
    out = torch.zeros(50, 1024, dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.inference_mode(), torch.cuda.graph(graph, stream=stream):
        st = torch.cuda.current_stream().cuda_stream
        native.check(lib.tk_fp8w_gemm_static(xg.data_ptr(), 4096, w.data.data_ptr(), w.scale.data_ptr(), out.data_ptr(), 1024, None, 0, 0, None, 50, 1024, 4096, 8, st), "tk_fp8w_gemm_static")
    x2, w82, s2 = gemm_case(16, 2048, 2048)
    w2 = tk.pack_fp8_weight(w82.cuda(), s2)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        got2, want2 = _both(x2.cuda(), w2, 4)  # eager work on the same scratch between the replays
        assert torch.equal(got2, want2)

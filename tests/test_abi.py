"""The C-ABI library loads and exports exactly what include/tybok_hip.h declares (no GPU needed)."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tybok_hip.h")


def _declared():
    text = open(HEADER, encoding="utf-8").read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tk_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    names = _declared()
    for required in ("tk_fp8w_gemm", "tk_fp8w_gated_ffn", "tk_expert_attn", "tk_pack_fp8_weight", "tk_last_error"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from tybok_amd import native

    if not os.path.exists(native.library_path()):
        pytest.skip("libtybok_hip.so not built (run python -m tybok_amd.csrc.build)")
    handle = ctypes.CDLL(native.library_path())
    for name in _declared():
        assert hasattr(handle, name), f"{name} declared in tybok_hip.h but not exported"
    # the ctypes table covers the header one to one
    assert sorted(native.SIGNATURES) == _declared()


def test_host_only_entry_points():
    from tybok_amd import native

    if not os.path.exists(native.library_path()):
        pytest.skip("libtybok_hip.so not built")
    lib = native.lib()
    assert lib.tk_version() >= 1
    assert lib.tk_fp8w_packed_bytes(2048, 720) == 64 * 23 * 1024  # K padded to 23 tiles of 32
    assert lib.tk_fp8w_packed_bytes(720, 2048) == 23 * 64 * 1024
    assert lib.tk_workspace_bytes() >= 32 << 20
    # argument validation happens on the host before any launch
    assert lib.tk_pack_fp8_weight(None, None, 32, 32, None) < 0
    assert b"bad argument" in lib.tk_last_error()


def test_missing_library_fails_loudly(monkeypatch):
    from tybok_amd import native

    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "_LIB_PATH", "/nonexistent/libtybok_hip.so")
    with pytest.raises(RuntimeError, match="no CPU or torch fallback"):
        native.lib()


P = 0x10000  # a 16-byte aligned stand-in for device pointers: every call below is rejected before any launch


def _cases():
    """(entry point, arguments, error code, fragment of tk_last_error()) -- one row per validation rule."""
    gemm = lambda **kw: _args(  # noqa: E731
        dict(x=P, ldx=2048, w=P, scale=P, y=P, ldy=16384, resid=None, ldr=0, rdt=0, gate=None, M=50, N=16384, K=2048, split=0, ws=None, wsb=0, st=None), kw
    )
    ffn = lambda **kw: _args(  # noqa: E731
        dict(x=P, ldx=720, wgu=P, sg=P, su=P, wd=P, sd=P, y=P, ldy=720, resid=None, ldr=0, rdt=0, gate=None, M=50, K=720, I=2048, act=0, ws=P, wsb=1 << 27, st=None), kw
    )
    attn = lambda **kw: _args(  # noqa: E731
        dict(q=P, q_sm=960, q_sh=64, k=P, k_lo=None, sl=320, sh=64, vt=P, vt_lo=None, vsd=256, vsh=64 * 256, ks=None, ssl=0, ssh=0, vts=None, svsd=0, svsh=0,
             pad=None, m2=None, mld=0, out=P, osm=960, M=50, Pk=241, S=0, H=15, G=5, D=64, mode=0, lb=0, ws=None, wsb=0, st=None), kw
    )  # fmt: skip
    tail = lambda **kw: _args(  # noqa: E731
        dict(x=P, ldx=720, nw=P, asc=None, ash=None, eps=1e-6, w=P, b=None, v=P, xt=None, xo=None, dt=0.0, M=50, N=32, K=720, st=None), kw
    )
    tail_e = lambda **kw: _args(  # noqa: E731
        dict(x=P, ldx=720, nw=P, asc=None, ash=None, eps=1e-6, w=P, b=None, v=None, xt=P, xo=P, dt=-0.1, M=50, N=32, K=720,
             ew=P, eb=None, en=720, eact=1, eo=P, eld=720, edt=1, st=None), kw
    )  # fmt: skip
    ln = lambda **kw: _args(dict(x=P, ldx=768, xdt=0, w=P, b=P, wdt=0, eps=1e-6, y=P, ldy=768, M=64, K=768, st=None), kw)  # noqa: E731
    tv = lambda **kw: _args(dict(v=P, sb=1 << 20, sl=2304, sh=64, vt=P, tsb=1 << 20, tsh=65536, tsd=1024, keys=1024, B=3, Pk=1024, G=12, D=64, st=None), kw)  # noqa: E731
    qa = lambda **kw: _args(dict(x=P, ldx=2048, a8=P, lda=2048, sa=P, M=712, K=2048, mode=0, st=None), kw)  # noqa: E731
    w8 = lambda **kw: _args(  # noqa: E731
        dict(a8=P, lda=2048, sa=P, w=P, sw=P, y=P, ldy=16384, resid=None, ldr=0, rdt=0, M=712, N=16384, K=2048, split=0, ws=None, wsb=0, st=None), kw
    )
    w8ffn = lambda **kw: _args(  # noqa: E731
        dict(x=P, ldx=2048, wgu=P, sg=P, su=P, wd=P, sd=P, y=P, ldy=2048, resid=None, ldr=0, rdt=0, M=712, K=2048, I=16384, act=1, qm=1, ws=P, wsb=1 << 27, st=None), kw
    )
    dense = lambda **kw: _args(  # noqa: E731
        dict(x=P, ldx=768, w=P, bias=P, act=0, y=P, ldy=3072, resid=None, ldr=0, rdt=0, M=3072, N=3072, K=768, tile=0, split=0, ws=None, wsb=0, st=None), kw
    )
    static = lambda **kw: _args(  # noqa: E731
        dict(x=P, ldx=2048, w=P, scale=P, y=P, ldy=16384, resid=None, ldr=0, rdt=0, gate=None, M=50, N=16384, K=2048, split=0, st=None), kw
    )
    sread = lambda **kw: _args(dict(src=P, bytes=1 << 25, blocks=256, sink=P, st=None), kw)  # noqa: E731
    meta = lambda **kw: _args(dict(pad=P, att=None, P=241, pp=256, pos=16384, S=50, mask=P, p32=P, suf=P, st=None), kw)  # noqa: E731
    patch = lambda **kw: _args(dict(i0=P, i1=P, i2=P, i3=None, n=3, H=512, W=512, ps=16, scale=2.0, shift=-1.0, out=P, st=None), kw)  # noqa: E731
    return [
        ("tk_quant_act_rows", qa(K=2044), -1, "multiple of 8"),
        ("tk_quant_act_rows", qa(K=32768, ldx=32768, lda=32768), -1, "at most"),
        ("tk_quant_act_rows", qa(mode=2), -1, "mode 2"),
        ("tk_quant_act_rows", qa(x=P + 8), -1, "16-byte"),
        ("tk_w8a8_gemm", w8(K=2040), -1, "multiple of 16"),
        ("tk_w8a8_gemm", w8(lda=2000), -1, "lda"),
        ("tk_w8a8_gemm", w8(sa=None), -1, "null pointer"),
        ("tk_w8a8_gemm", w8(N=16382), -1, "multiples of 4"),
        ("tk_w8a8_gemm", w8(split=4), -2, "partial space"),
        ("tk_w8a8_gated_ffn", w8ffn(act=9), -1, "unknown activation"),
        ("tk_w8a8_gated_ffn", w8ffn(qm=2), -1, "unknown quantisation mode"),
        ("tk_bf16w_dense", dense(K=776, ldx=776), -1, "multiple of 16"),
        ("tk_bf16w_dense", dense(ldy=3076), -1, "multiple of 8"),
        ("tk_bf16w_dense", dense(act=3), -1, "act=3"),
        ("tk_bf16w_dense", dense(tile=33), -1, "tile=33"),
        ("tk_bf16w_dense", dense(resid=P, ldr=3070, rdt=0), -1, "residual"),
        ("tk_bf16w_dense", dense(y=P + 8), -1, "16-byte aligned"),
        ("tk_fp8w_gemm_static", static(M=65), -1, "exceeds the 64 rows"),
        ("tk_debug_stream_read", sread(bytes=1000), -1, "multiple"),
        ("tk_bf16w_dense_rope", (P, 2048, P, P, 2560, P, P, P, 300, 2304, 128, 1, None, 0, 0, 712, 2560, 2048, 31, 0, None, 0, None), -1, "tile=31"),
        ("tk_bf16w_dense_rope", (P, 2048, P, P, 2560, P, P, P, 300, 2300, 128, 1, None, 0, 0, 712, 2560, 2048, 0, 0, None, 0, None), -1, "whole heads"),
        ("tk_bf16w_dense_rope", (P, 2048, P, P, 2560, None, P, P, 300, 2304, 128, 1, None, 0, 0, 712, 2560, 2048, 0, 0, None, 0, None), -1, "null table"),
        ("tk_bf16w_dense_rope", (P, 2048, P, P, 2560, P, P, P, 300, 2304, 128, 1, P, 2304, 712, 712, 2560, 2048, 0, 0, None, 0, None), -1, "vt_ld"),
        ("tk_bf16w_dense_vt", (P, 768, P, P, P, 2304, P, 1500, 1024, 1024, 786432, 0, 3072, 2304, 768, 0, 0, None, 0, None), -1, "multiple of 64"),
        ("tk_bf16w_dense_vt", (P, 768, P, P, P, 2304, P, 1536, 1024, 1000, 786432, 0, 3072, 2304, 768, 0, 0, None, 0, None), -1, "multiple of 32"),
        ("tk_bf16w_dense_vt", (P, 768, P, P, P, 2304, None, 1536, 1024, 1024, 786432, 0, 3072, 2304, 768, 0, 0, None, 0, None), -1, "16-byte aligned"),
        ("tk_debug_fp8w_gemm_cut", (P, 2040, P, P, P, 16384, 50, 16384, 2040, 1, None), -1, "multiple of 16"),
        ("tk_fp8w_gemm", gemm(K=2040), -1, "multiple of 16"),
        ("tk_fp8w_gemm", gemm(ldx=1024), -1, "ldx"),
        ("tk_fp8w_gemm", gemm(x=P + 2), -1, "16-byte aligned"),
        ("tk_fp8w_gemm", gemm(y=None), -1, "null pointer"),
        ("tk_fp8w_gemm", gemm(M=0), -1, "non-positive"),
        ("tk_fp8w_gemm", gemm(resid=P, ldr=8), -1, "ldr"),
        ("tk_fp8w_gemm", gemm(resid=P, ldr=16384, rdt=5), -1, "resid_dtype"),
        ("tk_fp8w_gemm", gemm(N=720, K=16384, ldx=16384, ldy=720, split=8), -2, "needs a workspace"),
        ("tk_fp8w_gated_ffn", ffn(act=7), -1, "unknown activation"),
        ("tk_fp8w_gated_ffn", ffn(I=2000), -1, "multiple of 32"),
        ("tk_fp8w_gated_ffn", ffn(ws=None), -2, "needs a workspace"),
        ("tk_fp8w_gated_ffn", ffn(M=100000, I=16384), -2, "intermediate"),
        ("tk_fp8w_gated_ffn", ffn(M=-3), -1, "non-positive"),
        ("tk_expert_attn", attn(D=80), -1, "head_dim"),
        ("tk_expert_attn", attn(G=4), -1, "bad shape"),
        ("tk_expert_attn", attn(sl=324), -1, "multiples of 8"),
        ("tk_expert_attn", attn(S=50, ks=P, vts=P, ssl=320, ssh=64, svsd=64, svsh=4096), -1, "suffix mask mode"),
        ("tk_expert_attn", attn(vsd=224), -1, "rounded up to 32"),
        ("tk_expert_attn", attn(k_lo=P), -1, "both K and V^T low planes"),
        ("tk_expert_attn", attn(osm=900), -1, "out_sm"),
        ("tk_expert_attn", attn(mode=3), -1, "mask_mode"),
        ("tk_expert_tail", tail(N=48), -1, "divide 256"),
        ("tk_expert_tail", tail(K=8200, ldx=8200), -1, "at most 8192"),
        ("tk_expert_tail", tail(asc=P, ash=P), -1, "exactly one"),
        ("tk_expert_tail", tail(v=None), -1, "no output"),
        ("tk_expert_tail_embed", tail_e(eo=None), -1, "emb_out is null"),
        ("tk_expert_tail_embed", tail_e(xo=None, v=P), -1, "computed from x_out"),
        ("tk_expert_tail_embed", tail_e(N=16), -1, "takes N=32 inputs"),
        ("tk_expert_tail_embed", tail_e(ew=P + 4), -1, "16-byte aligned"),
        ("tk_expert_tail_embed", tail_e(eld=700), -1, "bad embedding shape"),
        ("tk_expert_tail_embed", tail_e(eact=2), -1, "emb_act=2"),
        ("tk_expert_tail_embed", tail_e(edt=3), -1, "emb_dtype=3"),
        ("tk_layer_norm", ln(K=4096, ldx=4096, ldy=4096), -1, "at most"),
        ("tk_layer_norm", ln(wdt=1), -1, "both"),
        ("tk_layer_norm", ln(ldy=760), -1, "row pitch"),
        ("tk_add_layer_norm_rows", (P, 768, 0, P, 768, P, 768, P, P, 0, 1e-6, P + 65536, 768, None, 3072, 768, None), -1, "row map is null"),
        ("tk_add_layer_norm_rows", (P, 768, 0, P, 768, P, 768, P, P, 0, 1e-6, P, 768, P, 3072, 768, None), -1, "must not be x or xsum"),
        ("tk_add_layer_norm_rows", (P, 768, 0, None, 768, P, 768, P, P, 0, 1e-6, P + 65536, 768, P, 3072, 768, None), -1, "null residual"),
        ("tk_batched_transpose_v", tv(D=128), -1, "head_dim"),
        ("tk_batched_transpose_v", tv(keys=1000), -1, "rounded up to 32"),
        ("tk_batched_transpose_v", tv(sl=2300), -1, "multiples of 8"),
        ("tk_prefix_meta", meta(P=0), -1, "P=0"),
        ("tk_prefix_meta", meta(P=4096, pp=4096), -1, "P=4096"),
        ("tk_prefix_meta", meta(pad=None), -1, "null pad flags"),
        ("tk_prefix_meta", meta(S=50, suf=None), -1, "S without an output"),
        ("tk_prefix_meta", meta(pp=240), -1, "p_pad=240"),
        ("tk_prefix_meta", meta(pp=250), -1, "multiple of 16"),
        ("tk_prefix_meta", meta(mask=P + 4), -1, "16-byte aligned"),
        ("tk_expert_kv_project_layers", (17, P, P, 960, 241, 320, P, P, 320, P, P, P, P, 256, None), -1, "17 layers"),
        ("tk_expert_kv_project_layers", (8, P, P, 960, 241, 320, P, P, 300, P, P, P, P, 256, None), -1, "bad shape"),
        ("tk_expert_kv_project_layers", (8, P, P, 960, 241, 320, P, P, 320, P, P, P, P, 224, None), -1, "rounded up to 32"),
        ("tk_prefix_rows", (P, 0, 192, 30.0, P, P, 48, 49280, 30.9, P, 1, P, 1, 964, P, P, P, None, 3, P, P, None), -1, "H=964"),
        ("tk_prefix_rows", (P, 0, 192, 30.0, P, P + 4, 48, 49280, 30.9, P, 1, P, 1, 960, P, P, P, None, 3, P, P, None), -1, "8-byte aligned ids"),
        ("tk_prefix_rows", (P, 0, 192, 30.0, P, P, 48, 49280, 30.9, P, 1, P, 1, 960, P, P, None, None, 3, P, P, None), -1, "camera 2 is null"),
        ("tk_prefix_rows", (P, 0, 190, 30.0, P, P, 48, 49280, 30.9, P, 1, P, 1, 960, P, P, P, None, 3, P, P, None), -1, "do not split"),
        ("tk_prefix_rows", (P, 0, 192, 30.0, P, P, 48, 49280, 30.9, P, 1, None, 1, 960, P, P, P, None, 3, P, P, None), -1, "output is null"),
        ("tk_prefix_rows", (P, 2, 192, 30.0, P, P, 48, 49280, 30.9, P, 1, P, 1, 960, P, P, P, None, 3, P, P, None), -1, "img_dtype=2"),
        ("tk_patchify_images_f32", patch(H=224, W=224, ps=7), -1, "multiple of 2"),
        ("tk_patchify_images_f32", patch(H=224, W=224, ps=14, i2=None), -1, "image 2 is null"),
        ("tk_patchify_images", patch(n=5), -1, "n=5"),
        ("tk_patchify_images", patch(ps=12), -1, "patch=12"),
        ("tk_patchify_images", patch(H=500), -1, "divides"),
        ("tk_patchify_images", patch(i1=None), -1, "image 1 is null"),
        ("tk_patchify_images", patch(out=P + 8), -1, "output must be 16-byte aligned"),
    ]


def _args(defaults, overrides):
    unknown = set(overrides) - set(defaults)
    assert not unknown, unknown
    return list({**defaults, **overrides}.values())


@pytest.mark.parametrize("name,args,code,fragment", _cases(), ids=lambda v: v if isinstance(v, str) and v.startswith("tk_") else None)
def test_arguments_are_checked_on_the_host(name, args, code, fragment):
    # every entry point validates shapes, strides, alignment and workspace before it launches anything: a bad
    # call returns the documented error code and says why, with or without a GPU in the machine
    from tybok_amd import native

    if not os.path.exists(native.library_path()):
        pytest.skip("libtybok_hip.so not built")
    lib = native.lib()
    assert len(args) == len(native.SIGNATURES[name][1])
    rc = getattr(lib, name)(*args)
    message = lib.tk_last_error().decode()
    assert rc == code, f"{name}: rc {rc}, message {message!r}"
    assert fragment in message, message


@pytest.mark.parametrize("compiler,flags", [("gcc", ["-std=c99", "-x", "c"]), ("g++", ["-std=c++17", "-x", "c++"])])
def test_header_is_plain_c_and_cxx(tmp_path, compiler, flags):
    # the boundary is a C ABI: the header must be usable from C (cgo, ctypes generators, C hosts) and from C++
    import shutil
    import subprocess

    if shutil.which(compiler) is None:
        pytest.skip(f"{compiler} not installed")
    src = tmp_path / "use_header.c"
    src.write_text(f'#include "{HEADER}"\nint main(void) {{ return tk_version() > 0 && TK_OK == 0 ? 0 : 1; }}\n')
    done = subprocess.run([compiler, *flags, "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", str(src)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr

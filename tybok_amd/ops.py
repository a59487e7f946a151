"""Tensor-level wrappers over the C ABI: torch supplies device memory and the stream, nothing else.

Every function enqueues on ``torch.cuda.current_stream()`` and is legal under graph capture as
long as the output / workspace tensors were allocated before the capture (or come from the
capture's private pool).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import native

ACT = {"silu": 0, "gelu_tanh": 1}
MASK_NONE, MASK_BIDIR, MASK_CAUSAL = 0, 1, 2
_BF16, _F32 = 0, 1


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


class Workspace:
    """Caller-owned scratch of the library (split-K partials, FFN intermediate, counters).

    One per stream that may run kernels concurrently.  Created before graph capture.
    """

    def __init__(self, device: torch.device | str = "cuda"):
        lib = native.lib()
        self.nbytes = int(lib.tk_workspace_bytes())
        self.buf = torch.empty(self.nbytes, dtype=torch.uint8, device=device)
        native.check(lib.tk_workspace_init(self.buf.data_ptr(), self.nbytes, _stream()), "tk_workspace_init")

    @property
    def ptr(self) -> int:
        return self.buf.data_ptr()

    def reset(self) -> None:
        """Zero every arrival counter and the hand-off error word (after a launch that gave up waiting)."""
        native.check(native.lib().tk_workspace_init(self.buf.data_ptr(), self.nbytes, _stream()), "tk_workspace_init")

    def handoff_error(self) -> bool:
        """Whether a block of the single-launch FFN has given up its bounded wait since the last reset (synchronises)."""
        off = int(native.lib().tk_workspace_handoff_error_offset())
        return bool(self.buf[off : off + 4].view(torch.int32).item())


_default_ws: dict[int, Workspace] = {}


def default_workspace(device: torch.device | str | None = None) -> Workspace:
    """The per-device workspace used when a call passes none.  It serves launches that are ordered one
    after the other (one stream, or streams joined by events / graph capture of a single stream): the
    split hand-offs keep counters and partials in it, so code that runs kernels on two streams AT THE
    SAME TIME must give the second stream a :class:`Workspace` of its own (the SmolVLA overlap path does)."""
    dev = torch.device(device if device is not None else "cuda")
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    ws = _default_ws.get(idx)
    if ws is None:
        ws = Workspace(torch.device("cuda", idx))
        _default_ws[idx] = ws
    return ws


@dataclass
class PackedWeight:
    """An fp8 e4m3fn ``[N, K]`` weight in the library's tile order plus its fp32 row scales."""

    data: torch.Tensor  # uint8, packed tiles
    scale: torch.Tensor  # fp32 [N]
    n: int
    k: int


@dataclass
class PackedGateUp:
    """Gate and up weights (``[I, K]`` each) with interleaved 32-row tiles."""

    data: torch.Tensor
    scale_gate: torch.Tensor
    scale_up: torch.Tensor
    i: int
    k: int


@dataclass
class PackedBf16Weight:
    """A bf16 ``[N, K]`` weight in tile order; ``rope_half`` > 0 means rotary pair order."""

    data: torch.Tensor
    n: int
    k: int
    rope_half: int = 0
    dtype: torch.dtype = torch.bfloat16  # the 16-bit type of the packed words (fp16: the many-row kernel only)


@dataclass
class RopeTables:
    """fp32 ``[positions, rope_half]`` cos / sin tables of a half-split rotary embedding."""

    cos: torch.Tensor
    sin: torch.Tensor

    @property
    def positions(self) -> int:
        return self.cos.shape[0]

    @property
    def half(self) -> int:
        return self.cos.shape[1]


def _as_fp8_bytes(w8: torch.Tensor) -> torch.Tensor:
    if w8.dtype == torch.float8_e4m3fn:
        w8 = w8.view(torch.uint8)
    if w8.dtype != torch.uint8:
        raise TypeError(f"expected float8_e4m3fn or uint8 codes, got {w8.dtype}")
    if not w8.is_cuda:
        raise ValueError("weight must be on the GPU")
    return w8.contiguous()


def pack_fp8_weight(w8: torch.Tensor, scale: torch.Tensor) -> PackedWeight:
    """Row-major e4m3fn ``[N, K]`` (+ fp32 ``[N]`` scale) -> :class:`PackedWeight` (once per model)."""
    lib = native.lib()
    codes = _as_fp8_bytes(w8)
    n, k = codes.shape
    out = torch.empty(int(lib.tk_fp8w_packed_bytes(n, k)), dtype=torch.uint8, device=codes.device)
    native.check(lib.tk_pack_fp8_weight(codes.data_ptr(), out.data_ptr(), n, k, _stream()), "tk_pack_fp8_weight")
    return PackedWeight(out, scale.to(device=codes.device, dtype=torch.float32).contiguous(), n, k)


def pack_fp8_gate_up(wg8: torch.Tensor, sg: torch.Tensor, wu8: torch.Tensor, su: torch.Tensor) -> PackedGateUp:
    lib = native.lib()
    cg, cu = _as_fp8_bytes(wg8), _as_fp8_bytes(wu8)
    if cg.shape != cu.shape:
        raise ValueError("gate and up weights must have the same shape")
    i, k = cg.shape
    out = torch.empty(int(lib.tk_fp8w_packed_bytes(2 * i, k)), dtype=torch.uint8, device=cg.device)
    native.check(
        lib.tk_pack_fp8_gate_up(cg.data_ptr(), cu.data_ptr(), out.data_ptr(), i, k, _stream()), "tk_pack_fp8_gate_up"
    )
    f32 = dict(device=cg.device, dtype=torch.float32)
    return PackedGateUp(out, sg.to(**f32).contiguous(), su.to(**f32).contiguous(), i, k)


def _check_act(x: torch.Tensor, k: int) -> tuple[int, int]:
    if x.dtype != torch.bfloat16 or not x.is_cuda:
        raise TypeError("activations must be bf16 CUDA tensors")
    if x.dim() != 2 or x.shape[1] != k or x.stride(1) != 1:
        raise ValueError(f"activations must be [M, {k}] with unit inner stride, got {tuple(x.shape)}")
    return x.shape[0], x.stride(0)


def _resid_args(resid: torch.Tensor | None, m: int, n: int) -> tuple[int | None, int, int]:
    if resid is None:
        return None, 0, 0
    if resid.shape != (m, n) or resid.stride(1) != 1:
        raise ValueError("residual must be [M, N] with unit inner stride")
    if resid.dtype == torch.bfloat16:
        return resid.data_ptr(), resid.stride(0), _BF16
    if resid.dtype == torch.float32:
        return resid.data_ptr(), resid.stride(0), _F32
    raise TypeError("residual must be bf16 or fp32")


def _gate_ptr(gate: torch.Tensor | None, n: int) -> int | None:
    if gate is None:
        return None
    if gate.dtype != torch.bfloat16 or gate.numel() != n or not gate.is_contiguous():
        raise ValueError(f"gate must be a contiguous bf16 tensor of {n} elements")
    return gate.data_ptr()


def fp8w_gemm(
    x: torch.Tensor,
    w: PackedWeight,
    *,
    resid: torch.Tensor | None = None,
    gate: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    split_k: int = 0,
    ws: Workspace | None = None,
) -> torch.Tensor:
    """``bf16((x @ W8^T) * scale)`` (``* gate[n]``, ``+ residual``) for ``x [M, K]`` bf16."""
    lib = native.lib()
    m, ldx = _check_act(x, w.k)
    if out is None:
        out = torch.empty(m, w.n, dtype=torch.bfloat16, device=x.device)
    rp, ldr, rdt = _resid_args(resid, m, w.n)
    ws = ws or default_workspace(x.device)
    rc = lib.tk_fp8w_gemm(
        x.data_ptr(), ldx, w.data.data_ptr(), w.scale.data_ptr(), out.data_ptr(), out.stride(0), rp, ldr, rdt,
        _gate_ptr(gate, w.n), m, w.n, w.k, split_k, ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_fp8w_gemm")
    return out


def fp8w_gated_ffn(
    x: torch.Tensor,
    wgu: PackedGateUp,
    wd: PackedWeight,
    act: str = "silu",
    *,
    resid: torch.Tensor | None = None,
    gate: torch.Tensor | None = None,
    norm_w: torch.Tensor | None = None,
    eps: float = 0.0,
    ada: tuple[torch.Tensor, torch.Tensor] | None = None,
    out: torch.Tensor | None = None,
    ws: Workspace | None = None,
) -> torch.Tensor:
    """``down(act(gate(x)) * up(x))`` (``* gate[n]``, ``+ residual``) for ``x [M, K]`` bf16;
    with ``norm_w`` (RMSNorm) or ``ada = (scale, shift)`` (adaptive RMSNorm) the input is first
    normalised inside the gate/up launch."""
    lib = native.lib()
    m, ldx = _check_act(x, wgu.k)
    if wd.k != wgu.i or wd.n != wgu.k:
        raise ValueError("down weight must be [K, I]")
    if out is None:
        out = torch.empty(m, wd.n, dtype=torch.bfloat16, device=x.device)
    rp, ldr, rdt = _resid_args(resid, m, wd.n)
    ws = ws or default_workspace(x.device)
    if norm_w is not None or ada is not None:
        rc = lib.tk_fp8w_norm_gated_ffn(
            x.data_ptr(), ldx, _norm_ptr(norm_w, wgu.k), float(eps), *_ada_ptrs(ada, wgu.k), wgu.data.data_ptr(), wgu.scale_gate.data_ptr(),
            wgu.scale_up.data_ptr(), wd.data.data_ptr(), wd.scale.data_ptr(), out.data_ptr(), out.stride(0), rp, ldr, rdt,
            _gate_ptr(gate, wd.n), m, wgu.k, wgu.i, ACT[act], ws.ptr, ws.nbytes, _stream(),
        )  # fmt: skip
        native.check(rc, "tk_fp8w_norm_gated_ffn")
        return out
    rc = lib.tk_fp8w_gated_ffn(
        x.data_ptr(), ldx, wgu.data.data_ptr(), wgu.scale_gate.data_ptr(), wgu.scale_up.data_ptr(),
        wd.data.data_ptr(), wd.scale.data_ptr(), out.data_ptr(), out.stride(0), rp, ldr, rdt,
        _gate_ptr(gate, wd.n), m, wgu.k, wgu.i, ACT[act], ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_fp8w_gated_ffn")
    return out


def set_ffn_fusion(on: bool) -> bool:
    """Single-launch FFN for the action chunk on / off (the default: two launches everywhere); returns the previous setting."""
    return bool(native.lib().tk_set_ffn_fusion(1 if on else 0))


def set_handoff_spin(polls: int) -> int:
    """Bound (polls) of the wait inside the single-launch FFN; returns the previous value."""
    return int(native.lib().tk_set_handoff_spin(int(polls)))


def quant_act_rows(x: torch.Tensor, mode: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-token e4m3fn quantisation of ``x [M, K]`` bf16 -> ``(a8 [M, K] float8_e4m3fn, sa [M] fp32)``."""
    lib = native.lib()
    if x.dtype != torch.bfloat16 or not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
        raise TypeError("activations must be a bf16 CUDA matrix with unit inner stride")
    m, k = x.shape
    a8 = torch.empty(m, k, dtype=torch.uint8, device=x.device)
    sa = torch.empty(m, dtype=torch.float32, device=x.device)
    native.check(lib.tk_quant_act_rows(x.data_ptr(), x.stride(0), a8.data_ptr(), k, sa.data_ptr(), m, k, int(mode), _stream()), "tk_quant_act_rows")
    return a8.view(torch.float8_e4m3fn), sa


def w8a8_gemm(
    a8: torch.Tensor, sa: torch.Tensor, w: PackedWeight, *, resid: torch.Tensor | None = None, out: torch.Tensor | None = None,
    split_k: int = 0, ws: Workspace | None = None,
) -> torch.Tensor:  # fmt: skip
    """``bf16((a8 @ W8^T) * sa[m] * sw[n])`` (``+ residual``) on the fp8 matrix instruction."""
    lib = native.lib()
    if a8.dtype == torch.float8_e4m3fn:
        a8 = a8.view(torch.uint8)
    if a8.dtype != torch.uint8 or a8.dim() != 2 or a8.shape[1] != w.k or a8.stride(1) != 1:
        raise TypeError(f"a8 must be e4m3fn codes [M, {w.k}] with unit inner stride")
    m = a8.shape[0]
    if sa.dtype != torch.float32 or sa.numel() != m or not sa.is_contiguous():
        raise ValueError("sa must be contiguous fp32 [M]")
    if out is None:
        out = torch.empty(m, w.n, dtype=torch.bfloat16, device=a8.device)
    rp, ldr, rdt = _resid_args(resid, m, w.n)
    ws = ws or default_workspace(a8.device)
    rc = lib.tk_w8a8_gemm(
        a8.data_ptr(), a8.stride(0), sa.data_ptr(), w.data.data_ptr(), w.scale.data_ptr(), out.data_ptr(), out.stride(0), rp, ldr, rdt,
        m, w.n, w.k, split_k, ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_w8a8_gemm")
    return out


def w8a8_gated_ffn(
    x: torch.Tensor, wgu: PackedGateUp, wd: PackedWeight, act: str = "gelu_tanh", *, resid: torch.Tensor | None = None,
    out: torch.Tensor | None = None, ws: Workspace | None = None, mode: str = "fp32",
) -> torch.Tensor:  # fmt: skip
    """The W8A8 MLP: quantise, gate/up with the gated epilogue, quantise, down (``+ residual``).  ``mode``: the
    activation quantisation of both steps, ``"bf16"`` = the reference prefill's (scale and quotient rounded to bf16,
    tybok/policies/pi05/models/triton_prefill_mlp.py:26-59), ``"fp32"`` = one rounding."""
    if mode not in ("fp32", "bf16"):
        raise ValueError(f"unknown quantisation mode {mode!r}")
    lib = native.lib()
    m, ldx = _check_act(x, wgu.k)
    if wd.k != wgu.i or wd.n != wgu.k:
        raise ValueError("down weight must be [K, I]")
    if out is None:
        out = torch.empty(m, wd.n, dtype=torch.bfloat16, device=x.device)
    rp, ldr, rdt = _resid_args(resid, m, wd.n)
    ws = ws or default_workspace(x.device)
    rc = lib.tk_w8a8_gated_ffn(
        x.data_ptr(), ldx, wgu.data.data_ptr(), wgu.scale_gate.data_ptr(), wgu.scale_up.data_ptr(), wd.data.data_ptr(),
        wd.scale.data_ptr(), out.data_ptr(), out.stride(0), rp, ldr, rdt, m, wgu.k, wgu.i, ACT[act], 1 if mode == "bf16" else 0,
        ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_w8a8_gated_ffn")
    return out


def w8a8_ffn_intermediates(ws: Workspace, m: int, k: int, i: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Views of what the last :func:`w8a8_gated_ffn` of this shape left in ``ws``: the bf16 intermediate ``[m, i]``,
    its e4m3fn codes ``[m, i]`` and their fp32 row scales ``[m]``."""
    import ctypes

    offs = [ctypes.c_size_t() for _ in range(3)]
    native.check(native.lib().tk_w8a8_ffn_layout(m, k, i, *(ctypes.addressof(o) for o in offs)), "tk_w8a8_ffn_layout")
    h_off, h8_off, sh_off = (int(o.value) for o in offs)
    h = ws.buf[h_off : h_off + m * i * 2].view(torch.bfloat16).view(m, i)
    h8 = ws.buf[h8_off : h8_off + m * i].view(torch.float8_e4m3fn).view(m, i)
    sh = ws.buf[sh_off : sh_off + m * 4].view(torch.float32)
    return h, h8, sh


def pack_bf16_weight(w: torch.Tensor, rope_half: int = 0) -> PackedBf16Weight:
    """Row-major bf16 ``[N, K]`` -> :class:`PackedBf16Weight` (once per model).  An fp16 matrix is packed the same way
    (the tile order moves 16-bit words) for :func:`bf16w_dense` on fp16 activations."""
    lib = native.lib()
    if w.dtype not in (torch.bfloat16, torch.float16) or not w.is_cuda or w.dim() != 2:
        raise TypeError("expected a bf16 (or fp16) CUDA matrix")
    if w.dtype == torch.float16 and rope_half:
        raise ValueError("fp16 weights serve the many-row kernel only (natural tile order)")
    w = w.contiguous()
    n, k = w.shape
    out = torch.empty(int(lib.tk_bf16w_packed_bytes(n, k)), dtype=torch.uint8, device=w.device)
    native.check(lib.tk_pack_bf16_weight(w.data_ptr(), out.data_ptr(), n, k, rope_half, _stream()), "tk_pack_bf16_weight")
    return PackedBf16Weight(out, n, k, rope_half, w.dtype)


_DENSE_ACTS = {None: 0, "none": 0, "gelu_tanh": 1, "gelu_tanh_fp32": 2}


def bf16w_dense(
    x: torch.Tensor,
    w: PackedBf16Weight,
    bias: torch.Tensor | None = None,
    act: str | None = None,
    *,
    resid: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    tile: int = 0,
    split_k: int = 0,
    ws: Workspace | None = None,
    vt_out: torch.Tensor | None = None,
    vt_col0: int = 0,
) -> torch.Tensor:
    """``bf16(resid + act(bf16(x @ W^T + bias)))`` for ``x [M, K]`` bf16 and a packed bf16 weight: the linears of the
    vision towers on the many-row MFMA kernel.  With ``vt_out [B, G, D, P]`` (``B * P == M``, ``P`` a multiple of 32,
    ``G * D == N - vt_col0``) the columns from ``vt_col0`` on are also written transposed per problem -- the V^T
    operand of :func:`batched_attn` straight from a packed q|k|v projection (``tk_bf16w_dense_vt``; no ``act`` /
    ``resid`` in that form).  ``act``: ``"gelu_tanh"`` applies the tanh GELU to the bf16-rounded
    linear output (what ``gelu(linear(x))`` on bf16 tensors computes), ``"gelu_tanh_fp32"`` to the fp32 one (a GEMM
    with the activation in its epilogue).  ``tile`` picks the block tile (0 = by shape).  With fp16 activations and
    a weight packed from an fp16 matrix every 16-bit operand is fp16 (``tk_f16w_dense``: pi0.5's fp16 tower tiers)."""
    lib = native.lib()
    if w.rope_half:
        raise ValueError("bf16w_dense takes weights packed in natural tile order (rope_half = 0)")
    dt = w.dtype
    if x.dtype != dt or not x.is_cuda or x.dim() != 2 or x.shape[1] != w.k or x.stride(1) != 1:
        raise ValueError(f"activations must be a CUDA [M, {w.k}] matrix of the weight's type with unit inner stride")
    m, ldx = x.shape[0], x.stride(0)
    if bias is not None and (bias.dtype != dt or bias.numel() != w.n or not bias.is_contiguous() or bias.device != x.device):
        raise ValueError(f"bias must be a contiguous vector of {w.n} elements of the weight's type on the activations' device")
    if out is None:
        out = torch.empty(m, w.n, dtype=dt, device=x.device)
    if out.dtype != dt or out.shape != (m, w.n) or out.stride(1) != 1:
        raise ValueError("out must be [M, N] of the weight's type with unit inner stride")
    if resid is not None and resid.dtype == torch.float16 and dt == torch.float16:
        if resid.shape != (m, w.n) or resid.stride(1) != 1:
            raise ValueError("residual must be [M, N] with unit inner stride")
        rp, ldr, rdt = resid.data_ptr(), resid.stride(0), _BF16  # the 16-bit residual of the kernel's flavour
    else:
        rp, ldr, rdt = _resid_args(resid, m, w.n)
        if dt == torch.float16 and resid is not None and resid.dtype == torch.bfloat16:
            raise TypeError("an fp16 launch takes an fp16 or fp32 residual")
    ws = ws or default_workspace(x.device)
    if vt_out is not None:
        if act is not None or resid is not None:
            raise ValueError("vt_out: no activation or residual in this form")
        if vt_out.dtype != dt or vt_out.dim() != 4 or vt_out.stride(3) != 1 or vt_out.stride(1) != vt_out.shape[2] * vt_out.stride(2):
            raise ValueError("vt_out must be [B, G, D, P] of the weight's type with contiguous keys and evenly pitched (g, d) rows")
        nb, ng, nd, npk = vt_out.shape
        if nb * npk != m or npk % 32 or ng * nd != w.n - vt_col0:
            raise ValueError("vt_out: B * P must equal M, P be a multiple of 32 and G * D equal N - vt_col0")
        rc = lib.tk_bf16w_dense_vt(
            x.data_ptr(), ldx, w.data.data_ptr(), None if bias is None else bias.data_ptr(), out.data_ptr(), out.stride(0), vt_out.data_ptr(),
            vt_col0, vt_out.stride(2), npk, vt_out.stride(0), int(dt == torch.float16), m, w.n, w.k, tile, split_k, ws.ptr, ws.nbytes, _stream(),
        )  # fmt: skip
        native.check(rc, "tk_bf16w_dense_vt")
        return out
    entry = lib.tk_f16w_dense if dt == torch.float16 else lib.tk_bf16w_dense
    rc = entry(
        x.data_ptr(), ldx, w.data.data_ptr(), None if bias is None else bias.data_ptr(), _DENSE_ACTS[act], out.data_ptr(),
        out.stride(0), rp, ldr, rdt, m, w.n, w.k, tile, split_k, ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_f16w_dense" if dt == torch.float16 else "tk_bf16w_dense")
    return out


def bf16w_dense_rope(
    x: torch.Tensor,
    w: PackedBf16Weight,
    rope: "RopeTables",
    rope_pos: torch.Tensor,
    rope_cols: int,
    *,
    rope_bf16: bool = False,
    vt_out: torch.Tensor | None = None,
    vt_col0: int = 0,
    out: torch.Tensor | None = None,
    tile: int = 0,
    split_k: int = 0,
    ws: Workspace | None = None,
) -> torch.Tensor:
    """The many-row linear with the rotary epilogue: ``bf16(x @ W^T)`` for ``x [M, K]`` bf16 and a weight packed in
    rotary pair order (``pack_bf16_weight(w, rope_half)``), the columns ``< rope_cols`` rotated by the table row of
    ``rope_pos[m]``, and with ``vt_out [N - vt_col0, >= M rounded up to 32]`` the columns from ``vt_col0`` on also
    written transposed -- a many-row prefill's q|k|v projection in one launch (``tk_bf16w_dense_rope``)."""
    lib = native.lib()
    if w.dtype != torch.bfloat16 or not w.rope_half or rope.half != w.rope_half:
        raise ValueError("the weight must be bf16, packed in rotary pair order with the tables' rope_half")
    if x.dtype != torch.bfloat16 or not x.is_cuda or x.dim() != 2 or x.shape[1] != w.k or x.stride(1) != 1:
        raise ValueError(f"activations must be a CUDA bf16 [M, {w.k}] matrix with unit inner stride")
    m = x.shape[0]
    if rope_pos.dtype != torch.int32 or rope_pos.numel() != m or not rope_pos.is_contiguous():
        raise ValueError("rope_pos must be a contiguous int32 [M]")
    if rope.cos.dtype != torch.float32 or not rope.cos.is_contiguous() or not rope.sin.is_contiguous():
        raise ValueError("rotary tables must be contiguous fp32")
    if out is None:
        out = torch.empty(m, w.n, dtype=torch.bfloat16, device=x.device)
    if out.dtype != torch.bfloat16 or out.shape != (m, w.n) or out.stride(1) != 1:
        raise ValueError("out must be bf16 [M, N] with unit inner stride")
    vt_p, vt_ld = None, 0
    if vt_out is not None:
        if vt_out.dtype != torch.bfloat16 or vt_out.dim() != 2 or vt_out.stride(1) != 1 or vt_out.shape[0] != w.n - vt_col0:
            raise ValueError("vt_out must be bf16 [N - vt_col0, >= M] with unit inner stride")
        vt_p, vt_ld = vt_out.data_ptr(), vt_out.stride(0)
    ws = ws or default_workspace(x.device)
    rc = lib.tk_bf16w_dense_rope(
        x.data_ptr(), x.stride(0), w.data.data_ptr(), out.data_ptr(), out.stride(0), rope_pos.data_ptr(), rope.cos.data_ptr(),
        rope.sin.data_ptr(), rope.positions, rope_cols, rope.half, int(rope_bf16), vt_p, vt_col0, vt_ld, m, w.n, w.k, tile, split_k,
        ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_bf16w_dense_rope")
    return out


def _norm_ptr(norm_w: torch.Tensor | None, k: int) -> int | None:
    if norm_w is None:
        return None
    if norm_w.dtype != torch.bfloat16 or norm_w.numel() != k or not norm_w.is_contiguous():
        raise ValueError(f"norm weight must be a contiguous bf16 tensor of {k} elements")
    return norm_w.data_ptr()


def _ada_ptrs(ada, k: int) -> tuple[int | None, int | None]:
    if ada is None:
        return None, None
    scale, shift = ada
    for t in (scale, shift):
        if t.dtype != torch.float32 or t.numel() != k or t.stride(-1) != 1:
            raise ValueError(f"adaptive-norm scale / shift must be fp32 vectors of {k} contiguous elements")
    return scale.data_ptr(), shift.data_ptr()


def bf16w_linear(
    x: torch.Tensor,
    w: PackedBf16Weight,
    *,
    norm_w: torch.Tensor | None = None,
    eps: float = 0.0,
    ada: tuple[torch.Tensor, torch.Tensor] | None = None,
    rope: RopeTables | None = None,
    rope_pos: torch.Tensor | None = None,
    rope_cols: int = 0,
    rope_bf16: bool = False,
    vt_out: torch.Tensor | None = None,
    vt_col0: int = 0,
    resid: torch.Tensor | None = None,
    gate: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    split_k: int = 0,
    ws: Workspace | None = None,
) -> torch.Tensor:
    """``x [M, K] @ W^T`` with bf16 weights; optional RMSNorm prologue (``x`` bf16 or fp32), and
    either a rotary epilogue (``rope`` tables, int32 ``rope_pos [M]``, columns ``< rope_cols``
    rotated; with ``vt_out [N - vt_col0, >= M]`` the columns from ``vt_col0`` on are also written
    transposed) or a (gated) residual epilogue.  ``ada = (scale, shift)``, fp32 ``[K]`` each,
    selects the adaptive RMSNorm prologue instead of ``norm_w``; ``rope_bf16`` the bf16-arithmetic
    rotation."""
    lib = native.lib()
    if not x.is_cuda or x.dim() != 2 or x.shape[1] != w.k or x.stride(1) != 1:
        raise ValueError(f"activations must be CUDA [M, {w.k}] with unit inner stride")
    if x.dtype == torch.float32:
        if norm_w is None:
            raise TypeError("fp32 activations are accepted with the norm prologue only")
        xdt = _F32
    elif x.dtype == torch.bfloat16:
        xdt = _BF16
    else:
        raise TypeError("activations must be bf16 or fp32")
    m = x.shape[0]
    if out is None:
        out = torch.empty(m, w.n, dtype=torch.bfloat16, device=x.device)
    rp, ldr, rdt = _resid_args(resid, m, w.n)
    pos_p = cos_p = sin_p = None
    positions = half = 0
    if rope is not None:
        if rope_pos is None or rope_pos.dtype != torch.int32 or rope_pos.numel() != m or not rope_pos.is_contiguous():
            raise ValueError("rope_pos must be a contiguous int32 [M]")
        if rope.half != w.rope_half:
            raise ValueError("weight was packed for a different rotary head size")
        if rope.cos.dtype != torch.float32 or not rope.cos.is_contiguous() or not rope.sin.is_contiguous():
            raise ValueError("rotary tables must be contiguous fp32")
        pos_p, cos_p, sin_p = rope_pos.data_ptr(), rope.cos.data_ptr(), rope.sin.data_ptr()
        positions, half = rope.positions, rope.half
    elif w.rope_half:
        raise ValueError("a weight packed in rotary pair order needs the rotary epilogue")
    vt_p, vt_ld = None, 0
    if vt_out is not None:
        if vt_out.dtype != torch.bfloat16 or vt_out.dim() != 2 or vt_out.stride(1) != 1 or vt_out.shape[0] != w.n - vt_col0:
            raise ValueError("vt_out must be bf16 [N - vt_col0, >= M] with unit inner stride")
        vt_p, vt_ld = vt_out.data_ptr(), vt_out.stride(0)
    ws = ws or default_workspace(x.device)
    rc = lib.tk_bf16w_linear(
        x.data_ptr(), x.stride(0), xdt, w.data.data_ptr(), _norm_ptr(norm_w, w.k), float(eps), *_ada_ptrs(ada, w.k),
        pos_p, cos_p, sin_p, positions, rope_cols, half, int(rope_bf16), vt_p, vt_col0, vt_ld, out.data_ptr(),
        out.stride(0), rp, ldr, rdt, _gate_ptr(gate, w.n), m, w.n, w.k, split_k, ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_bf16w_linear")
    return out


def _eff_strides(t: torch.Tensor) -> tuple[int, int]:
    """(row, head) element strides of a ``[L, G, D]`` view; a size-1 dim never advances, so its
    stride is reported as 0 whatever torch recorded for it."""
    return (t.stride(0) if t.shape[0] > 1 else 0, t.stride(1) if t.shape[1] > 1 else 0)


def _same_layout(k: torch.Tensor, v: torch.Tensor) -> bool:
    return k.shape == v.shape and k.stride(2) == 1 and v.stride(2) == 1 and _eff_strides(k) == _eff_strides(v)


@dataclass
class PrefixKV:
    """One layer's prefix K/V in the attention kernel's layout (see :func:`prepare_prefix_kv`)."""

    k: torch.Tensor  # bf16 [P, G, D] (any row / head strides, d contiguous)
    vt: torch.Tensor  # bf16 [G, D, P rounded up to 32], zero padded
    k_lo: torch.Tensor | None = None  # low planes when the source was fp32
    vt_lo: torch.Tensor | None = None

    @property
    def length(self) -> int:
        return self.k.shape[0]


@dataclass
class SuffixKV:
    """The action tokens' own K ``[S, G, D]`` and V^T ``[G, D, >= S rounded up to 32]`` (zero padded)."""

    k: torch.Tensor
    vt: torch.Tensor


def _pad32(n: int) -> int:
    return (n + 31) // 32 * 32


def prepare_prefix_kv(k: torch.Tensor, v: torch.Tensor) -> PrefixKV:
    """``k, v [P, G, D]`` (bf16 or fp32 views sharing strides) -> :class:`PrefixKV`, one launch.

    bf16: ``k`` is used in place, ``v`` is transposed.  fp32: both are split into bf16 hi + lo planes.
    """
    lib = native.lib()
    if k.dtype != v.dtype or k.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError("prefix K/V must both be bf16 or both fp32")
    if not _same_layout(k, v):
        raise ValueError("prefix K and V must share strides and have a contiguous head dim")
    p, g, d = k.shape
    sl, sh = _eff_strides(k)
    bf = dict(dtype=torch.bfloat16, device=k.device)
    vt = torch.empty(g, d, _pad32(p), **bf)
    if k.dtype == torch.float32:
        k_hi, k_lo, vt_lo = torch.empty(p, g, d, **bf), torch.empty(p, g, d, **bf), torch.empty_like(vt)
        rc = lib.tk_attn_prepare_kv(k.data_ptr(), v.data_ptr(), _F32, sl, sh, p, g, d, k_hi.data_ptr(), k_lo.data_ptr(),
                                    vt.data_ptr(), vt_lo.data_ptr(), vt.shape[2], _stream())  # fmt: skip
        native.check(rc, "tk_attn_prepare_kv")
        return PrefixKV(k_hi, vt, k_lo, vt_lo)
    rc = lib.tk_attn_prepare_kv(None, v.data_ptr(), _BF16, sl, sh, p, g, d, None, None, vt.data_ptr(), None, vt.shape[2],
                                _stream())  # fmt: skip
    native.check(rc, "tk_attn_prepare_kv")
    return PrefixKV(k, vt)


def project_prefix_kv(k: torch.Tensor, v: torch.Tensor, wk: torch.Tensor, wv: torch.Tensor, d: int) -> PrefixKV:
    """fp32 expert K/V projection of a cached prefix, straight into the attention operand layout:
    ``k, v [P, KV]`` bf16 rows (views with a contiguous last dim and the same row stride), ``wk, wv
    [N, KV]`` fp32 -> :class:`PrefixKV` of ``float(k) @ wk.T`` / ``float(v) @ wv.T`` as bf16 hi + lo
    planes (``[P, N/d, d]`` and ``[N/d, d, P rounded up to 32]``).  One launch."""
    lib = native.lib()
    bf = torch.bfloat16
    if k.dtype != bf or v.dtype != bf or wk.dtype != torch.float32 or wv.dtype != torch.float32:
        raise TypeError("project_prefix_kv: k, v bf16 and wk, wv fp32")
    p, kv = k.shape
    n = wk.shape[0]
    if v.shape != k.shape or wk.shape != (n, kv) or wv.shape != (n, kv) or n % d or k.stride(1) != 1 or v.stride(1) != 1 or k.stride(0) != v.stride(0):
        raise ValueError("project_prefix_kv: k, v [P, KV] with equal row strides; wk, wv [N, KV]; N a multiple of d")
    wk, wv = wk.contiguous(), wv.contiguous()
    g = n // d
    opts = dict(dtype=bf, device=k.device)
    k_hi, k_lo = torch.empty(p, g, d, **opts), torch.empty(p, g, d, **opts)
    vt_hi, vt_lo = torch.empty(g, d, _pad32(p), **opts), torch.empty(g, d, _pad32(p), **opts)
    rc = lib.tk_expert_kv_project(k.data_ptr(), v.data_ptr(), k.stride(0), p, kv, wk.data_ptr(), wv.data_ptr(), n, k_hi.data_ptr(),
                                  k_lo.data_ptr(), vt_hi.data_ptr(), vt_lo.data_ptr(), vt_hi.shape[2], _stream())  # fmt: skip
    native.check(rc, "tk_expert_kv_project")
    return PrefixKV(k_hi, vt_hi, k_lo, vt_lo)


def project_prefix_kv_layers(ks, vs, wks, wvs, d: int) -> list[PrefixKV]:
    """:func:`project_prefix_kv` for several layers (at most 16) in one launch: lists of per-layer ``k, v [P, KV]`` views
    (one shape and row stride) and ``wk, wv [N, KV]`` fp32 weights -> one :class:`PrefixKV` per layer (views of stacked
    planes).  Same bits as one call per layer."""
    import ctypes

    lib = native.lib()
    bf = torch.bfloat16
    n_layers = len(ks)
    if not (1 <= n_layers <= 16) or not (len(vs) == len(wks) == len(wvs) == n_layers):
        raise ValueError("project_prefix_kv_layers: 1..16 layers, four lists of the same length")
    p, kv = ks[0].shape
    n = wks[0].shape[0]
    sl = ks[0].stride(0)
    wks, wvs = [w.contiguous() for w in wks], [w.contiguous() for w in wvs]
    for k, v, wk, wv in zip(ks, vs, wks, wvs):
        if k.dtype != bf or v.dtype != bf or wk.dtype != torch.float32 or wv.dtype != torch.float32:
            raise TypeError("project_prefix_kv_layers: k, v bf16 and wk, wv fp32")
        if k.shape != (p, kv) or v.shape != (p, kv) or wk.shape != (n, kv) or wv.shape != (n, kv) or n % d or k.stride(1) != 1 or v.stride(1) != 1 or k.stride(0) != sl or v.stride(0) != sl:
            raise ValueError("project_prefix_kv_layers: every layer k, v [P, KV] with one row stride; wk, wv [N, KV]; N a multiple of d")
    g = n // d
    opts = dict(dtype=bf, device=ks[0].device)
    k_hi, k_lo = torch.empty(n_layers, p, g, d, **opts), torch.empty(n_layers, p, g, d, **opts)
    vt_hi, vt_lo = torch.empty(n_layers, g, d, _pad32(p), **opts), torch.empty(n_layers, g, d, _pad32(p), **opts)
    arr = ctypes.c_void_p * n_layers
    rc = lib.tk_expert_kv_project_layers(
        n_layers, arr(*(t.data_ptr() for t in ks)), arr(*(t.data_ptr() for t in vs)), sl, p, kv, arr(*(t.data_ptr() for t in wks)),
        arr(*(t.data_ptr() for t in wvs)), n, k_hi.data_ptr(), k_lo.data_ptr(), vt_hi.data_ptr(), vt_lo.data_ptr(), vt_hi.shape[3], _stream(),
    )  # fmt: skip
    native.check(rc, "tk_expert_kv_project_layers")
    return [PrefixKV(k_hi[i], vt_hi[i], k_lo[i], vt_lo[i]) for i in range(n_layers)]


def expert_attn(
    q: torch.Tensor,
    prefix: PrefixKV | None,
    suffix: SuffixKV | None,
    prefix_pad: torch.Tensor | None,
    mask_mode: int,
    *,
    mask2d: torch.Tensor | None = None,
    logits_bf16: bool = False,
    out: torch.Tensor | None = None,
    ws: Workspace | None = None,
) -> torch.Tensor:
    """Attention of ``q [M, H, D]`` over ``[prefix; suffix]`` keys.  ``prefix_pad``: uint8/bool
    ``[P]`` or None; ``mask2d``: uint8/bool ``[M, >= P rounded up to 32]`` per-(query, prefix key)
    visibility, replaces ``prefix_pad``.  Returns bf16 ``[M, H*D]``."""
    lib = native.lib()
    if q.dtype != torch.bfloat16 or q.dim() != 3 or q.stride(2) != 1:
        raise TypeError("q must be bf16 [M, H, D] with a contiguous head dim")
    m, h, d = q.shape
    bf = torch.bfloat16

    def _vt_ok(vt: torch.Tensor, g: int, length: int) -> bool:
        return vt.dtype == bf and vt.dim() == 3 and vt.shape[:2] == (g, d) and vt.stride(2) == 1 and vt.shape[2] >= _pad32(length)

    p = g = 0
    kp = kpl = vp = vpl = None
    pre_sl = pre_sh = pre_sd = pre_vsh = 0
    if prefix is not None:
        p, g = prefix.k.shape[0], prefix.k.shape[1]
        if prefix.k.dtype != bf or prefix.k.shape[2] != d or prefix.k.stride(2) != 1 or not _vt_ok(prefix.vt, g, p):
            raise ValueError("prefix must hold bf16 K [P, G, D] and V^T [G, D, >= P rounded up to 32]")
        pre_sl, pre_sh = _eff_strides(prefix.k)
        pre_vsh, pre_sd = prefix.vt.stride(0) if g > 1 else 0, prefix.vt.stride(1)
        kp, vp = prefix.k.data_ptr(), prefix.vt.data_ptr()
        if prefix.k_lo is not None:
            if prefix.vt_lo is None or prefix.k_lo.stride() != prefix.k.stride() or prefix.vt_lo.stride() != prefix.vt.stride():
                raise ValueError("low planes must mirror the high planes' layout")
            kpl, vpl = prefix.k_lo.data_ptr(), prefix.vt_lo.data_ptr()
    s = 0
    ks = vs = None
    suf_sl = suf_sh = suf_sd = suf_vsh = 0
    if suffix is not None:
        s, gs = suffix.k.shape[0], suffix.k.shape[1]
        if prefix is not None and gs != g:
            raise ValueError("prefix and suffix must have the same number of kv heads")
        g = gs
        if suffix.k.dtype != bf or suffix.k.shape[2] != d or suffix.k.stride(2) != 1 or not _vt_ok(suffix.vt, g, s):
            raise ValueError("suffix must hold bf16 K [S, G, D] and V^T [G, D, >= S rounded up to 32]")
        suf_sl, suf_sh = _eff_strides(suffix.k)
        suf_vsh, suf_sd = suffix.vt.stride(0) if g > 1 else 0, suffix.vt.stride(1)
        ks, vs = suffix.k.data_ptr(), suffix.vt.data_ptr()
    pad = None
    if prefix_pad is not None:
        pad = prefix_pad.view(torch.uint8) if prefix_pad.dtype == torch.bool else prefix_pad
        if pad.dtype != torch.uint8 or pad.numel() != p or not pad.is_contiguous():
            raise ValueError("prefix_pad must be a contiguous uint8/bool [P]")
    m2_p, m2_ld = None, 0
    if mask2d is not None:
        m2 = mask2d.view(torch.uint8) if mask2d.dtype == torch.bool else mask2d
        if m2.dtype != torch.uint8 or m2.dim() != 2 or m2.shape[0] != m or m2.stride(1) != 1 or m2.shape[1] < _pad32(p):
            raise ValueError("mask2d must be uint8/bool [M, >= P rounded up to 32] with unit inner stride")
        m2_p, m2_ld = m2.data_ptr(), m2.stride(0)
    if out is None:
        out = torch.empty(m, h * d, dtype=bf, device=q.device)
    ws = ws or default_workspace(q.device)
    rc = lib.tk_expert_attn(
        q.data_ptr(), q.stride(0), q.stride(1), kp, kpl, pre_sl, pre_sh, vp, vpl, pre_sd, pre_vsh, ks, suf_sl, suf_sh,
        vs, suf_sd, suf_vsh, _ptr(pad), m2_p, m2_ld, out.data_ptr(), out.stride(0), m, p, s, h, max(g, 1), d, mask_mode,
        int(logits_bf16), ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_expert_attn")
    return out


CROSS_FUSED_MAX_K = 768    # widest hidden size the in-kernel q projection stages
CROSS_FUSED_MAX_P = 256    # 8 key tiles: one block of 8 waves covers the prefix


def cross_attn_fused(
    x: torch.Tensor,
    wq: PackedBf16Weight,
    norm_w: torch.Tensor,
    eps: float,
    rope: RopeTables,
    rope_pos: torch.Tensor,
    prefix: PrefixKV,
    prefix_pad: torch.Tensor | None,
    *,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Cross layer in one launch: ``q = rope(RMSNorm(x) @ Wq^T)`` computed per head inside the
    attention kernel, then attention over the fp32 (hi + lo planes) prefix ``K/V`` under the pad
    mask.  ``x [M, K]`` bf16 (``K <= 768``), ``wq`` packed with ``rope_half = 32`` (head size 64),
    ``prefix`` from :func:`project_prefix_kv` / :func:`prepare_prefix_kv` of fp32 tensors with at most
    256 keys.  Returns bf16 ``[M, H*64]``; equals :func:`bf16w_linear` + :func:`expert_attn`."""
    lib = native.lib()
    bf = torch.bfloat16
    if x.dtype != bf or x.dim() != 2 or x.stride(1) != 1 or norm_w.dtype != bf:
        raise TypeError("cross_attn_fused: x [M, K] and norm_w must be bf16, x rows contiguous")
    m, k = x.shape
    if wq.k != k or norm_w.numel() != k or wq.rope_half != 32 or wq.n % 64:
        raise ValueError("cross_attn_fused: wq must be the [H*64, K] q weight packed with rope_half=32")
    if prefix.k_lo is None or prefix.vt_lo is None:
        raise ValueError("cross_attn_fused: the prefix must carry hi + lo planes (fp32 expert K/V)")
    h, d = wq.n // 64, 64
    p, g = prefix.k.shape[0], prefix.k.shape[1]
    if prefix.k.shape[2] != d or prefix.k_lo.stride() != prefix.k.stride() or prefix.vt_lo.stride() != prefix.vt.stride():
        raise ValueError("cross_attn_fused: prefix planes must be [P, G, 64] / [G, 64, >= P rounded up to 32] with mirrored layouts")
    if rope_pos.dtype != torch.int32 or rope_pos.numel() != m or not rope_pos.is_contiguous():
        raise ValueError("cross_attn_fused: rope_pos must be a contiguous int32 [M]")
    pad = None
    if prefix_pad is not None:
        pad = prefix_pad.view(torch.uint8) if prefix_pad.dtype == torch.bool else prefix_pad
        if pad.dtype != torch.uint8 or pad.numel() != p or not pad.is_contiguous():
            raise ValueError("prefix_pad must be a contiguous uint8/bool [P]")
    if out is None:
        out = torch.empty(m, h * d, dtype=bf, device=x.device)
    pre_sl, pre_sh = _eff_strides(prefix.k)
    rc = lib.tk_expert_cross_attn_fused(
        x.data_ptr(), x.stride(0), norm_w.data_ptr(), float(eps), wq.data.data_ptr(), k, rope_pos.data_ptr(), rope.cos.data_ptr(),
        rope.sin.data_ptr(), rope.cos.shape[0], prefix.k.data_ptr(), prefix.k_lo.data_ptr(), pre_sl, pre_sh, prefix.vt.data_ptr(),
        prefix.vt_lo.data_ptr(), prefix.vt.stride(1), prefix.vt.stride(0) if g > 1 else 0, _ptr(pad), out.data_ptr(), out.stride(0),
        m, p, h, g, d, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_expert_cross_attn_fused")
    return out


def batched_attn(
    q: torch.Tensor,
    k: torch.Tensor,
    vt: torch.Tensor,
    *,
    logits_bf16: bool = False,
    scale: float | None = None,
    out: torch.Tensor | None = None,
    ws: Workspace | None = None,
) -> torch.Tensor:
    """``B`` independent unmasked attentions: ``q [B, M, H, D]``, ``k [B, P, G, D]`` (views with a
    contiguous head dim), ``vt [B, G, D, >= P rounded up to 32]`` (V transposed, zero padded) ->
    bf16 ``[B, M, H*D]``.  ``scale`` multiplies the logits (default ``D ** -0.5``; a head padded with
    zero columns up to a supported ``D`` passes the scale of its true size)."""
    lib = native.lib()
    bf = torch.bfloat16
    if q.dtype == torch.float16:
        # fp16 operands (pi0.5's fused tower): fp32 logits, probabilities rounded to fp16, bf16 output
        if logits_bf16:
            raise ValueError("fp16 operands keep the logits in fp32")
        logits_bf16 = 2
    elif q.dtype != bf:
        raise TypeError("q, k, vt must be 4-D bf16 (or fp16) tensors")
    if k.dtype != q.dtype or vt.dtype != q.dtype or q.dim() != 4 or k.dim() != 4 or vt.dim() != 4:
        raise TypeError("q, k, vt must be 4-D tensors of one 16-bit type")
    b, m, h, d = q.shape
    p, g = k.shape[1], k.shape[2]
    if k.shape[0] != b or k.shape[3] != d or vt.shape[:3] != (b, g, d) or vt.shape[3] < _pad32(p):
        raise ValueError("k must be [B, P, G, D] and vt [B, G, D, >= P rounded up to 32]")
    if q.stride(3) != 1 or k.stride(3) != 1 or vt.stride(3) != 1:
        raise ValueError("q, k need a contiguous head dim and vt contiguous keys")
    if out is None:
        out = torch.empty(b, m, h * d, dtype=bf, device=q.device)
    ws = ws or default_workspace(q.device)
    rc = lib.tk_batched_attn(
        q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), k.data_ptr(), k.stride(0), k.stride(1), k.stride(2) if g > 1 else 0,
        vt.data_ptr(), vt.stride(0), vt.stride(2), vt.stride(1) if g > 1 else 0, out.data_ptr(), out.stride(0), out.stride(1),
        b, m, p, h, g, d, int(logits_bf16), float(scale or 0.0), ws.ptr, ws.nbytes, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_batched_attn")
    return out


def linear_gelu_tanh(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``gelu_tanh(x @ weight^T + bias)`` for bf16 operands on the GPU as ONE library GEMM with the bias and the
    activation in its epilogue (the vision towers' fc1: 32 us instead of 46 us as GEMM + elementwise launch at
    3072 x 768 -> 3072).  The epilogue evaluates the tanh form on the fp32 accumulator, so the one difference
    from ``F.gelu(F.linear(...), approximate="tanh")`` is that the pre-activation is not rounded to bf16 first."""
    if not (x.is_cuda and x.dtype == weight.dtype == bias.dtype == torch.bfloat16):
        raise TypeError("linear_gelu_tanh: bf16 CUDA operands only")
    y = torch._addmm_activation(bias, x.reshape(-1, x.shape[-1]), weight.t(), use_gelu=True)
    return y.view(*x.shape[:-1], weight.shape[0])


def transpose_v(v: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """``v [B, P, G, D]`` bf16 (a view with a contiguous head dim, e.g. into a packed q|k|v buffer) ->
    ``vt [B, G, D, P rounded up to 32]`` with zero-filled padding keys: the V^T operand of
    :func:`batched_attn`, one launch for all problems.  ``D`` in {64, 96}."""
    lib = native.lib()
    if v.dtype not in (torch.bfloat16, torch.float16) or v.dim() != 4 or v.stride(3) != 1:
        raise TypeError("v must be a 4-D bf16 (or fp16) tensor with a contiguous head dim")
    b, p, g, d = v.shape
    if out is None:
        out = torch.empty(b, g, d, _pad32(p), dtype=v.dtype, device=v.device)
    if out.shape[:3] != (b, g, d) or out.shape[3] < _pad32(p) or out.stride(3) != 1 or out.dtype != v.dtype:
        raise ValueError("out must be [B, G, D, >= P rounded up to 32] of v's type with contiguous keys")
    rc = lib.tk_batched_transpose_v(
        v.data_ptr(), v.stride(0), v.stride(1), v.stride(2), out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
        out.shape[3], b, p, g, d, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_batched_transpose_v")
    return out


def expert_attn_plain(
    q: torch.Tensor,
    k_pre: torch.Tensor | None,
    v_pre: torch.Tensor | None,
    k_suf: torch.Tensor | None,
    v_suf: torch.Tensor | None,
    prefix_pad: torch.Tensor | None,
    mask_mode: int,
    **kw,
) -> torch.Tensor:
    """:func:`expert_attn` on plain ``[L, G, D]`` K/V tensors: lays the prefix out with
    :func:`prepare_prefix_kv` and transposes the suffix values with torch, then calls the kernel."""
    prefix = prepare_prefix_kv(k_pre, v_pre) if k_pre is not None and k_pre.shape[0] > 0 else None
    suffix = None
    if k_suf is not None and k_suf.shape[0] > 0:
        s, g, d = k_suf.shape
        vt = torch.zeros(g, d, _pad32(s), dtype=torch.bfloat16, device=k_suf.device)
        vt[:, :, :s] = v_suf.permute(1, 2, 0)
        suffix = SuffixKV(k_suf, vt)
    return expert_attn(q, prefix, suffix, prefix_pad, mask_mode, **kw)


def expert_tail(
    x: torch.Tensor,
    w: torch.Tensor,
    bias: torch.Tensor | None,
    *,
    norm_w: torch.Tensor | None = None,
    ada: tuple[torch.Tensor, torch.Tensor] | None = None,
    eps: float,
    x_t: torch.Tensor | None = None,
    dt: float = 0.0,
    want_v: bool = False,
    embed: tuple[torch.Tensor, torch.Tensor | None, str, torch.Tensor] | None = None,
) -> tuple[torch.Tensor | None, torch.Tensor | None]:
    """Final norm of ``x [M, K]`` bf16, fp32 projection with ``w [N, K]`` (+ ``bias``), and -- with
    ``x_t [M, N]`` -- the Euler update ``x_t + dt * v``.  Returns ``(v or None, x_new or None)``.
    ``embed = (E [J, N] fp32, c [J] fp32 or None, "none" | "silu", out [M, J] fp32 or bf16)``: the same launch
    also writes ``out = act(x_new @ E^T + c)``, the next step's suffix embedding."""
    lib = native.lib()
    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.stride(1) != 1:
        raise TypeError("x must be bf16 [M, K] with unit inner stride")
    m, k = x.shape
    if w.dtype != torch.float32 or w.shape[1] != k or not w.is_contiguous():
        raise ValueError("w must be contiguous fp32 [N, K]")
    n = w.shape[0]
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != n or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous fp32 [N]")
    f32 = dict(dtype=torch.float32, device=x.device)
    v = torch.empty(m, n, **f32) if (want_v or x_t is None) else None
    x_new = None
    if x_t is not None:
        if x_t.dtype != torch.float32 or x_t.shape != (m, n) or not x_t.is_contiguous():
            raise ValueError("x_t must be contiguous fp32 [M, N]")
        x_new = torch.empty(m, n, **f32)
    if embed is not None:
        ew, eb, eact, eout = embed
        if x_new is None:
            raise ValueError("embed needs x_t")
        if ew.dtype != torch.float32 or ew.dim() != 2 or ew.shape[1] != n or not ew.is_contiguous():
            raise ValueError("embed weight must be contiguous fp32 [J, N]")
        j = ew.shape[0]
        if eb is not None and (eb.dtype != torch.float32 or eb.numel() != j or not eb.is_contiguous()):
            raise ValueError("embed bias must be contiguous fp32 [J]")
        if eout.dtype not in (torch.float32, torch.bfloat16) or eout.shape != (m, j) or eout.stride(1) != 1:
            raise ValueError("embed out must be fp32 or bf16 [M, J] with unit inner stride")
        if eact not in ("none", "silu"):
            raise ValueError(f"embed activation {eact!r}")
        rc = lib.tk_expert_tail_embed(
            x.data_ptr(), x.stride(0), _norm_ptr(norm_w, k), *_ada_ptrs(ada, k), float(eps), w.data_ptr(), _ptr(bias), _ptr(v),
            _ptr(x_t), _ptr(x_new), float(dt), m, n, k, ew.data_ptr(), _ptr(eb), j, 1 if eact == "silu" else 0, eout.data_ptr(),
            eout.stride(0), _BF16 if eout.dtype == torch.bfloat16 else _F32, _stream(),
        )  # fmt: skip
        native.check(rc, "tk_expert_tail_embed")
        return v, x_new
    rc = lib.tk_expert_tail(
        x.data_ptr(), x.stride(0), _norm_ptr(norm_w, k), *_ada_ptrs(ada, k), float(eps), w.data_ptr(), _ptr(bias), _ptr(v),
        _ptr(x_t), _ptr(x_new), float(dt), m, n, k, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_expert_tail")
    return v, x_new


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``bf16(LayerNorm(x) * w + b)`` over the last dim of ``x [..., K]`` (fp32 with fp32 parameters, or
    bf16 with bf16 parameters; contiguous rows), statistics in fp32.  One launch, bf16 result -- or, for fp32 rows
    and ``out_dtype=torch.float16``, an fp16 one."""
    lib = native.lib()
    if x.dtype not in (torch.float32, torch.bfloat16) or w.dtype != x.dtype or b.dtype != x.dtype:
        raise TypeError("layer_norm: x, w, b must all be fp32 or all bf16")
    k = x.shape[-1]
    x2 = x.reshape(-1, k)
    if x2.stride(1) != 1 or w.numel() != k or b.numel() != k:
        raise ValueError("layer_norm: rows must be contiguous and w, b hold K values")
    if out_dtype == torch.float16:
        if x.dtype != torch.float32:
            raise TypeError("layer_norm: the fp16 result is built for fp32 rows")
        y = torch.empty(x2.shape, dtype=torch.float16, device=x.device)
        rc = lib.tk_layer_norm_f16(x2.data_ptr(), x2.stride(0), w.contiguous().data_ptr(), b.contiguous().data_ptr(), float(eps),
                                   y.data_ptr(), y.stride(0), x2.shape[0], k, _stream())  # fmt: skip
        native.check(rc, "tk_layer_norm_f16")
        return y.view(x.shape)
    y = torch.empty(x2.shape, dtype=torch.bfloat16, device=x.device)
    dt = _F32 if x.dtype == torch.float32 else _BF16
    rc = lib.tk_layer_norm(x2.data_ptr(), x2.stride(0), dt, w.contiguous().data_ptr(), b.contiguous().data_ptr(), dt, float(eps),
                           y.data_ptr(), y.stride(0), x2.shape[0], k, _stream())  # fmt: skip
    native.check(rc, "tk_layer_norm")
    return y.view(x.shape)


def add_layer_norm(
    x: torch.Tensor, r: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, out_dtype: torch.dtype = torch.bfloat16,
    *, y_rows: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:  # fmt: skip
    """``x += r`` in place (``r`` bf16: the linear that closes a residual branch; fp32 ``x`` takes
    ``float(r)``, bf16 ``x`` rounds the sum once) and ``bf16(LayerNorm(x) * w + b)`` of the sum, one launch.
    Returns ``(x, normalised)``; ``x`` must own contiguous rows.  ``y_rows`` (int32, one entry per row of the
    flattened ``x``, a permutation): normalised row ``m`` is written as row ``y_rows[m]`` (bf16 result only)."""
    lib = native.lib()
    if x.dtype not in (torch.float32, torch.bfloat16) or w.dtype != x.dtype or b.dtype != x.dtype or r.dtype != torch.bfloat16:
        raise TypeError("add_layer_norm: x, w, b all fp32 or all bf16; r bf16")
    k = x.shape[-1]
    if r.shape != x.shape or not x.is_contiguous() or w.numel() != k or b.numel() != k:
        raise ValueError("add_layer_norm: r must have x's shape, x contiguous, w and b hold K values")
    x2, r2 = x.view(-1, k), r.reshape(-1, k)
    if r2.stride(1) != 1:
        r2 = r2.contiguous()
    if out_dtype == torch.float16:
        if x.dtype != torch.float32 or y_rows is not None:
            raise TypeError("add_layer_norm: the fp16 result is built for fp32 rows in place")
        y = torch.empty(x2.shape, dtype=torch.float16, device=x.device)
        rc = lib.tk_add_layer_norm_f16(x2.data_ptr(), x2.stride(0), r2.data_ptr(), r2.stride(0), x2.data_ptr(), x2.stride(0),
                                       w.contiguous().data_ptr(), b.contiguous().data_ptr(), float(eps), y.data_ptr(), y.stride(0),
                                       x2.shape[0], k, _stream())  # fmt: skip
        native.check(rc, "tk_add_layer_norm_f16")
        return x, y.view(x.shape)
    y = torch.empty(x2.shape, dtype=torch.bfloat16, device=x.device)
    dt = _F32 if x.dtype == torch.float32 else _BF16
    if y_rows is not None:
        if y_rows.dtype != torch.int32 or y_rows.numel() < x2.shape[0] or not y_rows.is_contiguous() or y_rows.device != x.device:
            raise ValueError("add_layer_norm: y_rows must be a contiguous int32 tensor on x's device with an entry per row")
        rc = lib.tk_add_layer_norm_rows(x2.data_ptr(), x2.stride(0), dt, r2.data_ptr(), r2.stride(0), x2.data_ptr(), x2.stride(0),
                                        w.contiguous().data_ptr(), b.contiguous().data_ptr(), dt, float(eps), y.data_ptr(), y.stride(0),
                                        y_rows.data_ptr(), x2.shape[0], k, _stream())  # fmt: skip
        native.check(rc, "tk_add_layer_norm_rows")
        return x, y.view(x.shape)
    rc = lib.tk_add_layer_norm(x2.data_ptr(), x2.stride(0), dt, r2.data_ptr(), r2.stride(0), x2.data_ptr(), x2.stride(0),
                               w.contiguous().data_ptr(), b.contiguous().data_ptr(), dt, float(eps), y.data_ptr(), y.stride(0),
                               x2.shape[0], k, _stream())  # fmt: skip
    native.check(rc, "tk_add_layer_norm")
    return x, y.view(x.shape)


def rms_norm_rows(x: torch.Tensor, *, norm_w: torch.Tensor | None = None, ada: tuple[torch.Tensor, torch.Tensor] | None = None, eps: float) -> torch.Tensor:
    """RMSNorm of bf16 rows ``x [M, K]`` into a new bf16 tensor: Llama (``norm_w`` bf16 ``[K]``) or
    Gemma / adaptive (``ada = (scale, shift)`` fp32 ``[K]``: ``(x * rstd) * (1 + scale) + shift``).  The
    norm prologue of the fused projections as one launch, for projections that run as a library GEMM."""
    lib = native.lib()
    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.stride(1) != 1:
        raise TypeError("rms_norm_rows: x must be a 2-D bf16 tensor with contiguous rows")
    if (norm_w is None) == (ada is None):
        raise ValueError("rms_norm_rows: exactly one of norm_w and ada")
    m, k = x.shape
    if norm_w is not None and (norm_w.dtype != torch.bfloat16 or norm_w.numel() != k):
        raise TypeError("rms_norm_rows: norm_w must be bf16 [K]")
    if ada is not None and any(t.dtype != torch.float32 or t.numel() != k or not t.is_contiguous() for t in ada):
        raise TypeError("rms_norm_rows: ada scale / shift must be contiguous fp32 [K]")
    y = torch.empty(m, k, dtype=torch.bfloat16, device=x.device)
    rc = lib.tk_rms_norm_rows(
        x.data_ptr(), x.stride(0), norm_w.contiguous().data_ptr() if norm_w is not None else None,
        ada[0].data_ptr() if ada is not None else None, ada[1].data_ptr() if ada is not None else None, float(eps),
        y.data_ptr(), y.stride(0), m, k, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_rms_norm_rows")
    return y


def rope_rows(y: torch.Tensor, rope: RopeTables, rope_pos: torch.Tensor, rope_cols: int, *, rope_bf16: bool = False) -> torch.Tensor:
    """Rotary embedding in place on the first ``rope_cols`` columns of a bf16 projection output
    ``y [M, N]`` (heads of ``2 * rope.half`` columns), int32 positions ``[M]``.  Returns ``y``."""
    lib = native.lib()
    if y.dtype != torch.bfloat16 or y.dim() != 2 or y.stride(1) != 1:
        raise TypeError("rope_rows: y must be a 2-D bf16 tensor with contiguous rows")
    if rope_pos.dtype != torch.int32 or rope_pos.numel() != y.shape[0] or not rope_pos.is_contiguous():
        raise TypeError("rope_rows: positions must be contiguous int32 [M]")
    if rope_cols > y.shape[1]:
        raise ValueError("rope_rows: rope_cols exceeds the row width")
    rc = lib.tk_rope_rows(y.data_ptr(), y.stride(0), rope_pos.data_ptr(), rope.cos.data_ptr(), rope.sin.data_ptr(), rope.positions,
                          int(rope_cols), rope.half, int(rope_bf16), y.shape[0], _stream())  # fmt: skip
    native.check(rc, "tk_rope_rows")
    return y


def prefix_meta(pad: torch.Tensor, att: torch.Tensor | None, rope_positions: int, suffix_len: int = 0, *, want_mask: bool = True):
    """Prefix bookkeeping of one request in one launch: ``pad`` / ``att`` bool ``[P]`` ->
    ``(mask2d uint8 [P, P rounded up to 32] or None, pos32 int32 [P], suf_pos int32 [suffix_len] or None)``:
    the prefill's 2-D visibility ``(cumsum(att)[j] <= cumsum(att)[i]) & pad[i] & pad[j]``, the prefix positions
    ``clamp(cumsum(pad) - 1)`` and the action tokens' positions ``clamp(sum(pad) + s)``."""
    lib = native.lib()
    if pad.dtype != torch.bool or pad.dim() != 1 or not pad.is_contiguous():
        raise TypeError("prefix_meta: pad must be a contiguous 1-D bool tensor")
    if att is not None and (att.dtype != torch.bool or att.shape != pad.shape or not att.is_contiguous()):
        raise TypeError("prefix_meta: att must be a contiguous bool tensor of pad's shape")
    p_len = pad.shape[0]
    p_pad = (p_len + 31) // 32 * 32
    mask2d = torch.empty(p_len, p_pad, dtype=torch.uint8, device=pad.device) if want_mask else None
    pos32 = torch.empty(p_len, dtype=torch.int32, device=pad.device)
    suf = torch.empty(suffix_len, dtype=torch.int32, device=pad.device) if suffix_len > 0 else None
    rc = lib.tk_prefix_meta(pad.data_ptr(), _ptr(att), p_len, p_pad, int(rope_positions), int(suffix_len), _ptr(mask2d), pos32.data_ptr(),
                            _ptr(suf), _stream())  # fmt: skip
    native.check(rc, "tk_prefix_meta")
    return mask2d, pos32, suf


def patchify_images(images, patch: int, scale: float = 1.0, shift: float = 0.0, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Up to four fp32 images ``[1, 3, H, W]`` (or ``[3, H, W]``) -> ``[n, (H/patch) * (W/patch), 3 * patch * patch]``
    rows of ``x * scale + shift`` in the order of ``unfold``: the patch embedding's GEMM input, in bf16 (patch sizes
    that are multiples of 8) or fp32 (any even patch size)."""
    lib = native.lib()
    images = list(images)
    if not 1 <= len(images) <= 4:
        raise ValueError("patchify_images: one to four images")
    h, w = images[0].shape[-2:]
    for img in images:
        if img.dtype != torch.float32 or not img.is_contiguous() or img.numel() != 3 * h * w:
            raise TypeError("patchify_images: every image must be a contiguous fp32 tensor of 3 x H x W values")
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise TypeError("patchify_images: bf16 or fp32 patch rows")
    out = torch.empty(len(images), (h // patch) * (w // patch), 3 * patch * patch, dtype=out_dtype, device=images[0].device)
    ptrs = [img.data_ptr() for img in images] + [None] * (4 - len(images))
    fn = lib.tk_patchify_images if out_dtype == torch.bfloat16 else lib.tk_patchify_images_f32
    rc = fn(*ptrs, len(images), h, w, int(patch), float(scale), float(shift), out.data_ptr(), _stream())
    native.check(rc, "tk_patchify_images")
    return out


def prefix_rows(img, img_scale: float, table, tokens, tok_scale: float, last=None, *, cam_flags=None, tok_flags=None, out_dtype: torch.dtype = torch.float32):
    """The prefix ``[1, P, H]`` of one request in one launch: ``img [cams, per_cam, H]`` -- bf16: times ``img_scale``,
    rounded to bf16 as the tensor product is; fp32: as it is -- then ``table[tokens]`` (bf16 ``[vocab, H]``, ids int64
    ``[n_tok]``) times ``tok_scale``, rounded likewise, then ``last`` fp32 ``[n_last, H]`` (or None) as it is; written
    in fp32 or rounded to bf16 (``out_dtype``).  With ``cam_flags`` (a bool tensor of one element per camera) and
    ``tok_flags`` (bool ``[n_tok]``) also the pad flags ``[1, P]`` of those rows (the closing rows are always valid);
    returns ``(rows, flags or None)``."""
    lib = native.lib()
    bf = torch.bfloat16
    if img.dtype not in (bf, torch.float32) or table.dtype != bf or tokens.dtype != torch.int64 or (last is not None and last.dtype != torch.float32):
        raise TypeError("prefix_rows: img bf16 or fp32, table bf16, tokens int64, last fp32")
    if out_dtype not in (bf, torch.float32):
        raise TypeError("prefix_rows: fp32 or bf16 rows")
    h = table.shape[1]
    if img.dim() != 3 or img.shape[2] != h or not (img.is_contiguous() and table.is_contiguous() and tokens.is_contiguous()):
        raise ValueError("prefix_rows: img [cams, per_cam, H], table [vocab, H], tokens, all contiguous")
    if last is not None and (last.dim() != 2 or last.shape[1] != h or not last.is_contiguous()):
        raise ValueError("prefix_rows: last [n_last, H], contiguous")
    cams, n_img, n_tok, n_last = img.shape[0], img.shape[0] * img.shape[1], tokens.numel(), 0 if last is None else last.shape[0]
    total = n_img + n_tok + n_last
    out = torch.empty(1, total, h, dtype=out_dtype, device=img.device)
    flags, fl = None, [None] * 4
    if cam_flags is not None:
        cam_flags = list(cam_flags)
        if len(cam_flags) != cams or not 1 <= cams <= 4 or tok_flags is None or tok_flags.numel() != n_tok or not tok_flags.is_contiguous():
            raise ValueError("prefix_rows: a flag per camera (one to four) and a contiguous flag per token")
        if any(f.dtype != torch.bool or f.numel() != 1 for f in cam_flags) or tok_flags.dtype != torch.bool:
            raise TypeError("prefix_rows: flags are bool tensors")
        flags = torch.empty(1, total, dtype=torch.bool, device=img.device)
        fl = [f.data_ptr() for f in cam_flags] + [None] * (4 - cams)
    rc = lib.tk_prefix_rows(
        img.data_ptr(), _BF16 if img.dtype == bf else _F32, n_img, float(img_scale), table.data_ptr(), tokens.data_ptr(), n_tok, table.shape[0],
        float(tok_scale), None if last is None else last.data_ptr(), n_last, out.data_ptr(), _BF16 if out_dtype == bf else _F32, h, *fl, cams,
        tok_flags.data_ptr() if flags is not None else None, flags.data_ptr() if flags is not None else None, _stream(),
    )  # fmt: skip
    native.check(rc, "tk_prefix_rows")
    return out, flags


def decode_fp8_table(device: torch.device | str = "cuda") -> torch.Tensor:
    """Values of all 256 e4m3fn codes as the device's conversion instruction decodes them."""
    out = torch.empty(256, dtype=torch.float32, device=device)
    native.check(native.lib().tk_debug_decode_fp8(out.data_ptr(), _stream()), "tk_debug_decode_fp8")
    return out

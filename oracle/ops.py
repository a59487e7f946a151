"""Per-op CPU oracle for the fp8 action-inference path (test infrastructure, not the product).

Each function restates one op of the reference's eager torch path with the same rounding
points (where a bf16 tensor is materialised in the reference, it is materialised here).
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F  # noqa: N812

BF16 = torch.bfloat16


# --------------------------------------------------------------------------- #
# fp8-weight linear and gated FFN
# --------------------------------------------------------------------------- #
def lin_fp8w(x: torch.Tensor, w8: torch.Tensor, scale: torch.Tensor, out_dtype: torch.dtype = BF16) -> torch.Tensor:
    """``bf16((x.float() @ W8.float().T) * scale[None, :])`` -- weight-only fp8 linear.

    The per-output-channel scale multiplies the fp32 accumulator, as every fp8 kernel of the
    reference does (``acc * a_scale * w_scale``: tybok/policies/pi05/models/triton_prefill_mlp.py:89,
    tybok/policies/fastwam/models/fp8_linear.py:70); activations stay bf16 (no ``a_scale``).
    """
    acc = x.float() @ w8.float().t()
    return (acc * scale.float()[None, :]).to(out_dtype)


def lin_fp8w_f64(x: torch.Tensor, w8: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """Same contraction in float64 (summation-order-free yardstick for the tolerance tests)."""
    acc = x.double() @ w8.double().t()
    return acc * scale.double()[None, :]


def act_fn(name: str, x: torch.Tensor) -> torch.Tensor:
    if name == "silu":
        return F.silu(x)
    if name == "gelu_tanh":
        return F.gelu(x, approximate="tanh")
    raise ValueError(name)


def gated_ffn(
    x: torch.Tensor,
    wg8: torch.Tensor,
    sg: torch.Tensor,
    wu8: torch.Tensor,
    su: torch.Tensor,
    wd8: torch.Tensor,
    sd: torch.Tensor,
    act: str = "silu",
) -> torch.Tensor:
    """``down(act(gate(x)) * up(x))`` with a bf16 tensor after every op.

    SwiGLU: tybok/policies/smolvla/models/layers.py:75-76; GeGLU (``gelu_tanh``):
    tybok/policies/pi05/models/layers.py:94-95.  Linears are :func:`lin_fp8w`.
    """
    g = lin_fp8w(x, wg8, sg)
    u = lin_fp8w(x, wu8, su)
    h = act_fn(act, g) * u  # bf16 act output, bf16 product
    return lin_fp8w(h, wd8, sd)


# --------------------------------------------------------------------------- #
# W8A8 tier: per-token activation quantisation, fp8 x fp8 linear, the prefill MLP
# --------------------------------------------------------------------------- #
FP8 = torch.float8_e4m3fn


def quantize_activation_rows(x: torch.Tensor, mode: str = "fp32") -> tuple[torch.Tensor, torch.Tensor]:
    """Per-token e4m3fn quantisation of ``x [M, K]`` -> ``(a8 [M, K] float8_e4m3fn, sa [M] fp32)``.

    ``"fp32"``: ``sa = amax_k|x| / 448`` in fp32 and ``a8 = RNE(x / sa)`` from the fp32 quotient, one
    rounding (tybok/policies/fastwam/models/fp8_linear.py:223-243; the expert path's kernel multiplies by
    ``448 / amax`` instead: tybok/policies/pi05/models/triton_expert_mlp_fp8.py:268-274); an all-zero row
    gives ``sa = 0`` and zero codes.
    ``"bf16"``: the prefill path's torch expression evaluated on bf16 tensors -- the scale and the quotient
    are bf16 values before the fp8 cast (tybok/policies/pi05/models/triton_prefill_mlp.py:30-36,103-114).
    """
    if mode == "bf16":
        s = x.to(BF16).abs().amax(dim=-1, keepdim=True) / 448.0  # a bf16 tensor
        q = torch.where(s > 0, x.to(BF16) / s, torch.zeros((), dtype=BF16))
        return q.to(FP8), s.float().squeeze(-1)
    x32 = x.float()
    amax = x32.abs().amax(dim=-1, keepdim=True)
    sa = amax / 448.0
    q = torch.where(amax > 0, x32 / sa, torch.zeros(()))
    return q.to(FP8), sa.squeeze(-1)


def lin_w8a8(a8: torch.Tensor, sa: torch.Tensor, w8: torch.Tensor, sw: torch.Tensor) -> torch.Tensor:
    """``bf16((a8 @ W8^T) * sa[:, None] * sw[None, :])``: fp8 x fp8 products (exact in fp32), fp32
    accumulation, both scales on the accumulator, one bf16 rounding
    (tybok/policies/pi05/models/triton_prefill_mlp.py:62-91)."""
    acc = a8.float() @ w8.float().t()
    return (acc * sa.float()[:, None] * sw.float()[None, :]).to(BF16)


def gated_ffn_w8a8(x, wg8, sg, wu8, su, wd8, sd, act: str = "gelu_tanh", mode: str = "fp32") -> torch.Tensor:
    """The W8A8 MLP, `make_fp8_mlp_forward` (tybok/policies/pi05/models/triton_prefill_mlp.py:145-166): gate and up
    share the quantised input, ``act(gate) * up`` elementwise in bf16, a second per-token quantisation, down."""
    x8, sx = quantize_activation_rows(x, mode)
    g = lin_w8a8(x8, sx, wg8, sg)
    u = lin_w8a8(x8, sx, wu8, su)
    h = act_fn(act, g) * u
    h8, sh = quantize_activation_rows(h, mode)
    return lin_w8a8(h8, sh, wd8, sd)


# --------------------------------------------------------------------------- #
# norms
# --------------------------------------------------------------------------- #
def rms_norm_llama(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``weight * cast(x32 * rsqrt(mean(x32^2) + eps), x.dtype)``.

    tybok/policies/smolvla/models/layers.py:22-27.  The weight multiply happens after the cast
    back, so an fp32 input with a bf16 weight yields fp32 (type promotion), a bf16 input bf16.
    """
    x32 = x.to(torch.float32)
    var = x32.pow(2).mean(-1, keepdim=True)
    return weight * (x32 * torch.rsqrt(var + eps)).to(x.dtype)


def gemma_rms_norm(
    x: torch.Tensor,
    eps: float,
    weight: torch.Tensor | None = None,
    modulation: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Gemma RMSNorm / AdaRMS: returns ``(normed, gate)``.

    tybok/policies/pi05/models/layers.py:51-84.  ``x * rsqrt(mean(x32^2) + eps)`` keeps ``x``'s
    dtype for the first product only through promotion (``x`` bf16 times an fp32 rsqrt gives
    fp32), then ``* (1 + w)`` (plain) or ``* (1 + scale) + shift`` (adaptive) in fp32, cast to
    ``x.dtype``.  ``modulation`` is ``dense(cond)``: ``[*, 3*dim]`` (scale, shift, gate) or
    ``[*, 2*dim]`` (scale, shift).
    """
    dtype = x.dtype
    dim = x.shape[-1]
    var = torch.mean(torch.square(x.float()), dim=-1, keepdim=True)
    normed = x * torch.rsqrt(var + eps)
    if modulation is None:
        assert weight is not None
        return (normed * (1.0 + weight.float())).to(dtype), None
    if x.dim() == 3 and modulation.dim() == 2:
        modulation = modulation.unsqueeze(1)
    if modulation.shape[-1] == 2 * dim:
        scale, shift = modulation.chunk(2, dim=-1)
        return (normed * (1 + scale.float()) + shift.float()).to(dtype), None
    scale, shift, gate = modulation.chunk(3, dim=-1)
    return (normed * (1 + scale.float()) + shift.float()).to(dtype), gate.to(dtype)


# --------------------------------------------------------------------------- #
# rotary embeddings
# --------------------------------------------------------------------------- #
def rope_half_split(x: torch.Tensor, positions: torch.Tensor, base: float = 10_000.0) -> torch.Tensor:
    """SmolVLA RoPE on ``x [B, L, H, D]`` with integer ``positions [B, L]``.

    tybok/policies/smolvla/models/rope.py:51-73 (+ table :38-48): angle = ``pos / base**(2i/D)``
    in fp32, pairs ``(i, i + D/2)``, result cast back to ``x.dtype``.
    """
    d_half = x.shape[-1] // 2
    exponents = (2.0 / (d_half * 2)) * torch.arange(d_half, dtype=torch.float32)
    timescale = base**exponents
    radians = positions.to(torch.float32)[..., None] / timescale  # [B, L, d_half]
    sin = torch.sin(radians)[..., None, :]
    cos = torch.cos(radians)[..., None, :]
    x32 = x.to(torch.float32)
    a, b = x32[..., :d_half], x32[..., d_half:]
    out = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
    return out.to(x.dtype)


def gemma_rope_cos_sin(
    head_dim: int, position_ids: torch.Tensor, dtype: torch.dtype, theta: float = 10_000.0
) -> tuple[torch.Tensor, torch.Tensor]:
    """pi0.5 rotary tables ``(cos, sin) [B, L, D]`` in ``dtype``.

    tybok/policies/pi05/models/rope.py:19-41: inverse frequencies are rounded to bf16 first, the
    angle is an fp32 product, ``emb = cat(freqs, freqs)``, cos/sin cast to the activation dtype.
    """
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).to(torch.float32) / head_dim))
    inv = inv.to(BF16).to(torch.float32)
    freqs = position_ids.to(torch.float32)[..., None] * inv[None, None, :]
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def gemma_apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate ``x [B, H, L, D]`` with ``cos/sin [B, L, D]`` in ``x``'s dtype (bf16 arithmetic).

    tybok/policies/pi05/models/rope.py:44-75: ``x*cos + rotate_half(x)*sin`` with
    ``rotate_half(x) = cat(-x[D/2:], x[:D/2])``.
    """
    half = x.shape[-1] // 2
    rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return x * cos.unsqueeze(1) + rot * sin.unsqueeze(1)


# --------------------------------------------------------------------------- #
# masks, time embedding
# --------------------------------------------------------------------------- #
def make_att_2d_masks(pad_masks: torch.Tensor, att_masks: torch.Tensor) -> torch.Tensor:
    """``mask[b, i, j] = cumsum(att)[j] <= cumsum(att)[i]  and  pad[i] and pad[j]``.

    tybok/policies/smolvla/models/flow_matching.py:45-55 (same in pi05 :144-149).
    """
    c = torch.cumsum(att_masks, dim=1)
    allowed = c[:, None, :] <= c[:, :, None]
    valid = pad_masks[:, None, :].bool() & pad_masks[:, :, None].bool()
    return allowed & valid


def sinusoidal_time_embedding(time: torch.Tensor, dim: int, min_period: float, max_period: float) -> torch.Tensor:
    """``cat(sin, cos)(2*pi*t / period_i)`` in float64, ``period`` log-spaced over ``dim/2`` points.

    tybok/policies/smolvla/models/flow_matching.py:27-42 (identical in pi05 :119-141).
    """
    frac = torch.linspace(0.0, 1.0, dim // 2, dtype=torch.float64)
    period = min_period * (max_period / min_period) ** frac
    ang = (1.0 / period * 2 * math.pi)[None, :] * time.to(torch.float64)[:, None]
    return torch.cat([torch.sin(ang), torch.cos(ang)], dim=1)


# --------------------------------------------------------------------------- #
# attention
# --------------------------------------------------------------------------- #
def eager_attention(mask: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """SmolVLA GQA attention. ``q [B, Lq, H, D]``, ``k/v [B, Lk, G, D]``, bool ``mask [B, Lq, Lk]``.

    tybok/policies/smolvla/models/attention.py:136-187: K/V repeated per group (q head ``h`` reads
    kv head ``h // (H//G)``), q and k upcast to fp32, scores ``* D**-0.5``, masked entries set to
    ``finfo(float32).min``, fp32 softmax, probabilities cast to ``v.dtype``, ``P @ V`` in that
    dtype; output ``[B, Lq, H*D]``.
    """
    b, lq, h, d = q.shape
    g = k.shape[2]
    rep = h // g
    k_full = k[:, :, :, None, :].expand(b, k.shape[1], g, rep, d).reshape(b, k.shape[1], h, d)
    v_full = v[:, :, :, None, :].expand(b, v.shape[1], g, rep, d).reshape(b, v.shape[1], h, d)
    qf = q.to(torch.float32).transpose(1, 2)
    kf = k_full.to(torch.float32).transpose(1, 2)
    scores = torch.matmul(qf, kf.transpose(2, 3)) * d**-0.5
    scores = torch.where(mask[:, None, :, :], scores, torch.finfo(torch.float32).min)
    probs = F.softmax(scores, dim=-1).to(v_full.dtype)
    out = torch.matmul(probs, v_full.permute(0, 2, 1, 3))
    return out.permute(0, 2, 1, 3).reshape(b, lq, h * d)


def gemma_attention_core(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, add_mask: torch.Tensor, scaling: float
) -> torch.Tensor:
    """pi0.5 GQA attention core. ``q [B, H, Lq, D]``, ``k/v [B, G, Lk, D]``, additive ``add_mask [B,1,Lq,Lk]``.

    tybok/policies/pi05/models/layers.py:179-191: K/V repeated, logits ``q @ k^T`` in the
    activation dtype (bf16) times ``scaling``, plus the fp32 mask, softmax in fp32 cast back to
    the activation dtype, ``P @ V``; output ``[B, Lq, H*D]`` (before ``o_proj``).
    """
    b, h, lq, d = q.shape
    g = k.shape[1]
    rep = h // g
    if rep > 1:
        k = k[:, :, None].expand(b, g, rep, k.shape[2], d).reshape(b, h, k.shape[2], d)
        v = v[:, :, None].expand(b, g, rep, v.shape[2], d).reshape(b, h, v.shape[2], d)
    logits = torch.matmul(q, k.transpose(2, 3)) * scaling
    logits = logits + add_mask
    probs = F.softmax(logits, dim=-1, dtype=torch.float32).to(q.dtype)
    out = torch.matmul(probs, v)
    return out.transpose(1, 2).contiguous().reshape(b, lq, h * d)


MASK_NONE, MASK_BIDIR, MASK_CAUSAL = 0, 1, 2
OPENPI_MASK_VALUE = -2.3819763e38  # tybok/policies/pi05/models/flow_matching.py:25


def suffix_mask(prefix_pad: torch.Tensor, n_query: int, n_suffix: int, mode: int) -> torch.Tensor:
    """Bool ``[1, n_query, P + n_suffix]``: prefix column ``j`` visible iff ``prefix_pad[j]``;
    suffix column ``j`` visible to row ``i`` always (BIDIR) or iff ``j <= i`` (CAUSAL).

    This is what ``denoise_step`` builds from ``make_att_2d_masks`` for an all-valid suffix:
    smolvla ``att=[1]*50`` gives CAUSAL (tybok/policies/smolvla/models/flow_matching.py:296-336),
    pi05 ``att=[1]+[0]*49`` gives BIDIR (tybok/policies/pi05/models/flow_matching.py:492-531).
    """
    p = prefix_pad.shape[-1]
    pre = prefix_pad.reshape(1, 1, p).bool().expand(1, n_query, p)
    if n_suffix == 0 or mode == MASK_NONE:
        return pre.clone()
    if mode == MASK_BIDIR:
        suf = torch.ones(1, n_query, n_suffix, dtype=torch.bool)
    else:
        i = torch.arange(n_query)[:, None]
        j = torch.arange(n_suffix)[None, :]
        suf = (j <= i)[None]
    return torch.cat([pre, suf], dim=2)


def expert_attention(
    q: torch.Tensor,
    k_pre: torch.Tensor,
    v_pre: torch.Tensor,
    k_suf: torch.Tensor | None,
    v_suf: torch.Tensor | None,
    prefix_pad: torch.Tensor,
    mode: int,
    bf16_logits: bool = False,
) -> torch.Tensor:
    """Action-expert attention over ``[prefix; suffix]`` for one request (batch 1).

    ``q [M, H, D]``; ``k_pre/v_pre [P, G, D]`` (bf16 or fp32); ``k_suf/v_suf [S, G, D]`` or None;
    ``prefix_pad [P]`` bool.  ``bf16_logits=False`` is :func:`eager_attention` (SmolVLA),
    ``True`` is :func:`gemma_attention_core` (pi0.5).  Returns ``[M, H*D]``.
    """
    m, h, d = q.shape
    n_suf = 0 if k_suf is None else k_suf.shape[0]
    k = k_pre if k_suf is None else torch.cat([k_pre, k_suf], dim=0)
    v = v_pre if v_suf is None else torch.cat([v_pre, v_suf], dim=0)
    mask = suffix_mask(prefix_pad, m, n_suf, mode)
    if not bf16_logits:
        return eager_attention(mask, q[None], k[None], v[None])[0]
    add = torch.where(mask[:, None], 0.0, OPENPI_MASK_VALUE)
    out = gemma_attention_core(
        q[None].transpose(1, 2), k[None].transpose(1, 2), v[None].transpose(1, 2), add, d**-0.5
    )
    return out[0]


def attention_f64(q, k, v, mask) -> torch.Tensor:
    """Brute-force float64 softmax attention (``q [M,H,D]``, ``k/v [L,G,D]``, bool ``mask [M,L]``)."""
    m, h, d = q.shape
    g = k.shape[1]
    out = torch.zeros(m, h, d, dtype=torch.float64)
    for hh in range(h):
        kk = k[:, hh // (h // g)].double()
        vv = v[:, hh // (h // g)].double()
        s = (q[:, hh].double() @ kk.t()) * d**-0.5
        s = torch.where(mask, s, torch.full_like(s, float(torch.finfo(torch.float32).min)))
        p = torch.softmax(s, dim=-1)
        out[:, hh] = p @ vv
    return out.reshape(m, h * d)

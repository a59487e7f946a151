"""pi0.5-shaped action inference on the CPU -- oracle (test infrastructure, not the product).

Functional restatement of the reference's eager torch path over a state dict keyed by the
reference's own parameter names.  Follows (file:line in /root/reference):
  tybok/policies/pi05/models/flow_matching.py:405-462 (embed_prefix), :464-502 (embed_suffix),
    :376-381 (AdaRMS condition), :505-556 (denoise_step), :193-254 (Euler), :761-838 (sample_actions)
  tybok/policies/pi05/models/gemma.py:61-125 (decoder stack)
  tybok/policies/pi05/models/layers.py:34-84 (norms), :87-95 (GeGLU), :166-191 (attention),
    :268-308 (layer), :27-31 (gated residual)
  tybok/policies/pi05/models/paligemma_with_expert.py:137-161 (image / language embedding)
  tybok/policies/pi05/models/vision.py (SigLIP tower, fp32)

dtype rules: vision tower, projector, norms' weights, AdaRMS ``dense`` and the action/time
projections are fp32; decoder linears and the embedding table are bf16; the prefix embedding is
fp32 after ``torch.cat`` and cast to bf16 at the decoder entry; logits are bf16, softmax fp32.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F  # noqa: N812

from . import ops
from .smolvla import Weights

BF16 = torch.bfloat16
PWE = "paligemma_with_expert."
VIS = PWE + "paligemma.model.vision_tower.vision_model."
PROJ = PWE + "paligemma.model.multi_modal_projector.linear"
VLM = PWE + "paligemma.model.language_model."
EXP = PWE + "gemma_expert.model."
EPS = 1e-6


@dataclass
class PI05Shape:
    """Hyper-parameters (defaults = tybok/policies/pi05/config.py:15-80)."""

    vlm_width: int = 2048
    vlm_mlp: int = 16384
    exp_width: int = 1024
    exp_mlp: int = 4096
    depth: int = 18
    heads: int = 8
    kv_heads: int = 1
    head_dim: int = 256
    vis_hidden: int = 1152
    vis_heads: int = 16
    vis_layers: int = 27
    vis_mlp: int = 4304
    patch: int = 14
    image: int = 224
    chunk: int = 50
    max_action_dim: int = 32
    num_steps: int = 10
    min_period: float = 4e-3
    max_period: float = 4.0
    # drift tiers of the vision tower (tybok/policies/pi05/engine.py:196-230):
    #   vit_mlp_dtype: fc1 / gelu / fc2 run in that dtype, cast at the boundary (vision.py:79-87); pinned by a
    #                  fixture written from the reference's own tower after set_mlp_dtype
    #                  (tests/golden/pi05_small_vit_tiers.npz);
    vit_mlp_dtype: torch.dtype | None = None
    #   vit_fused: the reference's fused tower (``--tl-fused-vit``), restated from its kernels' source
    #                  (tybok/policies/pi05/models/triton_vision.py): LayerNorm in fp32; q|k|v from fp16 operands with
    #                  fp32 accumulation, kept as fp16; fp32 logits and softmax, probabilities rounded to fp16 for P.V,
    #                  bf16 attention output; out_proj, fc1, fc2 and the projector from bf16 operands with fp32
    #                  accumulation and fp32 results; tanh-GELU on the fp32 pre-activation, rounded to bf16 for fc2;
    #                  residuals in fp32.  The fp16 half (LayerNorm + q|k|v + attention) is pinned by a fixture written
    #                  from those kernels through Triton's CPU interpreter (tests/golden/pi05_small_vit_fused.npz).
    #                  The bf16 kernels (out_proj, MLP, projector) are restated from source only -- that interpreter
    #                  multiplies bf16 operands as raw integers and has no libdevice tanh -- PARITY UNPINNED for them;
    #                  what they compute (a 16-bit-operand linear with an fp32 accumulator, the tanh-GELU) is pinned
    #                  as arithmetic by the closed-form tests of oracle/ops.py.
    vit_fused: bool = False
    # W8A8 tier of the VLM MLP (tybok/policies/pi05/models/triton_prefill_mlp.py:145-166): activations quantised
    # per token as well; only with the VLM MLP's weights in fp8 (``fp8_linear_names(..., llm_mlp=True, ...)``)
    llm_w8a8: bool = False


def fp8_linear_names(shape: PI05Shape, llm_mlp: bool, expert_mlp: bool) -> frozenset:
    names = []
    for i in range(shape.depth):
        for proj in ("gate_proj", "up_proj", "down_proj"):
            if llm_mlp:
                names.append(f"{VLM}layers.{i}.mlp.{proj}")
            if expert_mlp:
                names.append(f"{EXP}layers.{i}.mlp.{proj}")
    return frozenset(names)


def _lin16(t: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, dt: torch.dtype) -> torch.Tensor:
    """``t . weight^T + bias`` with every operand rounded to the 16-bit type ``dt``, fp32 products and accumulation,
    fp32 result -- what a 16-bit matrix instruction with an fp32 accumulator computes, up to summation order."""
    return t.to(dt).float() @ weight.to(dt).float().t() + bias.to(dt).float()


def vit_fused_qkv_attention(w: Weights, shape: PI05Shape, layer: int, x: torch.Tensor):
    """The fp16 half of an attention block of the reference's fused tower: ``x [B, L, C]`` fp32 ->
    ``(q, k, v)`` fp32 ``[B, H, L, hd]`` as the projection kernel stores them and the attention output bf16
    ``[B, H, L, hd]`` (`_fused_qkv`, tybok/policies/pi05/models/vision.py:133-156; `_vision_qkv_kernel`,
    `_vision_attn_kernel`, triton_vision.py:38-110, 248-326): LayerNorm in fp32, the normalised row and the
    weights as fp16, fp32 accumulation; q, k, v rounded to fp16 by the attention kernel; fp32 logits and softmax;
    exp(s - max) rounded to fp16 for P.V; the normalised result rounded to bf16.  The kernel walks the keys in
    blocks with a running maximum; this is the same computation with all keys in one block."""
    p = f"{VIS}encoder.layers.{layer}."
    b, hd = x.shape[0], shape.vis_hidden // shape.vis_heads
    h = F.layer_norm(x, (shape.vis_hidden,), w[p + "layer_norm1.weight"], w[p + "layer_norm1.bias"], EPS)
    q, k, v = (
        _lin16(h, w[p + f"self_attn.{n}_proj.weight"], w[p + f"self_attn.{n}_proj.bias"], torch.float16)
        .view(b, -1, shape.vis_heads, hd).transpose(1, 2)
        for n in "qkv"
    )  # fmt: skip
    q16, k16, v16 = (t.to(torch.float16).float() for t in (q, k, v))
    s = torch.matmul(q16, k16.transpose(2, 3)) * hd**-0.5
    e = torch.exp(s - s.amax(dim=-1, keepdim=True))
    o = torch.matmul(e.to(torch.float16).float(), v16) / e.sum(dim=-1, keepdim=True)
    return (q, k, v), o.to(BF16)


def vit_fused_attn_block(w: Weights, shape: PI05Shape, layer: int, x: torch.Tensor) -> torch.Tensor:
    """One attention block of the fused tower, fp32 in and out (`SiglipEncoderLayer._attn_block`,
    tybok/policies/pi05/models/vision.py:120-131): the fp16 half above, then out_proj from bf16 operands with
    fp32 accumulation, bias and the fp32 residual added before the one fp32 store (`_vision_attn_out_kernel`,
    triton_vision.py:437-497)."""
    p = f"{VIS}encoder.layers.{layer}."
    _, a = vit_fused_qkv_attention(w, shape, layer, x)
    a = a.transpose(1, 2).reshape(x.shape[0], -1, shape.vis_hidden)
    return x + _lin16(a, w[p + "self_attn.out_proj.weight"], w[p + "self_attn.out_proj.bias"], BF16)


def vit_fused_mlp_block(w: Weights, shape: PI05Shape, layer: int, x: torch.Tensor) -> torch.Tensor:
    """One MLP block of the fused tower (`triton_vision_mlp`, triton_vision.py:113-245, 550-622): bf16 operands, the
    tanh-GELU on the fp32 pre-activation, the activation rounded to bf16 for fc2, fp32 residual."""
    p = f"{VIS}encoder.layers.{layer}."
    h = F.layer_norm(x, (shape.vis_hidden,), w[p + "layer_norm2.weight"], w[p + "layer_norm2.bias"], EPS)
    act = F.gelu(_lin16(h, w[p + "mlp.fc1.weight"], w[p + "mlp.fc1.bias"], BF16), approximate="tanh")
    return x + _lin16(act, w[p + "mlp.fc2.weight"], w[p + "mlp.fc2.bias"], BF16)


def vit_fused_projector(w: Weights, shape: PI05Shape, x: torch.Tensor) -> torch.Tensor:
    """post_layernorm + projector of the fused tower (`_vision_projector_kernel`, triton_vision.py:625-702): the
    normalised row rounded to bf16, bf16 weights, fp32 result."""
    h = F.layer_norm(x, (shape.vis_hidden,), w[VIS + "post_layernorm.weight"], w[VIS + "post_layernorm.bias"], EPS)
    return _lin16(h, w[PROJ + ".weight"], w[PROJ + ".bias"], BF16)


def embed_image(w: Weights, shape: PI05Shape, image: torch.Tensor) -> torch.Tensor:
    """``[1, 3, 224, 224]`` fp32 in [-1, 1] -> ``[1, 256, vlm_width]`` fp32 (vision.py + projector)."""
    x = F.conv2d(image.float(), w[VIS + "embeddings.patch_embedding.weight"], w[VIS + "embeddings.patch_embedding.bias"], stride=shape.patch)
    b = x.shape[0]
    x = x.flatten(2).transpose(1, 2)
    x = x + w[VIS + "embeddings.position_embedding.weight"][None]
    hd = shape.vis_hidden // shape.vis_heads
    mdt = shape.vit_mlp_dtype

    def lowp(name, t, dt):  # Linear with weights and bias converted to dt (vision.py:223-235)
        return F.linear(t.to(dt), w[name + ".weight"].to(dt), w[name + ".bias"].to(dt))

    if shape.vit_fused:
        for i in range(shape.vis_layers):
            x = vit_fused_mlp_block(w, shape, i, vit_fused_attn_block(w, shape, i, x))
        return vit_fused_projector(w, shape, x)
    for i in range(shape.vis_layers):
        p = f"{VIS}encoder.layers.{i}."
        h = F.layer_norm(x, (shape.vis_hidden,), w[p + "layer_norm1.weight"], w[p + "layer_norm1.bias"], EPS)
        q = w.linear(p + "self_attn.q_proj", h).view(b, -1, shape.vis_heads, hd).transpose(1, 2)
        k = w.linear(p + "self_attn.k_proj", h).view(b, -1, shape.vis_heads, hd).transpose(1, 2)
        v = w.linear(p + "self_attn.v_proj", h).view(b, -1, shape.vis_heads, hd).transpose(1, 2)
        a = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=0.0, scale=hd**-0.5, is_causal=False)
        a = a.transpose(1, 2).contiguous().reshape(b, -1, shape.vis_hidden)
        x = x + w.linear(p + "self_attn.out_proj", a)
        h = F.layer_norm(x, (shape.vis_hidden,), w[p + "layer_norm2.weight"], w[p + "layer_norm2.bias"], EPS)
        if mdt is not None:
            x = x + lowp(p + "mlp.fc2", F.gelu(lowp(p + "mlp.fc1", h, mdt), approximate="tanh"), mdt).float()
        else:
            x = x + w.linear(p + "mlp.fc2", F.gelu(w.linear(p + "mlp.fc1", h), approximate="tanh"))
    x = F.layer_norm(x, (shape.vis_hidden,), w[VIS + "post_layernorm.weight"], w[VIS + "post_layernorm.bias"], EPS)
    return w.linear(PROJ, x)


def embed_prefix(w: Weights, shape: PI05Shape, images, img_masks, tokens, masks):
    """-> ``(embs fp32 [1,P,W], pad_masks [1,P], att_masks [1,P] all False)``."""
    embs, pads = [], []
    for img, m in zip(images, img_masks):
        e = embed_image(w, shape, img)
        embs.append(e)
        pads.append(m[:, None].expand(e.shape[0], e.shape[1]))
    lang = F.embedding(tokens, w[VLM + "embed_tokens.weight"])
    lang = lang * torch.tensor(shape.vlm_width**0.5, dtype=BF16).to(lang.dtype)  # bf16-rounded sqrt(width)
    embs.append(lang)
    pads.append(masks)
    embs = torch.cat(embs, dim=1)
    pads = torch.cat(pads, dim=1)
    att = torch.zeros(pads.shape, dtype=torch.bool)
    return embs, pads, att


def _attention(w: Weights, shape: PI05Shape, prefix: str, h, add_mask, cos, sin, prefix_kv):
    b, length = h.shape[0], h.shape[1]
    q = w.linear(prefix + "q_proj", h).view(b, length, -1, shape.head_dim).transpose(1, 2)
    k = w.linear(prefix + "k_proj", h).view(b, length, -1, shape.head_dim).transpose(1, 2)
    v = w.linear(prefix + "v_proj", h).view(b, length, -1, shape.head_dim).transpose(1, 2)
    q = ops.gemma_apply_rope(q, cos, sin)
    k = ops.gemma_apply_rope(k, cos, sin)
    if prefix_kv is not None:
        k = torch.cat([prefix_kv[0], k], dim=2)
        v = torch.cat([prefix_kv[1], v], dim=2)
    out = ops.gemma_attention_core(q, k, v, add_mask, shape.head_dim**-0.5)
    return w.linear(prefix + "o_proj", out), k, v


def _mlp(w: Weights, prefix: str, x):
    return w.linear(prefix + "down_proj", F.gelu(w.linear(prefix + "gate_proj", x), approximate="tanh") * w.linear(prefix + "up_proj", x))


def _mlp_w8a8(w: Weights, prefix: str, x):
    """The W8A8 forward of one GeGLU MLP: both operands of every product in e4m3fn."""
    q = [w.quantised(prefix + n) for n in ("gate_proj", "up_proj", "down_proj")]
    # activation quantisation as `quantize_activation` computes it: scale and quotient are bf16 values
    # (tybok/policies/pi05/models/triton_prefill_mlp.py:26-59,103-114)
    y = ops.gated_ffn_w8a8(x.reshape(-1, x.shape[-1]), *q[0], *q[1], *q[2], "gelu_tanh", mode="bf16")
    return y.reshape(*x.shape[:-1], y.shape[-1])


def prefill(w: Weights, shape: PI05Shape, embs, pad_masks, att_masks):
    """VLM prefill -> per-layer post-RoPE ``(K, V)`` bf16 ``[1, G, P, D]``."""
    mask = ops.make_att_2d_masks(pad_masks, att_masks)
    add = torch.where(mask[:, None], 0.0, ops.OPENPI_MASK_VALUE)
    pos = torch.cumsum(pad_masks, dim=1) - 1
    hidden = embs.to(w.act_dtype)
    cos, sin = ops.gemma_rope_cos_sin(shape.head_dim, pos, hidden.dtype)
    kv = []
    for i in range(shape.depth):
        p = f"{VLM}layers.{i}."
        h, _ = ops.gemma_rms_norm(hidden, EPS, weight=w[p + "input_layernorm.weight"])
        a, k, v = _attention(w, shape, p + "self_attn.", h, add, cos, sin, None)
        kv.append((k, v))
        hidden = hidden + a
        h, _ = ops.gemma_rms_norm(hidden, EPS, weight=w[p + "post_attention_layernorm.weight"])
        hidden = hidden + (_mlp_w8a8(w, p + "mlp.", h) if shape.llm_w8a8 else _mlp(w, p + "mlp.", h))
    return kv


def adarms_cond(w: Weights, shape: PI05Shape, time: float) -> torch.Tensor:
    t = torch.tensor(time, dtype=torch.float32).expand(1)
    te = ops.sinusoidal_time_embedding(t, shape.exp_width, shape.min_period, shape.max_period).to(torch.float32)
    c = F.silu(w.linear("time_mlp_in", te))
    return F.silu(w.linear("time_mlp_out", c))


def denoise_step(w: Weights, shape: PI05Shape, prefix_pad, kv, x_t, time: float):
    """One velocity evaluation fp32 ``[1, chunk, max_action_dim]`` (flow_matching.py:505-556)."""
    cond = adarms_cond(w, shape, time)
    hidden = w.linear("action_in_proj", x_t).to(w.act_dtype)
    s = hidden.shape[1]
    mask = ops.suffix_mask(prefix_pad[0], s, s, ops.MASK_BIDIR)
    add = torch.where(mask[:, None], 0.0, ops.OPENPI_MASK_VALUE)
    pos = prefix_pad.sum(dim=-1)[:, None] + torch.arange(s)[None, :]
    cos, sin = ops.gemma_rope_cos_sin(shape.head_dim, pos, hidden.dtype)
    for i in range(shape.depth):
        p = f"{EXP}layers.{i}."
        h, gate = ops.gemma_rms_norm(hidden, EPS, modulation=w.linear(p + "input_layernorm.dense", cond))
        a, _, _ = _attention(w, shape, p + "self_attn.", h, add, cos, sin, kv[i])
        hidden = hidden + a * gate
        h, gate = ops.gemma_rms_norm(hidden, EPS, modulation=w.linear(p + "post_attention_layernorm.dense", cond))
        hidden = hidden + _mlp(w, p + "mlp.", h) * gate
    out, _ = ops.gemma_rms_norm(hidden, EPS, modulation=w.linear(EXP + "norm.dense", cond))
    return w.linear("action_out_proj", out.to(torch.float32))


def sample_actions(w: Weights, shape: PI05Shape, images, img_masks, tokens, masks, noise, trace: dict | None = None):
    embs, pads, att = embed_prefix(w, shape, images, img_masks, tokens, masks)
    kv = prefill(w, shape, embs, pads, att)
    if trace is not None:
        trace["prefix_embs"] = embs
        trace["kv"] = kv
        trace["pad_masks"] = pads
    dt = -1.0 / shape.num_steps
    x_t = noise
    for step in range(shape.num_steps):
        v_t = denoise_step(w, shape, pads, kv, x_t, 1.0 + step * dt)
        if trace is not None and step == 0:
            trace["v0"] = v_t
        x_t = x_t + dt * v_t
    return x_t

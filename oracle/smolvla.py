"""SmolVLA-shaped action inference on the CPU -- oracle (test infrastructure, not the product).

Functional restatement of the reference's eager torch path over a state dict keyed by the
reference's own parameter names (``vlm_with_expert.lm_expert.layers.3.mlp.gate_proj.weight`` ...),
so the same tensors can be loaded into the reference modules to write golden vectors.

Follows (file:line in /root/reference):
  tybok/policies/smolvla/models/flow_matching.py:160-257 (embed_prefix), :259-311 (embed_suffix),
    :316-350 (denoise_step), :406-451 (sample_actions), :553-578 (expert prefix KV), :580-644 (Euler)
  tybok/policies/smolvla/models/vlm_with_expert.py:124-231 (self layer), :233-321 (cross layer),
    :323-410 (residual/MLP plumbing), :470-511 (layer loop + final norm)
  tybok/policies/smolvla/models/vision.py (SigLIP tower + pixel-shuffle connector)
  tybok/policies/smolvla/models/policy.py:117-170 (prepare_images / prepare_state)

dtype rules that matter for parity: everything is bf16 except state/action/time projections and
the cross-layer expert k/v projections (fp32); the prefix embedding is fp32 after ``torch.cat``
and is downcast by the first in-place residual add; the suffix embedding is fp32 likewise.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch
import torch.nn.functional as F  # noqa: N812

from . import fp8 as ofp8
from . import ops

BF16 = torch.bfloat16


@dataclass
class SmolVLAShape:
    """Hyper-parameters (defaults = tybok/policies/smolvla/config.py:21-168)."""

    hidden: int = 960
    heads: int = 15
    kv_heads: int = 5
    head_dim: int = 64
    mlp: int = 2560
    num_vlm_layers: int = 16
    vocab: int = 49280
    rms_eps: float = 1e-5
    expert_width_multiplier: float = 0.75
    self_attn_every_n_layers: int = 2
    vis_hidden: int = 768
    vis_mlp: int = 3072
    vis_layers: int = 12
    vis_heads: int = 12
    image_size: int = 512
    patch: int = 16
    ln_eps: float = 1e-6
    scale_factor: int = 4
    chunk: int = 50
    max_action_dim: int = 32
    max_state_dim: int = 32
    num_steps: int = 10
    min_period: float = 4e-3
    max_period: float = 4.0
    tok_len: int = 48

    @property
    def expert_hidden(self) -> int:
        return int(self.hidden * self.expert_width_multiplier)

    @property
    def expert_mlp(self) -> int:
        # tybok/policies/smolvla/models/vlm_with_expert.py:536-540
        h = int(2 * self.expert_hidden / 3)
        h = int(4 * h)
        return 256 * ((h + 255) // 256)

    @property
    def image_tokens(self) -> int:
        return (self.image_size // self.patch) ** 2 // self.scale_factor**2

    def is_cross(self, layer: int) -> bool:
        return not (self.self_attn_every_n_layers > 0 and layer % self.self_attn_every_n_layers == 0)


@dataclass
class Weights:
    """State dict + which linears run as fp8-weight linears (quantised lazily, cached)."""

    sd: dict
    fp8_names: frozenset = frozenset()
    _q: dict = field(default_factory=dict)
    # bf16 = the reference's dtypes.  float32 = the same weight VALUES (bf16-rounded, fp8 codes) with every
    # activation kept in fp32: the yardstick that tells rounding noise of a bf16 execution order from error.
    act_dtype: torch.dtype = BF16
    # not None: every linear sums its products in another order (the K dimension of activations and weights
    # permuted alike, seeded) -- the same arithmetic and rounding points, mathematically the same result; what
    # differs between two such runs is what any two executions of the reference's bf16 arithmetic may differ by
    k_order_seed: int | None = None

    def __post_init__(self):
        if self.act_dtype != BF16:
            self.sd_quant = self.sd  # quantisation starts from the stored (bf16) weights in either mode
            self.sd = {k: (v.to(self.act_dtype) if v.is_floating_point() else v) for k, v in self.sd.items()}
        else:
            self.sd_quant = self.sd

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.sd[name]

    def quantised(self, prefix: str) -> tuple[torch.Tensor, torch.Tensor]:
        """``(W8, scale)`` of the linear named ``prefix`` (quantised once from the stored weights)."""
        q = self._q.get(prefix)
        if q is None:
            q = ofp8.quantize_weight_rows(self.sd_quant[prefix + ".weight"])
            self._q[prefix] = q
        return q

    def linear(self, prefix: str, x: torch.Tensor) -> torch.Tensor:
        """``nn.Linear`` named ``prefix`` applied to ``x`` (bias if the state dict has one)."""
        w = self.sd[prefix + ".weight"]
        b = self.sd.get(prefix + ".bias")
        perm = None
        if self.k_order_seed is not None:
            perm = torch.randperm(w.shape[1], generator=torch.Generator().manual_seed(self.k_order_seed + w.shape[1]))
            x = x[..., perm]
        if prefix in self.fp8_names:
            q = self.quantised(prefix)
            w8 = q[0] if perm is None else q[0][:, perm]
            y = ops.lin_fp8w(x.reshape(-1, x.shape[-1]), w8, q[1], self.act_dtype).reshape(*x.shape[:-1], w.shape[0])
            return y if b is None else y + b
        return F.linear(x, w if perm is None else w[:, perm], b)


def fp8_linear_names(shape: SmolVLAShape, llm_mlp: bool, expert_mlp: bool) -> frozenset:
    names = []
    for i in range(shape.num_vlm_layers):
        for proj in ("gate_proj", "up_proj", "down_proj"):
            if llm_mlp:
                names.append(f"vlm_with_expert.vlm.model.text_model.layers.{i}.mlp.{proj}")
            if expert_mlp:
                names.append(f"vlm_with_expert.lm_expert.layers.{i}.mlp.{proj}")
    return frozenset(names)


# --------------------------------------------------------------------------- #
# vision tower + connector (plain torch; not a kernel target)
# --------------------------------------------------------------------------- #
VIS = "vlm_with_expert.vlm.model.vision_model."
TXT = "vlm_with_expert.vlm.model.text_model."
EXP = "vlm_with_expert.lm_expert."


def _vision_position_ids(shape: SmolVLAShape, n_h: int, n_w: int) -> torch.Tensor:
    """Bucketised position ids of a fully valid image (tybok/policies/smolvla/models/vision.py:51-73)."""
    side = shape.image_size // shape.patch
    boundaries = torch.arange(1 / side, 1.0, 1 / side)
    frac_h = (torch.arange(n_h, dtype=BF16) / n_h) * (1 - 1e-6)
    frac_w = (torch.arange(n_w, dtype=BF16) / n_w) * (1 - 1e-6)
    bh = torch.bucketize(frac_h, boundaries, right=True)
    bw = torch.bucketize(frac_w, boundaries, right=True)
    return (bh[:, None] * side + bw[None, :]).reshape(-1)


def embed_image(w: Weights, shape: SmolVLAShape, image: torch.Tensor) -> torch.Tensor:
    """``[1, 3, H, W]`` in [-1, 1] -> ``[1, 64, hidden]`` bf16 (vision.py:197-257)."""
    x = image.to(w.act_dtype)
    x = F.conv2d(x, w[VIS + "embeddings.patch_embedding.weight"], w[VIS + "embeddings.patch_embedding.bias"], stride=shape.patch)
    b = x.shape[0]
    n_h, n_w = x.shape[2], x.shape[3]
    x = x.flatten(2).transpose(1, 2)
    pos = _vision_position_ids(shape, n_h, n_w)
    x = x + w[VIS + "embeddings.position_embedding.weight"][pos][None]
    hd = shape.vis_hidden // shape.vis_heads
    mask = torch.zeros(b, 1, 1, x.shape[1], dtype=x.dtype)  # all patches valid -> additive zeros
    for i in range(shape.vis_layers):
        p = f"{VIS}encoder.layers.{i}."
        h = F.layer_norm(x, (shape.vis_hidden,), w[p + "layer_norm1.weight"], w[p + "layer_norm1.bias"], shape.ln_eps)
        q = w.linear(p + "self_attn.q_proj", h).view(b, -1, shape.vis_heads, hd).transpose(1, 2)
        k = w.linear(p + "self_attn.k_proj", h).view(b, -1, shape.vis_heads, hd).transpose(1, 2)
        v = w.linear(p + "self_attn.v_proj", h).view(b, -1, shape.vis_heads, hd).transpose(1, 2)
        a = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, dropout_p=0.0, is_causal=False, scale=hd**-0.5)
        a = a.transpose(1, 2).contiguous().reshape(b, -1, shape.vis_hidden)
        x = x + w.linear(p + "self_attn.out_proj", a)
        h = F.layer_norm(x, (shape.vis_hidden,), w[p + "layer_norm2.weight"], w[p + "layer_norm2.bias"], shape.ln_eps)
        h = w.linear(p + "mlp.fc2", F.gelu(w.linear(p + "mlp.fc1", h), approximate="tanh"))
        x = x + h
    x = F.layer_norm(x, (shape.vis_hidden,), w[VIS + "post_layernorm.weight"], w[VIS + "post_layernorm.bias"], shape.ln_eps)
    # pixel shuffle (vision.py:243-252)
    s = shape.scale_factor
    seq, dim = x.shape[1], x.shape[2]
    side = int(seq**0.5)
    x = x.view(b, side, side, dim).view(b, side, side // s, dim * s).permute(0, 2, 1, 3)
    x = x.reshape(b, side // s, side // s, dim * s * s).permute(0, 2, 1, 3).reshape(b, seq // (s * s), dim * s * s)
    return w.linear("vlm_with_expert.vlm.model.connector.modality_projection.proj", x)


def prepare_images(images01: list[torch.Tensor]) -> list[torch.Tensor]:
    """``[1,3,H,W]`` in [0,1], already at the model resolution -> [-1,1] (policy.py:137-138)."""
    return [img * 2.0 - 1.0 for img in images01]


# --------------------------------------------------------------------------- #
# prefix
# --------------------------------------------------------------------------- #
def embed_prefix(w: Weights, shape: SmolVLAShape, images, img_masks, lang_tokens, lang_masks, state):
    """-> ``(embs fp32 [1,P,hidden], pad_masks bool [1,P], att_masks bool [1,P])``."""
    embs, pads, att = [], [], []
    for img, m in zip(images, img_masks):
        e = embed_image(w, shape, img)
        e = e * torch.tensor(e.shape[-1] ** 0.5, dtype=BF16).to(e.dtype)  # bf16-rounded sqrt(hidden)
        embs.append(e)
        pads.append(m[:, None].expand(e.shape[0], e.shape[1]))
        att += [0] * e.shape[1]
    lang = F.embedding(lang_tokens, w[TXT + "embed_tokens.weight"])
    lang = lang * math.sqrt(lang.shape[-1])
    embs.append(lang)
    pads.append(lang_masks)
    att += [0] * lang.shape[1]
    st = w.linear("state_proj", state)[:, None, :]
    embs.append(st)
    pads.append(torch.ones(st.shape[0], 1, dtype=torch.bool))
    att += [1]
    embs = torch.cat(embs, dim=1)  # promotes to fp32
    pads = torch.cat(pads, dim=1)
    att = torch.tensor(att, dtype=torch.bool)[None, :].expand(pads.shape[0], -1)
    return embs, pads, att


def _layer_tail(w: Weights, shape: SmolVLAShape, prefix: str, att_out: torch.Tensor, hidden: torch.Tensor) -> torch.Tensor:
    """o_proj, first residual (in-place add), post norm, MLP, second residual (vlm_with_expert.py:370-410)."""
    out = w.linear(prefix + "self_attn.o_proj", att_out.to(w.act_dtype))
    out += hidden  # bf16 += (fp32|bf16): fp32 math, bf16 result
    after_first = out.clone()
    h = ops.rms_norm_llama(out, w[prefix + "post_attention_layernorm.weight"], shape.rms_eps)
    g = w.linear(prefix + "mlp.gate_proj", h)
    u = w.linear(prefix + "mlp.up_proj", h)
    out = w.linear(prefix + "mlp.down_proj", F.silu(g) * u)
    out += after_first
    return out


def prefill(w: Weights, shape: SmolVLAShape, embs, pad_masks, att_masks):
    """VLM prefill -> per-layer post-RoPE prefix ``(K, V)`` bf16 ``[1, P, G, D]``."""
    mask = ops.make_att_2d_masks(pad_masks, att_masks)
    pos = torch.cumsum(pad_masks, dim=1) - 1
    hidden = embs
    kv = []
    b, length = embs.shape[0], embs.shape[1]
    for i in range(shape.num_vlm_layers):
        p = f"{TXT}layers.{i}."
        h = ops.rms_norm_llama(hidden, w[p + "input_layernorm.weight"], shape.rms_eps).to(w.act_dtype)
        q = w.linear(p + "self_attn.q_proj", h).view(b, length, -1, shape.head_dim)
        k = w.linear(p + "self_attn.k_proj", h).view(b, length, -1, shape.head_dim)
        v = w.linear(p + "self_attn.v_proj", h).view(b, length, -1, shape.head_dim)
        q = ops.rope_half_split(q, pos)
        k = ops.rope_half_split(k, pos)
        kv.append((k, v))
        att = ops.eager_attention(mask, q, k, v)
        hidden = _layer_tail(w, shape, p, att, hidden)
    return kv


def expert_prefix_kv(w: Weights, shape: SmolVLAShape, kv):
    """fp32 expert K/V projections of the VLM prefix K/V for the cross layers (flow_matching.py:553-578)."""
    out = {}
    for i in range(shape.num_vlm_layers):
        if not shape.is_cross(i):
            continue
        p = f"{EXP}layers.{i}.self_attn."
        k, v = kv[i]
        b, length = k.shape[0], k.shape[1]
        ek = w.linear(p + "k_proj", k.to(torch.float32).reshape(b, length, -1)).view(b, length, -1, shape.head_dim)
        ev = w.linear(p + "v_proj", v.to(torch.float32).reshape(b, length, -1)).view(b, length, -1, shape.head_dim)
        out[i] = (ek, ev)
    return out


# --------------------------------------------------------------------------- #
# denoising
# --------------------------------------------------------------------------- #
def embed_suffix(w: Weights, shape: SmolVLAShape, x_t: torch.Tensor, time: float) -> torch.Tensor:
    """fp32 ``[1, chunk, expert_hidden]`` (flow_matching.py:259-311)."""
    a = w.linear("action_in_proj", x_t)
    t = torch.tensor(time, dtype=torch.float32).expand(x_t.shape[0])
    te = ops.sinusoidal_time_embedding(t, shape.expert_hidden, shape.min_period, shape.max_period).to(a.dtype)
    te = te[:, None, :].expand_as(a)
    h = w.linear("action_time_mlp_in", torch.cat([a, te], dim=2))
    return w.linear("action_time_mlp_out", F.silu(h))


def denoise_step(w: Weights, shape: SmolVLAShape, prefix_pad, kv, ekv, x_t, time: float):
    """One velocity evaluation ``v_t`` fp32 ``[1, chunk, max_action_dim]`` (flow_matching.py:316-350)."""
    hidden = embed_suffix(w, shape, x_t, time)
    b, s = hidden.shape[0], hidden.shape[1]
    p_len = prefix_pad.shape[1]
    full_mask = ops.suffix_mask(prefix_pad[0], s, s, ops.MASK_CAUSAL)
    pos = prefix_pad.sum(dim=-1)[:, None] + torch.arange(s)[None, :]
    for i in range(shape.num_vlm_layers):
        p = f"{EXP}layers.{i}."
        h = ops.rms_norm_llama(hidden, w[p + "input_layernorm.weight"], shape.rms_eps)
        if not shape.is_cross(i):
            h = h.to(w.act_dtype)
            q = w.linear(p + "self_attn.q_proj", h).view(b, s, -1, shape.head_dim)
            k = w.linear(p + "self_attn.k_proj", h).view(b, s, -1, shape.head_dim)
            v = w.linear(p + "self_attn.v_proj", h).view(b, s, -1, shape.head_dim)
            q = ops.rope_half_split(q, pos)
            k = ops.rope_half_split(k, pos)
            kk = torch.cat([kv[i][0], k], dim=1)
            vv = torch.cat([kv[i][1], v], dim=1)
            att = ops.eager_attention(full_mask, q, kk, vv)
        else:
            q = w.linear(p + "self_attn.q_proj", h.to(w.act_dtype)).view(b, s, -1, shape.head_dim)
            q = ops.rope_half_split(q, pos - pos.min(dim=1, keepdim=True).values)
            att = ops.eager_attention(full_mask[:, :, :p_len], q, ekv[i][0], ekv[i][1])
        hidden = _layer_tail(w, shape, p, att, hidden)
    out = ops.rms_norm_llama(hidden, w[EXP + "norm.weight"], shape.rms_eps)
    return w.linear("action_out_proj", out.to(torch.float32))


def sample_actions(w: Weights, shape: SmolVLAShape, images, img_masks, lang_tokens, lang_masks, state, noise, trace: dict | None = None, sampler: str = "euler"):
    """Full inference: prefix embed, prefill, expert prefix KV, Euler (or Heun) loop -> ``[1, chunk, max_action_dim]`` fp32."""
    embs, pads, att = embed_prefix(w, shape, images, img_masks, lang_tokens, lang_masks, state)
    kv = prefill(w, shape, embs, pads, att)
    ekv = expert_prefix_kv(w, shape, kv)
    if trace is not None:
        trace["prefix_embs"] = embs
        trace["kv"] = kv
        trace["ekv"] = ekv
        trace["pad_masks"] = pads
    dt = -1.0 / shape.num_steps
    x_t = noise
    for step in range(shape.num_steps):
        t = 1.0 + step * dt
        v_t = denoise_step(w, shape, pads, kv, ekv, x_t, t)
        if trace is not None and step == 0:
            trace["v0"] = v_t
        if sampler == "heun":  # corrector evaluation at t + dt (flow_matching.py:596-625)
            v_1 = denoise_step(w, shape, pads, kv, ekv, x_t + dt * v_t, t + dt)
            x_t = x_t + (dt * 0.5) * (v_t + v_1)
        else:
            x_t = x_t + dt * v_t
    return x_t

"""Parameter inventory of the SmolVLA policy (names, shapes, dtypes of the reference checkpoint
layout: tybok/policies/smolvla/models/{text,expert,vision,flow_matching}.py) and a seeded random
initialiser for benchmarking without a checkpoint.

Random init: every parameter ~ N(0, 0.02) drawn on the CPU from one ``torch.Generator`` in
inventory order, except norm scales (RMSNorm / LayerNorm weight = 1, LayerNorm bias = 0).
"""

from __future__ import annotations

import torch

from .config import SmolVLAConfig

BF16, F32 = torch.bfloat16, torch.float32
VIS = "vlm_with_expert.vlm.model.vision_model."
TXT = "vlm_with_expert.vlm.model.text_model."
EXP = "vlm_with_expert.lm_expert."
CONNECTOR = "vlm_with_expert.vlm.model.connector.modality_projection.proj"


def parameter_inventory(cfg: SmolVLAConfig) -> list[tuple[str, tuple[int, ...], torch.dtype, str]]:
    """``[(name, shape, dtype, kind)]`` with kind in {"normal", "ones", "zeros"}."""
    assert cfg.vlm_config is not None
    t, v = cfg.vlm_config.text_config, cfg.vlm_config.vision_config
    inv: list[tuple[str, tuple[int, ...], torch.dtype, str]] = []

    def lin(name: str, out_f: int, in_f: int, bias: bool = False, dtype=BF16):
        inv.append((name + ".weight", (out_f, in_f), dtype, "normal"))
        if bias:
            inv.append((name + ".bias", (out_f,), dtype, "normal"))

    # vision tower
    inv.append((VIS + "embeddings.patch_embedding.weight", (v.hidden_size, 3, v.patch_size, v.patch_size), BF16, "normal"))
    inv.append((VIS + "embeddings.patch_embedding.bias", (v.hidden_size,), BF16, "normal"))
    n_pos = (v.image_size // v.patch_size) ** 2
    inv.append((VIS + "embeddings.position_embedding.weight", (n_pos, v.hidden_size), BF16, "normal"))
    for i in range(v.num_hidden_layers):
        p = f"{VIS}encoder.layers.{i}."
        for ln in ("layer_norm1", "layer_norm2"):
            inv.append((p + ln + ".weight", (v.hidden_size,), BF16, "ones"))
            inv.append((p + ln + ".bias", (v.hidden_size,), BF16, "zeros"))
        for proj in ("q_proj", "k_proj", "v_proj", "out_proj"):
            lin(p + "self_attn." + proj, v.hidden_size, v.hidden_size, bias=True)
        lin(p + "mlp.fc1", v.intermediate_size, v.hidden_size, bias=True)
        lin(p + "mlp.fc2", v.hidden_size, v.intermediate_size, bias=True)
    inv.append((VIS + "post_layernorm.weight", (v.hidden_size,), BF16, "ones"))
    inv.append((VIS + "post_layernorm.bias", (v.hidden_size,), BF16, "zeros"))
    lin(CONNECTOR, t.hidden_size, v.hidden_size * cfg.vlm_config.scale_factor**2)

    # VLM text decoder (first num_vlm_layers layers)
    inv.append((TXT + "embed_tokens.weight", (t.vocab_size, t.hidden_size), BF16, "normal"))
    q_dim, kv_dim = t.num_attention_heads * t.head_dim, t.num_key_value_heads * t.head_dim
    for i in range(cfg.num_vlm_layers):
        p = f"{TXT}layers.{i}."
        inv.append((p + "input_layernorm.weight", (t.hidden_size,), BF16, "ones"))
        lin(p + "self_attn.q_proj", q_dim, t.hidden_size)
        lin(p + "self_attn.k_proj", kv_dim, t.hidden_size)
        lin(p + "self_attn.v_proj", kv_dim, t.hidden_size)
        lin(p + "self_attn.o_proj", t.hidden_size, q_dim)
        inv.append((p + "post_attention_layernorm.weight", (t.hidden_size,), BF16, "ones"))
        lin(p + "mlp.gate_proj", t.intermediate_size, t.hidden_size)
        lin(p + "mlp.up_proj", t.intermediate_size, t.hidden_size)
        lin(p + "mlp.down_proj", t.hidden_size, t.intermediate_size)
    inv.append((TXT + "norm.weight", (t.hidden_size,), BF16, "ones"))

    # action expert
    eh, ei = cfg.expert_hidden_size, cfg.expert_intermediate_size
    for i in range(cfg.n_expert_layers):
        p = f"{EXP}layers.{i}."
        inv.append((p + "input_layernorm.weight", (eh,), BF16, "ones"))
        lin(p + "self_attn.q_proj", q_dim, eh)
        if cfg.is_cross_layer(i):
            # fp32 projections of the VLM prefix K/V (a checkpoint quirk the reference preserves)
            lin(p + "self_attn.k_proj", kv_dim, kv_dim, dtype=F32)
            lin(p + "self_attn.v_proj", kv_dim, kv_dim, dtype=F32)
        else:
            lin(p + "self_attn.k_proj", kv_dim, eh)
            lin(p + "self_attn.v_proj", kv_dim, eh)
        lin(p + "self_attn.o_proj", eh, q_dim)
        inv.append((p + "post_attention_layernorm.weight", (eh,), BF16, "ones"))
        lin(p + "mlp.gate_proj", ei, eh)
        lin(p + "mlp.up_proj", ei, eh)
        lin(p + "mlp.down_proj", eh, ei)
    inv.append((EXP + "norm.weight", (eh,), BF16, "ones"))

    # flow-matching head (fp32)
    lin("state_proj", t.hidden_size, cfg.max_state_dim, bias=True, dtype=F32)
    lin("action_in_proj", eh, cfg.max_action_dim, bias=True, dtype=F32)
    lin("action_out_proj", cfg.max_action_dim, eh, bias=True, dtype=F32)
    lin("action_time_mlp_in", eh, 2 * eh, bias=True, dtype=F32)
    lin("action_time_mlp_out", eh, eh, bias=True, dtype=F32)
    return inv


def random_state_dict(cfg: SmolVLAConfig, seed: int = 0, std: float = 0.02) -> dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(int(seed))
    sd: dict[str, torch.Tensor] = {}
    for name, shape, dtype, kind in parameter_inventory(cfg):
        if kind == "ones":
            sd[name] = torch.ones(shape, dtype=dtype)
        elif kind == "zeros":
            sd[name] = torch.zeros(shape, dtype=dtype)
        else:
            sd[name] = (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)
    return sd

"""Parameter inventory of the pi0.5 policy (names, shapes, dtypes of the reference checkpoint
layout: tybok/policies/pi05/models/{paligemma_with_expert,gemma,layers,vision,flow_matching}.py)
and a seeded random initialiser for benchmarking without a checkpoint.

Random init: every parameter ~ N(0, 0.02) from one CPU ``torch.Generator`` in inventory order,
except norm scales (LayerNorm weight 1 / bias 0, plain Gemma RMSNorm weight 0, i.e. scale 1).
"""

from __future__ import annotations

import torch

from .config import PI05Config

BF16, F32 = torch.bfloat16, torch.float32
PWE = "paligemma_with_expert."
VIS = PWE + "paligemma.model.vision_tower.vision_model."
PROJ = PWE + "paligemma.model.multi_modal_projector.linear"
VLM = PWE + "paligemma.model.language_model."
EXP = PWE + "gemma_expert.model."


def parameter_inventory(cfg: PI05Config) -> list[tuple[str, tuple[int, ...], torch.dtype, str]]:
    inv: list[tuple[str, tuple[int, ...], torch.dtype, str]] = []

    def lin(name: str, out_f: int, in_f: int, bias: bool, dtype):
        inv.append((name + ".weight", (out_f, in_f), dtype, "normal"))
        if bias:
            inv.append((name + ".bias", (out_f,), dtype, "normal"))

    vh = cfg.vision_hidden
    inv.append((VIS + "embeddings.patch_embedding.weight", (vh, 3, cfg.vision_patch, cfg.vision_patch), F32, "normal"))
    inv.append((VIS + "embeddings.patch_embedding.bias", (vh,), F32, "normal"))
    inv.append((VIS + "embeddings.position_embedding.weight", (cfg.image_tokens, vh), F32, "normal"))
    for i in range(cfg.vision_layers):
        p = f"{VIS}encoder.layers.{i}."
        inv.append((p + "layer_norm1.weight", (vh,), F32, "ones"))
        inv.append((p + "layer_norm1.bias", (vh,), F32, "zeros"))
        for proj in ("k_proj", "v_proj", "q_proj", "out_proj"):
            lin(p + "self_attn." + proj, vh, vh, True, F32)
        inv.append((p + "layer_norm2.weight", (vh,), F32, "ones"))
        inv.append((p + "layer_norm2.bias", (vh,), F32, "zeros"))
        lin(p + "mlp.fc1", cfg.vision_mlp, vh, True, F32)
        lin(p + "mlp.fc2", vh, cfg.vision_mlp, True, F32)
    inv.append((VIS + "post_layernorm.weight", (vh,), F32, "ones"))
    inv.append((VIS + "post_layernorm.bias", (vh,), F32, "zeros"))
    lin(PROJ, cfg.paligemma_dims["width"], vh, True, F32)

    def decoder(prefix: str, d: dict[str, int], adarms: bool, vocab: int | None):
        width, q_dim, kv_dim = d["width"], d["num_heads"] * d["head_dim"], d["num_kv_heads"] * d["head_dim"]

        def norm(name: str):
            if adarms:
                lin(name + ".dense", 3 * width, width, True, F32)
            else:
                inv.append((name + ".weight", (width,), F32, "zeros"))

        for i in range(d["depth"]):
            p = f"{prefix}layers.{i}."
            lin(p + "self_attn.q_proj", q_dim, width, False, BF16)
            lin(p + "self_attn.k_proj", kv_dim, width, False, BF16)
            lin(p + "self_attn.v_proj", kv_dim, width, False, BF16)
            lin(p + "self_attn.o_proj", width, q_dim, False, BF16)
            lin(p + "mlp.gate_proj", d["mlp_dim"], width, False, BF16)
            lin(p + "mlp.up_proj", d["mlp_dim"], width, False, BF16)
            lin(p + "mlp.down_proj", width, d["mlp_dim"], False, BF16)
            norm(p + "input_layernorm")
            norm(p + "post_attention_layernorm")
        norm(prefix + "norm")
        if vocab is not None:
            inv.append((prefix + "embed_tokens.weight", (vocab, width), BF16, "normal"))

    decoder(VLM, cfg.paligemma_dims, False, cfg.vocab_size)
    decoder(EXP, cfg.expert_dims, True, None)
    ew = cfg.expert_dims["width"]
    lin("action_in_proj", ew, cfg.max_action_dim, True, F32)
    lin("action_out_proj", cfg.max_action_dim, ew, True, F32)
    lin("time_mlp_in", ew, ew, True, F32)
    lin("time_mlp_out", ew, ew, True, F32)
    return inv


def random_state_dict(cfg: PI05Config, seed: int = 0, std: float = 0.02) -> dict[str, torch.Tensor]:
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

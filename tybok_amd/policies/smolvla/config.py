"""SmolVLA checkpoint configuration (same JSON fields and defaults as the reference's
``tybok/policies/smolvla/config.py:21-258``) plus the random-init marker used for benchmarking
without a checkpoint.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any


@dataclass
class TextConfig:
    hidden_size: int = 960
    intermediate_size: int = 2560
    num_hidden_layers: int = 32
    num_attention_heads: int = 15
    num_key_value_heads: int = 5
    head_dim: int = 64
    rms_norm_eps: float = 1e-5
    vocab_size: int = 49280

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "TextConfig":
        return cls(**{k: d[k] for k in cls.__dataclass_fields__ if k in d})


@dataclass
class VisionConfig:
    hidden_size: int = 768
    intermediate_size: int = 3072
    num_hidden_layers: int = 12
    num_attention_heads: int = 12
    image_size: int = 512
    patch_size: int = 16
    layer_norm_eps: float = 1e-6

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "VisionConfig":
        return cls(**{k: d[k] for k in cls.__dataclass_fields__ if k in d})


@dataclass
class VLMConfig:
    text_config: TextConfig = field(default_factory=TextConfig)
    vision_config: VisionConfig = field(default_factory=VisionConfig)
    scale_factor: int = 4

    @property
    def image_seq_len(self) -> int:
        side = self.vision_config.image_size // self.vision_config.patch_size
        return side * side // (self.scale_factor**2)

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "VLMConfig":
        return cls(
            text_config=TextConfig.from_dict(d.get("text_config", {})),
            vision_config=VisionConfig.from_dict(d.get("vision_config", {})),
            scale_factor=d.get("scale_factor", 4),
        )


@dataclass
class SmolVLAConfig:
    chunk_size: int = 50
    n_action_steps: int = 50
    max_state_dim: int = 32
    max_action_dim: int = 32
    action_feature_shape: tuple[int, ...] = (6,)
    resize_imgs_with_padding: tuple[int, int] = (512, 512)  # (width, height)
    empty_cameras: int = 0
    tokenizer_max_length: int = 48
    num_steps: int = 10
    sampler: str = "euler"
    cache_expert_prefix_kv: bool = True
    attention_mode: str = "cross_attn"
    self_attn_every_n_layers: int = 2
    num_vlm_layers: int = 16
    num_expert_layers: int = -1
    expert_width_multiplier: float = 0.75
    min_period: float = 4e-3
    max_period: float = 4.0
    normalization_mapping: dict[str, str] = field(
        default_factory=lambda: {"VISUAL": "IDENTITY", "STATE": "MEAN_STD", "ACTION": "MEAN_STD"}
    )
    checkpoint_dir: str = ""
    vlm_model_name: str = ""
    vlm_dir: str = ""
    vlm_config: VLMConfig | None = None
    image_features: list[str] = field(default_factory=list)
    # {"seed": int}: no safetensors in the checkpoint dir, weights are drawn N(0, 0.02) (benchmarks)
    random_init: dict[str, Any] | None = None

    @property
    def n_expert_layers(self) -> int:
        return self.num_vlm_layers if not self.num_expert_layers or self.num_expert_layers <= 0 else self.num_expert_layers

    @property
    def expert_hidden_size(self) -> int:
        assert self.vlm_config is not None
        return int(self.vlm_config.text_config.hidden_size * self.expert_width_multiplier)

    @property
    def expert_intermediate_size(self) -> int:
        # reference: get_intermediate_size, tybok/policies/smolvla/models/vlm_with_expert.py:536-540
        h = int(4 * int(2 * self.expert_hidden_size / 3))
        return 256 * ((h + 255) // 256)

    def is_cross_layer(self, layer: int) -> bool:
        return "cross" in self.attention_mode and not (
            self.self_attn_every_n_layers > 0 and layer % self.self_attn_every_n_layers == 0
        )

    @classmethod
    def from_pretrained(cls, checkpoint_dir: str) -> "SmolVLAConfig":
        with open(os.path.join(checkpoint_dir, "config.json"), "r", encoding="utf-8") as f:
            cfg = json.load(f)
        vlm_name = cfg.get("vlm_model_name", "")
        vlm_dir = ""
        vlm_config = None
        for cand in (vlm_name, os.path.join(checkpoint_dir, vlm_name) if vlm_name else ""):
            if cand and os.path.isfile(os.path.join(cand, "config.json")):
                vlm_dir = cand
                with open(os.path.join(cand, "config.json"), "r", encoding="utf-8") as f:
                    vlm_config = VLMConfig.from_dict(json.load(f))
                break
        if vlm_config is None and "vlm_config" in cfg:  # self-contained (random-init) checkpoints
            vlm_config = VLMConfig.from_dict(cfg["vlm_config"])
            vlm_dir = checkpoint_dir
        image_features = [k for k, feat in cfg.get("input_features", {}).items() if feat.get("type") == "VISUAL"]
        resize = cfg.get("resize_imgs_with_padding", [512, 512])
        names = set(cls.__dataclass_fields__)
        plain = {
            k: cfg[k]
            for k in (
                "chunk_size", "n_action_steps", "max_state_dim", "max_action_dim", "empty_cameras",
                "tokenizer_max_length", "num_steps", "sampler", "cache_expert_prefix_kv", "attention_mode",
                "self_attn_every_n_layers", "num_vlm_layers", "num_expert_layers", "expert_width_multiplier",
                "min_period", "max_period", "normalization_mapping", "random_init",
            )
            if k in cfg and k in names
        }  # fmt: skip
        return cls(
            action_feature_shape=tuple(cfg.get("output_features", {}).get("action", {}).get("shape", (6,))),
            resize_imgs_with_padding=(int(resize[0]), int(resize[1])),
            checkpoint_dir=checkpoint_dir,
            vlm_model_name=vlm_name,
            vlm_dir=vlm_dir,
            vlm_config=vlm_config,
            image_features=image_features,
            **plain,
        )

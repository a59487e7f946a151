"""What a SmolVLA checkpoint directory says about the model.

The attribute names are the keys of the checkpoint's ``config.json`` and of the VLM's own
``config.json`` (``text_config`` / ``vision_config``), with the defaults of the released
``smolvla_base`` -- the same schema the reference reads (tybok/policies/smolvla/config.py:21-258).
One extra key, ``random_init``, marks a directory without weight files (benchmarks, CI).
"""

from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass, field
from typing import Any, TypeVar

T = TypeVar("T")


def _read_json(path: str) -> dict[str, Any]:
    with open(path, encoding="utf-8") as handle:
        return json.load(handle)


def _from_keys(cls: type[T], values: dict[str, Any], **explicit: Any) -> T:
    """``cls`` built from the entries of ``values`` whose key is one of its fields; ``explicit`` wins."""
    known = {f.name for f in dataclasses.fields(cls)}
    picked = {key: value for key, value in values.items() if key in known and key not in explicit}
    return cls(**picked, **explicit)


@dataclass
class TextConfig:
    """Decoder of the VLM (SmolLM2) -- ``text_config``."""

    vocab_size: int = 49280
    hidden_size: int = 960
    num_hidden_layers: int = 32
    num_attention_heads: int = 15  # query heads
    num_key_value_heads: int = 5  # grouped-query attention: 3 query heads per K/V head
    head_dim: int = 64
    intermediate_size: int = 2560  # gated MLP width
    rms_norm_eps: float = 1e-5

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "TextConfig":
        return _from_keys(cls, values)


@dataclass
class VisionConfig:
    """SigLIP-B/16 tower -- ``vision_config``."""

    image_size: int = 512
    patch_size: int = 16  # 32 x 32 patches per image
    hidden_size: int = 768
    num_hidden_layers: int = 12
    num_attention_heads: int = 12
    intermediate_size: int = 3072
    layer_norm_eps: float = 1e-6

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "VisionConfig":
        return _from_keys(cls, values)


@dataclass
class VLMConfig:
    """The VLM's ``config.json``: the two stacks and the connector's pixel-shuffle factor."""

    scale_factor: int = 4
    vision_config: VisionConfig = field(default_factory=VisionConfig)
    text_config: TextConfig = field(default_factory=TextConfig)

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "VLMConfig":
        return cls(
            scale_factor=int(values.get("scale_factor", 4)),
            vision_config=VisionConfig.from_dict(values.get("vision_config") or {}),
            text_config=TextConfig.from_dict(values.get("text_config") or {}),
        )

    @property
    def image_seq_len(self) -> int:
        """Tokens one image contributes to the prefix: patches after the connector's s x s merge."""
        patches_per_side = self.vision_config.image_size // self.vision_config.patch_size
        return (patches_per_side * patches_per_side) // (self.scale_factor * self.scale_factor)


@dataclass
class SmolVLAConfig:
    # -- where things are ---------------------------------------------------------------------
    checkpoint_dir: str = ""
    vlm_model_name: str = ""  # as written in config.json: a path or a hub name
    vlm_dir: str = ""  # the directory the VLM config was actually found in
    vlm_config: VLMConfig | None = None
    # {"seed": int}: no safetensors in the checkpoint dir, weights are drawn N(0, 0.02) (benchmarks)
    random_init: dict[str, Any] | None = None
    # -- observation and action spaces --------------------------------------------------------
    image_features: list[str] = field(default_factory=list)  # "observation.images.<camera>", in order
    resize_imgs_with_padding: tuple[int, int] = (512, 512)  # (width, height)
    empty_cameras: int = 0
    tokenizer_max_length: int = 48
    max_state_dim: int = 32
    max_action_dim: int = 32  # the model's padded action width
    action_feature_shape: tuple[int, ...] = (6,)  # the robot's action width
    normalization_mapping: dict[str, str] = field(default_factory=lambda: dict(VISUAL="IDENTITY", STATE="MEAN_STD", ACTION="MEAN_STD"))
    # -- sampling -----------------------------------------------------------------------------
    chunk_size: int = 50
    n_action_steps: int = 50
    num_steps: int = 10  # Euler steps of the flow-matching sampler
    sampler: str = "euler"
    min_period: float = 4e-3  # sinusoidal time embedding
    max_period: float = 4.0
    # -- the two stacks -----------------------------------------------------------------------
    num_vlm_layers: int = 16  # decoder layers of the VLM that are kept
    num_expert_layers: int = -1  # <= 0: as many as the VLM keeps
    expert_width_multiplier: float = 0.75
    attention_mode: str = "cross_attn"
    self_attn_every_n_layers: int = 2  # expert layers 0, n, 2n, ... attend to [prefix; suffix], the others to the prefix only
    cache_expert_prefix_kv: bool = True

    # ------------------------------------------------------------------ derived sizes
    @property
    def n_expert_layers(self) -> int:
        return self.num_expert_layers if self.num_expert_layers and self.num_expert_layers > 0 else self.num_vlm_layers

    @property
    def expert_hidden_size(self) -> int:
        if self.vlm_config is None:
            raise ValueError("the VLM configuration has not been loaded")
        return int(self.expert_width_multiplier * self.vlm_config.text_config.hidden_size)

    @property
    def expert_intermediate_size(self) -> int:
        """8/3 of the hidden size, rounded up to a multiple of 256
        (``get_intermediate_size``, tybok/policies/smolvla/models/vlm_with_expert.py:536-540)."""
        two_thirds = int(2 * self.expert_hidden_size / 3)
        return -(-(4 * two_thirds) // 256) * 256

    def is_cross_layer(self, layer: int) -> bool:
        """Whether expert layer ``layer`` attends to the prefix only (expert.py:66-79)."""
        if "cross" not in self.attention_mode:
            return False
        every = self.self_attn_every_n_layers
        return not (every > 0 and layer % every == 0)

    # ------------------------------------------------------------------ loading
    _PLAIN_KEYS = (
        "chunk_size", "n_action_steps", "num_steps", "sampler", "min_period", "max_period", "max_state_dim", "max_action_dim",
        "empty_cameras", "tokenizer_max_length", "normalization_mapping", "num_vlm_layers", "num_expert_layers",
        "expert_width_multiplier", "attention_mode", "self_attn_every_n_layers", "cache_expert_prefix_kv", "random_init",
    )  # fmt: skip

    @classmethod
    def from_pretrained(cls, checkpoint_dir: str) -> "SmolVLAConfig":
        raw = _read_json(os.path.join(checkpoint_dir, "config.json"))
        vlm_name = raw.get("vlm_model_name", "")
        # the VLM's own config: next to the name as given, else relative to the checkpoint, else embedded
        vlm_dir, vlm_config = "", None
        for candidate in filter(None, (vlm_name, vlm_name and os.path.join(checkpoint_dir, vlm_name))):
            if os.path.isfile(os.path.join(candidate, "config.json")):
                vlm_dir, vlm_config = candidate, VLMConfig.from_dict(_read_json(os.path.join(candidate, "config.json")))
                break
        if vlm_config is None and "vlm_config" in raw:
            vlm_dir, vlm_config = checkpoint_dir, VLMConfig.from_dict(raw["vlm_config"])
        width, height = raw.get("resize_imgs_with_padding", (512, 512))
        action_shape = raw.get("output_features", {}).get("action", {}).get("shape", (6,))
        cameras = [name for name, feature in raw.get("input_features", {}).items() if feature.get("type") == "VISUAL"]
        return cls(
            checkpoint_dir=checkpoint_dir, vlm_model_name=vlm_name, vlm_dir=vlm_dir, vlm_config=vlm_config,
            image_features=cameras, resize_imgs_with_padding=(int(width), int(height)), action_feature_shape=tuple(action_shape),
            **{key: raw[key] for key in cls._PLAIN_KEYS if key in raw},
        )  # fmt: skip

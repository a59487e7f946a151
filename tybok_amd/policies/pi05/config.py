"""pi0.5 checkpoint configuration (fields/defaults of the reference's
``tybok/policies/pi05/config.py:15-174``) plus the random-init marker used for benchmarking
without a checkpoint.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any

GEMMA_VARIANTS: dict[str, dict[str, int]] = {
    "gemma_300m": {"width": 1024, "depth": 18, "mlp_dim": 4096, "num_heads": 8, "num_kv_heads": 1, "head_dim": 256},
    "gemma_2b": {"width": 2048, "depth": 18, "mlp_dim": 16384, "num_heads": 8, "num_kv_heads": 1, "head_dim": 256},
}
PALIGEMMA_VOCAB_SIZE = 257152


@dataclass
class PI05Config:
    chunk_size: int = 50
    n_action_steps: int = 50
    max_state_dim: int = 32
    max_action_dim: int = 32
    action_feature_shape: tuple[int, ...] = (7,)
    paligemma_variant: str = "gemma_2b"
    action_expert_variant: str = "gemma_300m"
    image_resolution: tuple[int, int] = (224, 224)  # (height, width)
    empty_cameras: int = 0
    tokenizer_max_length: int = 200
    num_steps: int = 10
    min_period: float = 4e-3
    max_period: float = 4.0
    sampler: str = "euler"
    normalization_mapping: dict[str, str] = field(
        default_factory=lambda: {"VISUAL": "IDENTITY", "STATE": "MEAN_STD", "ACTION": "MEAN_STD"}
    )
    checkpoint_dir: str = ""
    tokenizer_dir: str = ""
    image_features: list[str] = field(default_factory=list)
    # SigLIP-So400m/14 tower
    vision_hidden: int = 1152
    vision_heads: int = 16
    vision_layers: int = 27
    vision_mlp: int = 4304
    vision_patch: int = 14
    vocab_size: int = PALIGEMMA_VOCAB_SIZE
    # explicit decoder dims override the named variants (reduced-depth test models)
    paligemma_dims: dict[str, int] = field(default_factory=dict)
    expert_dims: dict[str, int] = field(default_factory=dict)
    random_init: dict[str, Any] | None = None

    def __post_init__(self):
        if not self.paligemma_dims:
            self.paligemma_dims = dict(GEMMA_VARIANTS[self.paligemma_variant])
        if not self.expert_dims:
            self.expert_dims = dict(GEMMA_VARIANTS[self.action_expert_variant])

    @property
    def real_camera_keys(self) -> list[str]:
        return [k for k in self.image_features if "empty_camera" not in k]

    def live_camera_keys(self, batch: dict) -> list[str]:
        """``pad_free``: the camera slots a request populates -- no ``empty_camera_*`` placeholder slots, no real
        camera missing from the frame (tybok/policies/pi05/config.py:113-123).  One rule for the eager path and for
        the recorded shapes, so both build the same prefix length."""
        return [k for k in self.real_camera_keys if k in batch]

    @property
    def image_tokens(self) -> int:
        return (self.image_resolution[0] // self.vision_patch) ** 2

    @classmethod
    def shaped(cls, depth: int = 18, vision_layers: int = 27, cameras: int = 2, num_steps: int = 10) -> "PI05Config":
        """pi0.5-shaped config with the given decoder / tower depth (benchmarks, tests)."""
        vlm = dict(GEMMA_VARIANTS["gemma_2b"], depth=depth)
        exp = dict(GEMMA_VARIANTS["gemma_300m"], depth=depth)
        names = ["base_0_rgb", "left_wrist_0_rgb", "right_wrist_0_rgb"][:cameras]
        return cls(
            num_steps=num_steps,
            vision_layers=vision_layers,
            paligemma_dims=vlm,
            expert_dims=exp,
            image_features=[f"observation.images.{n}" for n in names],
        )

    @classmethod
    def from_pretrained(cls, checkpoint_dir: str, tokenizer_dir: str | None = None) -> "PI05Config":
        with open(os.path.join(checkpoint_dir, "config.json"), "r", encoding="utf-8") as f:
            cfg = json.load(f)
        image_features = [k for k, feat in cfg.get("input_features", {}).items() if feat.get("type") == "VISUAL"]
        res = cfg.get("image_resolution", [224, 224])
        kw: dict[str, Any] = {}
        for k in ("chunk_size", "n_action_steps", "max_state_dim", "max_action_dim", "paligemma_variant",
                  "action_expert_variant", "empty_cameras", "tokenizer_max_length", "min_period", "max_period",
                  "sampler", "normalization_mapping", "random_init", "vision_layers", "paligemma_dims", "expert_dims"):  # fmt: skip
            if k in cfg:
                kw[k] = cfg[k]
        return cls(
            action_feature_shape=tuple(cfg.get("output_features", {}).get("action", {}).get("shape", (7,))),
            image_resolution=(int(res[0]), int(res[1])),
            num_steps=cfg.get("num_inference_steps", cfg.get("num_steps", 10)),
            checkpoint_dir=checkpoint_dir,
            tokenizer_dir=tokenizer_dir or cfg.get("tokenizer_dir", ""),
            image_features=image_features,
            **kw,
        )

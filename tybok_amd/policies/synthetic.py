"""Random-init checkpoint directories (a ``config.json`` only) for benchmarks and tests: the
engines draw N(0, 0.02) weights from the recorded seed instead of reading safetensors, and use a
synthetic tokenizer.  The layout follows the lerobot ``config.json`` conventions the reference
reads (``type``, ``input_features``, ``output_features``)."""

from __future__ import annotations

import json
import os


def write_smolvla_checkpoint(path: str, cameras: int = 3, seed: int = 0, num_vlm_layers: int = 16, vision_layers: int = 12, num_steps: int = 10) -> str:
    os.makedirs(path, exist_ok=True)
    cfg = {
        "type": "smolvla",
        "input_features": {
            **{f"observation.images.camera{i + 1}": {"type": "VISUAL", "shape": [3, 512, 512]} for i in range(cameras)},
            "observation.state": {"type": "STATE", "shape": [6]},
        },
        "output_features": {"action": {"type": "ACTION", "shape": [6]}},
        "num_vlm_layers": num_vlm_layers,
        "num_steps": num_steps,
        "vlm_config": {"text_config": {}, "vision_config": {"num_hidden_layers": vision_layers}, "scale_factor": 4},
        "random_init": {"seed": seed},
    }
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    return path


def write_pi05_checkpoint(path: str, cameras: int = 2, seed: int = 0, depth: int = 18, vision_layers: int = 27, num_steps: int = 10) -> str:
    from .pi05.config import GEMMA_VARIANTS

    os.makedirs(path, exist_ok=True)
    names = ["base_0_rgb", "left_wrist_0_rgb", "right_wrist_0_rgb"][:cameras]
    cfg = {
        "type": "pi05",
        "input_features": {
            **{f"observation.images.{n}": {"type": "VISUAL", "shape": [3, 224, 224]} for n in names},
            "observation.state": {"type": "STATE", "shape": [8]},
        },
        "output_features": {"action": {"type": "ACTION", "shape": [7]}},
        "num_inference_steps": num_steps,
        "vision_layers": vision_layers,
        "paligemma_dims": dict(GEMMA_VARIANTS["gemma_2b"], depth=depth),
        "expert_dims": dict(GEMMA_VARIANTS["gemma_300m"], depth=depth),
        "random_init": {"seed": seed},
    }
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    return path


def write_weight_files(path: str) -> str:
    """Materialise the random-init weights of a synthetic checkpoint as ``model.safetensors`` and
    switch its config to read weights from files (``random_init.weights = "files"``; tokenizer and
    normalisation statistics stay synthetic).  Lets the file loaders -- including the fp8 checkpoint
    format -- run without a downloaded model."""
    from safetensors.torch import save_file

    with open(os.path.join(path, "config.json"), encoding="utf-8") as f:
        cfg = json.load(f)
    seed = int(cfg["random_init"]["seed"])
    if cfg["type"] == "smolvla":
        from .smolvla.config import SmolVLAConfig
        from .smolvla.weights import random_state_dict

        sd = random_state_dict(SmolVLAConfig.from_pretrained(path), seed=seed)
    else:
        from .pi05.config import PI05Config
        from .pi05.weights import random_state_dict

        sd = random_state_dict(PI05Config.from_pretrained(path), seed=seed)
    save_file({k: v.contiguous() for k, v in sd.items()}, os.path.join(path, "model.safetensors"))
    cfg["random_init"]["weights"] = "files"
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    return path

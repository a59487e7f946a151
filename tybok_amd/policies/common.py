"""Pieces shared by the two backends: dataset-statistics (un)normalisation, the task tokenizers
and the safetensors parameter loader.  Behaviour follows the reference's per-backend copies
(tybok/policies/smolvla/preprocess.py:36-182, tybok/policies/smolvla/tokenizer.py:31-87,
tybok/policies/smolvla/models/policy.py:38-68).
"""

from __future__ import annotations

import glob
import hashlib
import os
from dataclasses import dataclass, field
from typing import Any

import torch

OBS_STATE = "observation.state"
OBS_LANGUAGE_TOKENS = "observation.language.tokens"
OBS_LANGUAGE_ATTENTION_MASK = "observation.language.attention_mask"
ACTION = "action"


@dataclass
class Normalizer:
    """Per-feature MEAN_STD (un)normalisation; identity when the key has no statistics."""

    norm_map: dict[str, str]
    stats: dict[str, dict[str, torch.Tensor]] = field(default_factory=dict)
    eps: float = 1e-8

    @classmethod
    def from_files(cls, pattern: str, norm_map: dict[str, str]) -> "Normalizer":
        stats: dict[str, dict[str, torch.Tensor]] = {}
        for file in sorted(glob.glob(pattern)):
            from safetensors import safe_open

            with safe_open(file, "pt", "cpu") as f:
                for flat in f.keys():
                    key, stat = flat.rsplit(".", 1)
                    stats.setdefault(key, {})[stat] = f.get_tensor(flat).float()
        return cls(norm_map=norm_map, stats=stats)

    def _apply(self, t: torch.Tensor, key: str, ftype: str, inverse: bool) -> torch.Tensor:
        mode = self.norm_map.get(ftype, "IDENTITY")
        if mode == "IDENTITY" or key not in self.stats:
            return t
        if mode != "MEAN_STD":
            raise ValueError(f"Unsupported normalization mode: {mode}")
        mean, std = self.stats[key].get("mean"), self.stats[key].get("std")
        if mean is None or std is None:
            raise ValueError("MEAN_STD normalization mode requires mean and std stats")
        mean, std = mean.to(t.device), std.to(t.device)
        return t * std + mean if inverse else (t - mean) / (std + self.eps)

    def normalize(self, t, key, ftype):
        return self._apply(t, key, ftype, False)

    def unnormalize(self, t, key, ftype):
        return self._apply(t, key, ftype, True)


def load_normalizer(checkpoint_dir: str, norm_map: dict[str, str]) -> Normalizer:
    return Normalizer.from_files(
        os.path.join(checkpoint_dir, "policy_preprocessor_step_*_normalizer_processor.safetensors"), norm_map
    )


def load_unnormalizer(checkpoint_dir: str, norm_map: dict[str, str]) -> Normalizer:
    return Normalizer.from_files(
        os.path.join(checkpoint_dir, "policy_postprocessor_step_*_unnormalizer_processor.safetensors"), norm_map
    )


class FileTokenizer:
    """``tokenizers`` tokenizer loaded from ``tokenizer.json``: truncation + right padding to ``max_length``."""

    def __init__(self, tokenizer_dir: str, max_length: int, pad_token: str, append_newline: bool = True):
        from tokenizers import Tokenizer

        self.tok = Tokenizer.from_file(os.path.join(tokenizer_dir, "tokenizer.json"))
        self.max_length = max_length
        self.tok.enable_truncation(max_length=max_length)
        pad_id = self.tok.token_to_id(pad_token)
        self.tok.enable_padding(pad_id=pad_id if pad_id is not None else 0, pad_token=pad_token, length=max_length, direction="right")

    def encode_task(self, task: str) -> tuple[torch.Tensor, torch.Tensor]:
        enc = self.tok.encode(task)
        return torch.tensor([enc.ids], dtype=torch.long), torch.tensor([enc.attention_mask], dtype=torch.bool)


class SyntheticTokenizer:
    """Stand-in for random-init checkpoints (no ``tokenizer.json``): ``max_length`` token ids drawn
    from a generator seeded by the task string, all unmasked.  Deterministic per task."""

    def __init__(self, vocab_size: int, max_length: int):
        self.vocab_size, self.max_length = int(vocab_size), int(max_length)

    def encode_task(self, task: str) -> tuple[torch.Tensor, torch.Tensor]:
        seed = int.from_bytes(hashlib.sha256(task.encode("utf-8")).digest()[:4], "little")
        g = torch.Generator().manual_seed(seed)
        ids = torch.randint(0, self.vocab_size, (1, self.max_length), generator=g)
        return ids, torch.ones(1, self.max_length, dtype=torch.bool)


def load_state_dict(checkpoint_dir: str, wanted: dict[str, tuple], remap: dict[str, str] | None = None) -> dict[str, torch.Tensor]:
    """Read the checkpoint's ``*.safetensors`` (processor statistics aside) and return the tensors
    whose names (minus a leading ``model.``) are in ``wanted``; raises if one is missing.

    A file that contains ``*.scale_weight`` keys is a self-contained fp8 file: when one is present,
    only fp8 files are read (docs/fastWAM_weight_quantization.md:9), and the ``<module>.scale_weight``
    of every wanted fp8 ``<module>.weight`` is returned beside it."""
    from safetensors import safe_open

    from ..fp8_checkpoint import SCALE_SUFFIX, fp8_files

    files = fp8_files(checkpoint_dir) or [
        f for f in sorted(glob.glob(os.path.join(checkpoint_dir, "*.safetensors"))) if "processor" not in os.path.basename(f)
    ]
    out: dict[str, torch.Tensor] = {}
    for file in files:
        with safe_open(file, "pt", "cpu") as f:
            for name in f.keys():
                key = (remap or {}).get(name, name)
                for cand in (key, key[len("model.") :] if key.startswith("model.") else None):
                    if cand is None:
                        continue
                    if cand in wanted:
                        out[cand] = f.get_tensor(name)
                        break
                    if cand.endswith(SCALE_SUFFIX) and cand[: -len(SCALE_SUFFIX)] + ".weight" in wanted:
                        out[cand] = f.get_tensor(name)
                        break
    missing = [k for k in wanted if k not in out]
    if missing:
        raise FileNotFoundError(f"{len(missing)} parameters missing from {checkpoint_dir} (e.g. {missing[0]})")
    return out


# ---------------------------------------------------------------------- validate() plumbing
DUMP_FILES = ("frame.pt", "batch.pt", "prefix.pt", "prefix_kv.pt", "denoise.pt", "chunk.pt")
REQUIRED_DUMP_FILES = ("frame.pt", "chunk.pt")


def load_reference_dump(reference_dir: str) -> dict[str, Any]:
    """The files of a ``validate`` dump directory by stem (``frame``, ``batch``, ``prefix``, ``prefix_kv``,
    ``denoise``, ``chunk``; the layout of tybok/policies/smolvla/engine.py:668-673).  ``frame`` and
    ``chunk`` must exist, a missing optional file maps to ``None``.  Files are read with
    ``weights_only=True``: tensors and plain containers, nothing executable."""
    dump: dict[str, Any] = {}
    for name in DUMP_FILES:
        path = os.path.join(reference_dir, name)
        if os.path.exists(path):
            dump[name[:-3]] = torch.load(path, weights_only=True)
        elif name in REQUIRED_DUMP_FILES:
            raise FileNotFoundError(f"reference dump {path} missing")
        else:
            dump[name[:-3]] = None
    return dump


class ErrorReport(dict):
    """``{"<component>.max": ..., "<component>.mean": ...}`` -- the keys of the reference's validation report."""

    def compare(self, component: str, got: torch.Tensor, want: torch.Tensor) -> None:
        got, want = got.detach().float().cpu(), want.detach().float().cpu()
        if got.shape != want.shape:
            raise AssertionError(f"{component}: shape mismatch {tuple(got.shape)} vs {tuple(want.shape)}")
        distance = (got - want).abs()
        self[f"{component}.max"] = float(distance.max())
        self[f"{component}.mean"] = float(distance.mean())

    def compare_batch(self, batch: dict[str, torch.Tensor], want: dict[str, Any] | None, keys: tuple[str, ...]) -> None:
        """The preprocessed request: the named keys plus every camera image of the dump."""
        if want is None:
            return
        for key in (*keys, *(k for k in want if k.startswith("observation.images."))):
            if key in batch and key in want:
                self.compare(f"batch.{key}", batch[key], want[key])

    def compare_prefix_kv(self, kv, want: dict[str, Any] | None) -> None:
        """``kv``: per layer ``(keys, values)``; the dump holds ``layer<i>: {"keys", "values"}``."""
        if want is None:
            return
        for i, (keys, values) in enumerate(kv):
            self.compare(f"prefix_kv.layer{i}.keys", keys, want[f"layer{i}"]["keys"])
            self.compare(f"prefix_kv.layer{i}.values", values, want[f"layer{i}"]["values"])

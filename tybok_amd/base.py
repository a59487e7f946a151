"""Model-agnostic engine interface, API-compatible with the reference's ``tybok/base.py``.

The gateway / worker layers of the reference only depend on this interface
(``PolicyEngine.{describe, select_action, predict_action_chunk, validate, profile}``:
tybok/base.py:50-235), so a backend registered under the same name with the same constructor
keywords is a drop-in.  ``compile_region`` (torch.compile plumbing) has no counterpart here: the
HIP tiers replace it, and ``compile_model=True`` is rejected by the backends.
"""

from __future__ import annotations

import logging
import time
from abc import ABC, abstractmethod
from collections.abc import Mapping
from typing import Any

import numpy as np
import torch

log = logging.getLogger("tybok.engine")


class PolicyEngine(ABC):
    """Base class of the policy backends (inference only)."""

    config: Any
    compile_model: bool
    graph_enabled: bool

    def __init__(self, checkpoint_dir: str, device: str = "auto", **kwargs):
        self.checkpoint_dir = checkpoint_dir
        if device == "auto":
            device = "cuda" if torch.cuda.is_available() else "cpu"
        self.device = device
        self.compiled_regions: list[str] = []
        if isinstance(device, str) and device.startswith("cuda"):
            dev = torch.device(device)
            if dev.index is not None:
                torch.cuda.set_device(dev)

    # ------------------------------------------------------------------ interface
    @abstractmethod
    def describe(self) -> dict[str, Any]:
        """``{"model_type", "cameras", "resize": [W, H], "action_dim", "chunk_size", ...}``."""

    @abstractmethod
    def select_action(self, frame: dict[str, Any], noise: torch.Tensor | None = None) -> np.ndarray:
        """One action ``(action_dim,)`` for one observation frame."""

    @abstractmethod
    def predict_action_chunk(self, frame: dict[str, Any], noise: torch.Tensor | None = None) -> np.ndarray:
        """Full chunk ``(chunk_size, action_dim)`` for one observation frame."""

    @abstractmethod
    def validate(self, reference_dir: str) -> dict[str, float]:
        """Score this backend against a reference dump directory."""

    def supports_rtc(self) -> bool:
        return False

    # ------------------------------------------------------------------ shared helpers
    def make_frame(
        self,
        images: Mapping[str, torch.Tensor | np.ndarray],
        state: torch.Tensor | np.ndarray | list,
        task: str,
    ) -> dict[str, Any]:
        """Raw frame dict: ``(C,H,W)`` fp32 images in [0,1] under ``observation.images.<cam>``,
        a 1-D fp32 ``observation.state`` and the ``task`` string."""
        frame: dict[str, Any] = {}
        for key, img in images.items():
            if isinstance(img, np.ndarray):
                img = torch.from_numpy(img)
            if not torch.is_tensor(img):
                raise TypeError(f"image {key} must be a tensor or ndarray")
            if img.ndim == 3 and img.shape[0] not in (1, 3, 4):
                img = img.permute(2, 0, 1)  # HWC -> CHW
            frame[f"observation.images.{key}"] = img.float().contiguous()
        if isinstance(state, (list, tuple)):
            state = np.asarray(state, dtype=np.float32)
        if isinstance(state, np.ndarray):
            state = torch.from_numpy(state.astype(np.float32))
        frame["observation.state"] = state.float().contiguous()
        frame["task"] = task
        return frame

    def _warmup(self) -> None:
        """One dummy inference so lazy initialisation does not land on the first request."""
        spec = self.describe()
        t0 = time.perf_counter()
        images = {cam: torch.zeros(3, spec["resize"][1], spec["resize"][0]) for cam in spec["cameras"]}
        frame = self.make_frame(images, torch.zeros(8), "warmup")
        self.predict_action_chunk(frame)
        if str(self.device).startswith("cuda"):
            torch.cuda.synchronize()
        log.info(f"warmup done in {time.perf_counter() - t0:.1f}s")

    def _profile_frame(self, cameras: int | None = None, seed: int = 0) -> dict[str, Any]:
        """Synthetic frame: random images for the configured (or requested) cameras + random state."""
        spec = self.describe()
        g = torch.Generator().manual_seed(seed)
        cams = spec["cameras"] if cameras is None else spec["cameras"][:cameras]
        images = {
            cam.split("observation.images.")[-1]: torch.rand(3, spec["resize"][1], spec["resize"][0], generator=g)
            for cam in cams
        }
        state = torch.rand(int(getattr(self.config, "proprio_dim", None) or 8), generator=g)
        return self.make_frame(images, state, "profile")

    def profile(self, iters: int = 5, warmup: int = 3, cameras: int | None = None, seed: int = 0) -> dict[str, Any]:
        """Wall-time latency of :meth:`predict_action_chunk` on a synthetic frame, engine as configured."""
        frame = self._profile_frame(cameras, seed)
        for _ in range(warmup):
            self.predict_action_chunk(frame)
        cuda = str(self.device).startswith("cuda") and torch.cuda.is_available()
        if cuda:
            torch.cuda.synchronize()
        samples = []
        for _ in range(iters):
            t0 = time.perf_counter()
            self.predict_action_chunk(frame)
            if cuda:
                torch.cuda.synchronize()
            samples.append((time.perf_counter() - t0) * 1e3)
        spec = self.describe()
        cams = spec["cameras"] if cameras is None else spec["cameras"][:cameras]
        report: dict[str, Any] = {
            "wall_ms": float(np.mean(samples)),
            "p50_ms": float(np.percentile(samples, 50)),
            "p95_ms": float(np.percentile(samples, 95)),
            "iters": iters,
            "cameras": len(cams),
            "spec": spec,
            "phases": self._profile_phases(iters=iters, warmup=warmup, cameras=cameras, seed=seed),
        }
        path = "hip-graph" if getattr(self, "graph_enabled", False) else "eager"
        logging.getLogger(f"tybok.{spec.get('model_type')}").info(
            f"profile: device={self.device} path={path} cameras={report['cameras']} iters={iters} "
            f"wall {report['wall_ms']:.2f} ms/iter (p50 {report['p50_ms']:.2f}, p95 {report['p95_ms']:.2f})"
        )
        return report

    def _profile_phases(self, iters: int = 5, warmup: int = 3, cameras: int | None = None, seed: int = 0) -> dict[str, float]:
        return {}

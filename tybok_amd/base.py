"""The engine interface the serving side of tybok programs against.

The reference's gateway and worker only touch ``PolicyEngine.{describe, select_action,
predict_action_chunk, validate, profile, make_frame}`` (tybok/base.py:50-235); a backend registered
under the same model name, with the same constructor keywords and the same return types, is a
drop-in for them.  The reference's ``compile_region`` (torch.compile plumbing) has no counterpart: the
HIP tiers take its place and the backends reject ``compile_model=True``.
"""

from __future__ import annotations

import abc
import logging
import time
from collections import deque
from collections.abc import Mapping, Sequence
from typing import Any

import numpy as np
import torch

from .graph import CaptureSession, GraphRunner

log = logging.getLogger("tybok.engine")

_IMAGE_PREFIX = "observation.images."
_CHANNEL_COUNTS = (1, 3, 4)


def _resolve_device(device: str) -> str:
    return ("cuda" if torch.cuda.is_available() else "cpu") if device == "auto" else device


def _as_chw_float(name: str, image: Any) -> torch.Tensor:
    """One camera image as a contiguous fp32 ``(C, H, W)`` tensor; ``(H, W, C)`` input is transposed."""
    if isinstance(image, np.ndarray):
        image = torch.from_numpy(image)
    if not isinstance(image, torch.Tensor):
        raise TypeError(f"image {name} must be a tensor or ndarray")
    channels_last = image.ndim == 3 and image.shape[0] not in _CHANNEL_COUNTS
    return (image.permute(2, 0, 1) if channels_last else image).float().contiguous()


def _as_state(state: Any) -> torch.Tensor:
    if isinstance(state, torch.Tensor):
        return state.float().contiguous()
    return torch.from_numpy(np.asarray(state, dtype=np.float32)).contiguous()


class PolicyEngine(abc.ABC):
    """Base class of the policy backends (inference only)."""

    config: Any
    compile_model: bool
    graph_enabled: bool

    def __init__(self, checkpoint_dir: str, device: str = "auto", **kwargs):
        self.checkpoint_dir = checkpoint_dir
        self.device = _resolve_device(device)
        self.compiled_regions: list[str] = []  # kept for callers that report it; always empty here
        if str(self.device).startswith("cuda") and torch.device(self.device).index is not None:
            torch.cuda.set_device(torch.device(self.device))

    # ------------------------------------------------------------------ what a backend implements
    @abc.abstractmethod
    def describe(self) -> dict[str, Any]:
        """``{"model_type", "cameras", "resize": [W, H], "action_dim", "chunk_size", ...}``."""

    @abc.abstractmethod
    def select_action(self, frame: dict[str, Any], noise: torch.Tensor | None = None) -> np.ndarray:
        """The next action ``(action_dim,)`` for one observation frame."""

    @abc.abstractmethod
    def predict_action_chunk(self, frame: dict[str, Any], noise: torch.Tensor | None = None) -> np.ndarray:
        """A whole chunk ``(chunk_size, action_dim)`` for one observation frame."""

    @abc.abstractmethod
    def validate(self, reference_dir: str) -> dict[str, float]:
        """Per-component errors of this backend against a dump directory of the reference."""

    def supports_rtc(self) -> bool:
        return False

    # ------------------------------------------------------------------ frames
    def make_frame(self, images: Mapping[str, torch.Tensor | np.ndarray], state: torch.Tensor | np.ndarray | Sequence[float], task: str) -> dict[str, Any]:
        """The raw frame dict of a request: fp32 ``(C, H, W)`` images in [0, 1] under
        ``observation.images.<camera>``, a 1-D fp32 ``observation.state`` and the ``task`` string."""
        frame: dict[str, Any] = {_IMAGE_PREFIX + name: _as_chw_float(name, image) for name, image in images.items()}
        frame["observation.state"] = _as_state(state)
        frame["task"] = task
        return frame

    def _camera_names(self, cameras: int | None) -> list[str]:
        names = [c.split(_IMAGE_PREFIX)[-1] for c in self.describe()["cameras"]]
        return names if cameras is None else names[:cameras]

    def _profile_frame(self, cameras: int | None = None, seed: int = 0) -> dict[str, Any]:
        """A seeded synthetic frame: uniform images for the configured (or the first ``cameras``)
        cameras, drawn in camera order, then a uniform state -- the draw order of the reference, whose
        tests feed ``_profile_frame(seed=...)`` to the engines they compare."""
        width, height = self.describe()["resize"]
        rng = torch.Generator().manual_seed(seed)
        images = {}
        for name in self._camera_names(cameras):
            images[name] = torch.rand(3, height, width, generator=rng)
        state_dim = int(getattr(self.config, "proprio_dim", None) or 8)
        return self.make_frame(images, torch.rand(state_dim, generator=rng), "profile")

    # ------------------------------------------------------------------ start-up and timing
    def _sync(self) -> None:
        if str(self.device).startswith("cuda") and torch.cuda.is_available():
            torch.cuda.synchronize()

    def _warmup(self) -> None:
        """One inference on an all-zero frame, so lazy initialisation never lands on a request."""
        width, height = self.describe()["resize"]
        started = time.perf_counter()
        blank = {name: torch.zeros(3, height, width) for name in self._camera_names(None)}
        self.predict_action_chunk(self.make_frame(blank, torch.zeros(8), "warmup"))
        self._sync()
        log.info("warmup done in %.1fs", time.perf_counter() - started)

    def profile(self, iters: int = 5, warmup: int = 3, cameras: int | None = None, seed: int = 0) -> dict[str, Any]:
        """Wall-clock latency of :meth:`predict_action_chunk` on a synthetic frame, engine as configured."""
        frame = self._profile_frame(cameras, seed)
        for _ in range(warmup):
            self.predict_action_chunk(frame)
        self._sync()
        wall_ms = np.empty(iters, dtype=np.float64)
        for i in range(iters):
            started = time.perf_counter()
            self.predict_action_chunk(frame)
            self._sync()
            wall_ms[i] = (time.perf_counter() - started) * 1e3
        spec = self.describe()
        report: dict[str, Any] = {
            "wall_ms": float(wall_ms.mean()),
            "p50_ms": float(np.percentile(wall_ms, 50)),
            "p95_ms": float(np.percentile(wall_ms, 95)),
            "iters": iters,
            "cameras": len(self._camera_names(cameras)),
            "spec": spec,
            "phases": self._profile_phases(iters=iters, warmup=warmup, cameras=cameras, seed=seed),
        }
        logging.getLogger(f"tybok.{spec.get('model_type')}").info(
            "profile: device=%s path=%s cameras=%d iters=%d wall %.2f ms/iter (p50 %.2f, p95 %.2f)",
            self.device, "hip-graph" if getattr(self, "graph_enabled", False) else "eager", report["cameras"], iters,
            report["wall_ms"], report["p50_ms"], report["p95_ms"],
        )  # fmt: skip
        return report

    def _profile_phases(self, iters: int = 5, warmup: int = 3, cameras: int | None = None, seed: int = 0) -> dict[str, float]:
        """Per-phase timings a backend may add to :meth:`profile`'s report."""
        return {}


class ChunkRuntime:
    """What the two flow-matching backends share once their model is built: the seeded noise source,
    the queue ``select_action`` drains, recorded shapes, and the order of the start-up steps.  A backend
    provides ``_infer(batch, noise)``, ``_batch_from_frame(frame)``, ``_capture_graph(key, request)``, an
    ``unnormalizer`` and a ``config`` with ``chunk_size``, ``n_action_steps``, ``max_action_dim`` and
    ``action_feature_shape``."""

    def _init_sampling(self, seed: int | None) -> None:
        self.seed = seed
        self._noise_gen = None if seed is None else torch.Generator(device=self.device).manual_seed(int(seed))
        self._action_queue: deque[torch.Tensor] = deque(maxlen=self.config.n_action_steps)

    def _init_graphs(self, graph: bool, label: str, logger: logging.Logger) -> None:
        self.graph_requested = bool(graph)
        self.graph_enabled = self.graph_requested and str(self.device).startswith("cuda")
        self._sess = CaptureSession(self.device)
        self._graph_runner = GraphRunner(self._capture_graph, self.device, label=label, logger=logger)

    def _start(self, *, warmup: bool, graph_keys: Sequence[Any], profile: bool, logger: logging.Logger) -> None:
        """Start-up in the reference's order: one warm-up inference, the shapes named on the command
        line recorded (none recordable: back to eager, loudly), an optional latency report."""
        if warmup:
            self._warmup()
        if self.graph_enabled and not self._graph_runner.precapture(list(graph_keys)):
            logger.warning("no requested shape could be recorded as a graph; running eagerly")
            self.graph_enabled = False
            self._graph_runner.forget()
        if profile:
            try:
                self.profile()
            except Exception as exc:  # noqa: BLE001 - a diagnostic must not stop the server from starting
                logger.warning("profile failed: %s", exc)

    # ------------------------------------------------------------------ noise and outputs
    def _sample_noise(self, out: torch.Tensor | None = None) -> torch.Tensor:
        shape = (1, self.config.chunk_size, self.config.max_action_dim)
        return torch.normal(0.0, 1.0, size=shape, dtype=torch.float32, device=self.device, generator=self._noise_gen, out=out)

    def _prepare_noise(self, noise: torch.Tensor | None) -> torch.Tensor | None:
        """A caller's noise on the device in fp32, at the caller's width (at most the model's action width):
        :meth:`_pad_noise` widens it for the eager path, a recorded shape takes it as it is
        (``StaticCall.store_leading``)."""
        if noise is None:
            return None
        if noise.shape[-1] > self.config.max_action_dim:
            raise ValueError(f"noise has {noise.shape[-1]} action columns, the model {self.config.max_action_dim}")
        return noise.to(self.device, dtype=torch.float32)

    def _pad_noise(self, noise: torch.Tensor) -> torch.Tensor:
        """Zero-padded to the model's action width."""
        missing = self.config.max_action_dim - noise.shape[-1]
        return torch.nn.functional.pad(noise, (0, missing)) if missing else noise

    def _robot_actions(self, frame: dict[str, Any], noise: torch.Tensor | None) -> torch.Tensor:
        """Normalised actions ``[1, chunk, action_dim]`` of one request (the padded columns dropped)."""
        actions = self._infer(self._batch_from_frame(frame), self._prepare_noise(noise))
        return actions[:, :, : self.config.action_feature_shape[0]]

    def _to_robot_units(self, actions: torch.Tensor) -> np.ndarray:
        return self.unnormalizer.unnormalize(actions, "action", "ACTION").cpu().numpy()[0]

    def _next_queued_action(self, frame: dict[str, Any], noise: torch.Tensor | None) -> np.ndarray:
        """``select_action``: infer a chunk only when the queue of the previous one is empty."""
        if not self._action_queue:
            # (the queue outlives this request: it gets its own copy, not a view of a graph's static output)
            self._action_queue.extend(self._robot_actions(frame, noise).transpose(0, 1)[: self.config.n_action_steps].clone())
        return self._to_robot_units(self._action_queue.popleft())

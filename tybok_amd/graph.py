"""hipGraph plumbing shared by the backends, with the reference's contract
(tybok/graph.py:60-251): graph keys start with the number of image inputs, warm-up on a side
stream before capture, lazy capture on first sight, startup pre-capture that tolerates a failing
key, and input copies on a dedicated stream joined by one event before the replay.

On PyTorch-ROCm ``torch.cuda.CUDAGraph`` is a hipGraph; the HIP kernels of this package are
launched on torch's current stream, so stream capture records them like any torch op.
"""

from __future__ import annotations

import contextlib
import logging
from collections.abc import Callable, Hashable, Iterable
from typing import Any

import torch

log = logging.getLogger("tybok.graph")

GRAPH_CAMERAS_HELP = (
    "comma-separated image counts to pre-capture at startup, e.g. '2,3' "
    "(default: the configured image count; other counts are captured lazily)"
)


def camera_counts(graph_cameras: Iterable[int] | None, *, default: int, max_images: int) -> tuple[int, ...]:
    """Image counts to pre-capture: the valid, de-duplicated, sorted entries of ``--graph-cameras``,
    else the (clamped) configured count."""
    hi = max(1, int(max_images))
    counts = sorted({int(n) for n in (graph_cameras or ()) if 1 <= int(n) <= hi})
    return tuple(counts) if counts else (min(max(1, int(default)), hi),)


class CaptureSession:
    """Warm-up (side stream, joined back) + capture, both under ``inference_mode``."""

    def __init__(self, device: str | torch.device, warmup_iters: int = 3):
        self.device = torch.device(device)
        self.warmup_iters = int(warmup_iters)

    def prime(self, fn: Callable[[], Any], iters: int | None = None) -> None:
        iters = self.warmup_iters if iters is None else int(iters)
        main = torch.cuda.current_stream(self.device)
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(main)
        with torch.inference_mode(), torch.cuda.stream(side):
            for _ in range(iters):
                fn()
        main.wait_stream(side)

    @staticmethod
    def capture(fn: Callable[[], Any]) -> torch.cuda.CUDAGraph:
        graph = torch.cuda.CUDAGraph()
        with torch.inference_mode(), torch.cuda.graph(graph):
            fn()
        return graph

    def prime_and_capture(self, fn: Callable[[], Any]) -> torch.cuda.CUDAGraph:
        self.prime(fn)
        return self.capture(fn)

    def sync(self) -> None:
        torch.cuda.synchronize()


class GraphRunner:
    """``key -> entry`` registry plus the per-request copy/replay primitives."""

    def __init__(self, capture_fn: Callable[[Hashable, Any], Any], device, *, label: str = "graph", logger=None):
        self.device = torch.device(device)
        self.label = label
        self._capture_fn = capture_fn
        self._log = logger or log
        self._entries: dict[Hashable, Any] = {}
        self.copy_stream: torch.cuda.Stream | None = None
        self.ev_in: torch.cuda.Event | None = None

    def __bool__(self) -> bool:
        return bool(self._entries)

    def __contains__(self, key: Hashable) -> bool:
        return key in self._entries

    def __len__(self) -> int:
        return len(self._entries)

    def keys(self):
        return self._entries.keys()

    @property
    def entries(self) -> dict[Hashable, Any]:
        return self._entries

    def get(self, key: Hashable, default: Any = None) -> Any:
        return self._entries.get(key, default)

    def set(self, key: Hashable, entry: Any) -> None:
        self._entries[key] = entry

    def clear(self) -> None:
        self._entries.clear()

    def entry(self, key: Hashable, request: Any = None) -> Any:
        got = self._entries.get(key)
        if got is None:
            got = self._capture_fn(key, request)
            self._entries[key] = got
        return got

    def precapture(self, keys: Iterable[Hashable]) -> bool:
        """Capture ``keys`` now; True if at least one succeeded (a failing key is logged and skipped)."""
        ok = False
        for key in keys:
            try:
                self.set(key, self._capture_fn(key, None))
                ok = True
            except Exception as e:  # noqa: BLE001 - a failed shape is a result, not a crash
                self._log.warning(f"{self.label} capture for {key} failed ({e}); that shape falls back to eager")
        return ok

    @contextlib.contextmanager
    def copy_inputs(self):
        """Fork the main stream into the copy stream for the input copies (joined by :meth:`wait_inputs`)."""
        if self.copy_stream is None:
            self.copy_stream = torch.cuda.Stream(device=self.device)
            self.ev_in = torch.cuda.Event()
        main = torch.cuda.current_stream(self.device)
        with torch.cuda.stream(self.copy_stream):
            self.copy_stream.wait_stream(main)
            yield self.copy_stream
            assert self.ev_in is not None
            self.ev_in.record(self.copy_stream)

    def wait_inputs(self) -> None:
        assert self.ev_in is not None, "copy_inputs() must run before wait_inputs()"
        torch.cuda.current_stream(self.device).wait_event(self.ev_in)

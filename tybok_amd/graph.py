"""hipGraph plumbing shared by the two backends.

Behaviour follows the reference's helper of the same name (tybok/graph.py:60-251): a captured graph
is looked up by a key whose first element is the number of image inputs; a shape is run eagerly a
few times on a forked stream before it is recorded; shapes named at start-up are recorded then and a
shape that fails to record is reported and left to the eager path; any other shape is recorded the
first time a request needs it; per request the inputs are copied into the graph's static tensors
(optionally on a stream of their own that the replay waits for through one event, as the reference does).

On PyTorch-ROCm ``torch.cuda.CUDAGraph`` is a hipGraph, and this package's HIP kernels are launched
on torch's current stream, so stream capture records them exactly like torch's own launches.
"""

from __future__ import annotations

import logging
from collections.abc import Callable, Hashable, Iterable, Iterator
from contextlib import contextmanager
from typing import Any

import torch

_LOG = logging.getLogger("tybok.graph")


def camera_counts(graph_cameras: Iterable[int] | None, *, default: int, max_images: int) -> tuple[int, ...]:
    """Image counts to record at start-up: the valid, de-duplicated, sorted entries of ``--graph-cameras``,
    else the (clamped) configured count."""
    hi = max(1, int(max_images))
    counts = sorted({int(n) for n in (graph_cameras or ()) if 1 <= int(n) <= hi})
    return tuple(counts) if counts else (min(max(1, int(default)), hi),)


class CaptureSession:
    """Turns a zero-argument callable into a replayable graph: eager passes first, then the recording."""

    def __init__(self, device: str | torch.device, warmup_iters: int = 3):
        self.device = torch.device(device)
        self.warmup_iters = max(0, int(warmup_iters))

    def prime(self, fn: Callable[[], Any], iters: int | None = None) -> None:
        """Eager passes on a stream forked from the current one (lazy initialisation, workspace and
        allocator warm-up happen here, outside any recording); the current stream waits for them."""
        current = torch.cuda.current_stream(self.device)
        fork = torch.cuda.Stream(device=self.device)
        fork.wait_stream(current)
        with torch.inference_mode(), torch.cuda.stream(fork):
            for _ in range(self.warmup_iters if iters is None else max(0, int(iters))):
                fn()
        current.wait_stream(fork)

    def capture(self, fn: Callable[[], Any]) -> torch.cuda.CUDAGraph:
        recorded = torch.cuda.CUDAGraph()
        with torch.inference_mode(), torch.cuda.graph(recorded):
            fn()
        return recorded

    def prime_and_capture(self, fn: Callable[[], Any]) -> torch.cuda.CUDAGraph:
        self.prime(fn)
        return self.capture(fn)


class StaticCall:
    """One recorded call ``output <- fn(**inputs)``: the static tensors it reads (by keyword; a value
    may be a list of tensors), the static tensor it writes, and the graph that replays it."""

    def __init__(self, output: torch.Tensor, **inputs: Any):
        self.inputs = inputs
        self.output = output
        self.graph: torch.cuda.CUDAGraph | None = None

    def record(self, session: CaptureSession, fn: Callable[..., torch.Tensor]) -> "StaticCall":
        def body() -> None:
            self.output.copy_(fn(**self.inputs))

        self.graph = session.prime_and_capture(body)
        torch.cuda.synchronize()  # a failed recording surfaces here, not at the first request
        return self

    def store(self, **values: Any) -> None:
        """Copy a request's values into the static tensors of the same names (on the current stream)."""
        for name, value in values.items():
            slot = self.inputs[name]
            getattr(self, "_stored_width", {}).pop(name, None)
            if isinstance(slot, (list, tuple)):
                if len(value) != len(slot):
                    raise ValueError(f"{name}: {len(value)} tensors for {len(slot)} static slots")
                for dst, src in zip(slot, value):
                    dst.copy_(src)
            else:
                slot.copy_(value)

    def store_leading(self, **values: torch.Tensor) -> None:
        """:meth:`store` for values that may be narrower than their static tensor in the last dimension: the value
        goes into the leading columns and the rest stays zero (zeroed again only after a wider value was stored),
        which is what zero-padding the value first and copying it whole would leave -- with one launch, not three."""
        if not hasattr(self, "_stored_width"):
            self._stored_width: dict[str, int] = {}
        for name, value in values.items():
            slot = self.inputs[name]
            width = int(value.shape[-1])
            if value.shape[:-1] != slot.shape[:-1] or width > slot.shape[-1]:
                raise ValueError(f"{name}: {tuple(value.shape)} does not fit the static {tuple(slot.shape)}")
            if width == slot.shape[-1]:
                slot.copy_(value)
            else:
                if self._stored_width.get(name, slot.shape[-1]) > width:  # (the first store: whatever recording left there)
                    slot[..., width:].zero_()
                slot[..., :width].copy_(value)
            self._stored_width[name] = width

    def store_owned(self, **values: Any) -> None:
        """:meth:`store` for tensors the backend owns and never changes in place (cached token ids, all-true
        masks): a value that is the very object stored last time is not copied again."""
        if not hasattr(self, "_last_owned"):
            self._last_owned: dict[str, Any] = {}
        for name, value in values.items():
            objects = tuple(value) if isinstance(value, (list, tuple)) else (value,)
            last = self._last_owned.get(name, ())
            if len(last) != len(objects) or any(a is not b for a, b in zip(last, objects)):
                self.store(**{name: value})
                self._last_owned[name] = objects

    def forget_leading(self, *names: str) -> None:
        """The static tensors ``names`` were written in full by something else (noise drawn in place): the next
        :meth:`store_leading` of a narrower value clears the columns behind it."""
        for name in names:
            getattr(self, "_stored_width", {}).pop(name, None)

    def forget_owned(self, *names: str) -> None:
        """The static tensors ``names`` were overwritten by a plain :meth:`store`: the next
        :meth:`store_owned` of those names copies again."""
        for name in names:
            getattr(self, "_last_owned", {}).pop(name, None)

    def replay(self, *, copy: bool = True) -> torch.Tensor:
        """Run the graph.  By default the result is copied out so that the next replay cannot overwrite
        it; ``copy=False`` returns the static tensor itself, for callers that finish with it (or copy it)
        before they replay again."""
        if self.graph is None:
            raise RuntimeError("replay() before record()")
        self.graph.replay()
        return self.output.clone() if copy else self.output


class GraphRunner:
    """Recorded shapes by key, and the two-stream hand-over of a request's inputs.

    ``record(key, request)`` is the backend's function that builds static tensors for ``key``, records
    the graph and returns whatever the backend wants to keep for replays (an "entry")."""

    def __init__(
        self, record: Callable[[Hashable, Any], Any], device, *, label: str = "graph", logger: logging.Logger | None = None,
        input_stream: bool = False,
    ):  # fmt: skip
        self.device = torch.device(device)
        self.label = label
        # The reference copies a request's inputs on a stream of their own and joins it to the replay with
        # one event.  The engine API is synchronous (one request at a time, the result returned to the
        # host), so nothing can overlap with those copies; on this stack the fork / join costs 0.1 ms per
        # request, and the copies run on the current stream unless ``input_stream`` asks for the other way.
        self.use_input_stream = bool(input_stream)
        self._record = record
        self._log = logger if logger is not None else _LOG
        self._shapes: dict[Hashable, Any] = {}
        self._input_stream: torch.cuda.Stream | None = None
        self._inputs_ready: torch.cuda.Event | None = None

    # -- recorded shapes ------------------------------------------------------------------------
    def __bool__(self) -> bool:  # "is there anything to replay"
        return len(self._shapes) > 0

    def keys(self):
        return self._shapes.keys()

    def forget(self) -> None:
        """Drop every recorded shape (the backend is going back to the eager path)."""
        self._shapes.clear()

    def entry(self, key: Hashable, request: Any = None) -> Any:
        """The entry of ``key``, recording it now if this is the first request of that shape."""
        if key not in self._shapes:
            self._shapes[key] = self._record(key, request)
        return self._shapes[key]

    def precapture(self, keys: Iterable[Hashable]) -> bool:
        """Record every key of ``keys`` that can be recorded; False if none could."""
        recorded = 0
        for key in keys:
            try:
                self._shapes[key] = self._record(key, None)
            except Exception as exc:  # noqa: BLE001 - the shape simply stays on the eager path
                self._log.warning("%s: recording %s failed (%s); requests of that shape run eagerly", self.label, key, exc)
            else:
                recorded += 1
        return recorded > 0

    # -- inputs of one request ------------------------------------------------------------------
    @contextmanager
    def copy_inputs(self) -> Iterator[torch.cuda.Stream]:
        """Inside the block, copies into the static tensors run on the input stream (ordered after
        everything already queued on the current stream); leaving it marks the inputs ready."""
        if not self.use_input_stream:
            yield torch.cuda.current_stream(self.device)
            return
        if self._input_stream is None:
            self._input_stream = torch.cuda.Stream(device=self.device)
            self._inputs_ready = torch.cuda.Event()
        self._input_stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(self._input_stream):
            yield self._input_stream
            self._inputs_ready.record(self._input_stream)

    def wait_inputs(self) -> None:
        """Order the current stream (the replay) after the copies of the last :meth:`copy_inputs` block."""
        if not self.use_input_stream:
            return
        if self._inputs_ready is None:
            raise RuntimeError("wait_inputs() called before any copy_inputs() block")
        torch.cuda.current_stream(self.device).wait_event(self._inputs_ready)

"""Stream-dependency wrapper returned by dispatch (DeepEP's ``EventOverlap`` shape).

Semantics follow the reference (pcie_ep/utils/event.py:12-100): waiting enqueues
a device-side wait on the current stream, never blocks the CPU, records the
retained tensors with the caching allocator, tells the owning buffer which
stream consumes its output pool, and runs an optional one-shot epilogue hook.
"""

from __future__ import annotations

from typing import Any, Callable, Optional

import torch


def record_tensors(value: Any, stream: Any) -> None:
    """``record_stream`` every CUDA tensor nested in ``value``; other objects are ignored."""
    if isinstance(value, torch.Tensor):
        if value.is_cuda:
            value.record_stream(stream)
    elif isinstance(value, dict):
        for item in value.values():
            record_tensors(item, stream)
    elif isinstance(value, (list, tuple)):
        for item in value:
            record_tensors(item, stream)


class EventOverlap:
    def __init__(self, event: Any = None, extra_tensors: Any = None, on_wait: Optional[Callable[[Any], None]] = None) -> None:
        self.event = event
        self.extra_tensors = extra_tensors
        self.hook_after_wait: Optional[Callable[[], Any]] = None
        self._on_wait = on_wait
        self._release_on_exit = False

    def current_stream_wait(self, release_handle: bool = False) -> Any:
        if self.event is None:
            raise RuntimeError("The event has already been released")
        stream = torch.cuda.current_stream()
        stream.wait_event(self.event)
        record_tensors(self.extra_tensors, stream)
        if self._on_wait is not None:
            self._on_wait(stream)
        hook, self.hook_after_wait = self.hook_after_wait, None
        result = hook() if hook is not None else None
        if release_handle:
            self.event = self.extra_tensors = self._on_wait = None
        return result

    def wait(self) -> Any:
        return self.current_stream_wait()

    def register_hook_after_wait(self, hook_after_wait: Callable[[], Any]) -> None:
        if self.hook_after_wait is not None:
            raise RuntimeError("An epilogue hook is already registered")
        self.hook_after_wait = hook_after_wait

    def __call__(self, release_handle: bool = False) -> "EventOverlap":
        self._release_on_exit = release_handle
        return self

    def __enter__(self) -> "EventOverlap":
        return self

    def __exit__(self, exc_type: Any, exc_value: Any, traceback: Any) -> None:
        release, self._release_on_exit = self._release_on_exit, False
        if self.event is not None:
            self.current_stream_wait(release)

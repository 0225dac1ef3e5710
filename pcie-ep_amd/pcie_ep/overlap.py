"""The stream dependency a dispatch hands back (DeepEP's ``EventOverlap`` shape).

Contract, as the reference documents it (pcie_ep/utils/event.py:12-100; API.md):
waiting makes the *current* stream wait for the dispatch on the device and never
blocks the CPU; tensors kept alive for the dispatch are recorded on the waiting
stream; the owning buffer learns which stream consumes its result pool; a hook
registered by a deferred dispatch runs on the first wait only; after a release
the object is spent.

Implementation: the object is a small state holder around three optional
parts — the device event, the things to keep alive, and a "consumer seen"
callback — and one operation, ``_attach(stream)``, that applies all of them to
a stream.  Waiting, the call form and the context-manager form are thin
wrappers over ``_attach``.
"""

from __future__ import annotations

from typing import Any, Callable, Iterator, Optional

import torch


def _cuda_tensors(value: Any) -> Iterator[torch.Tensor]:
    """Every CUDA tensor nested in dicts / lists / tuples of ``value``."""
    stack = [value]
    while stack:
        item = stack.pop()
        if isinstance(item, torch.Tensor):
            if item.is_cuda:
                yield item
        elif isinstance(item, dict):
            stack.extend(item.values())
        elif isinstance(item, (list, tuple)):
            stack.extend(item)


def record_tensors(value: Any, stream: Any) -> None:
    """Tell the caching allocator that ``stream`` uses every CUDA tensor in ``value``."""
    for tensor in _cuda_tensors(value):
        tensor.record_stream(stream)


class EventOverlap:
    def __init__(self, event: Any = None, extra_tensors: Any = None, on_wait: Optional[Callable[[Any], None]] = None) -> None:
        self.event = event
        self.extra_tensors = extra_tensors
        self.hook_after_wait: Optional[Callable[[], Any]] = None
        self._consumer_seen = on_wait
        self._release_when_left = False

    # ---- the one operation ------------------------------------------------------------
    def _attach(self, stream: Any) -> Any:
        """Order ``stream`` after the event, keep the retained tensors valid for
        it, report it as a consumer and run the pending hook (once)."""
        stream.wait_event(self.event)
        record_tensors(self.extra_tensors, stream)
        if self._consumer_seen is not None:
            self._consumer_seen(stream)
        pending, self.hook_after_wait = self.hook_after_wait, None
        return None if pending is None else pending()

    def _spend(self) -> None:
        self.event = self.extra_tensors = self._consumer_seen = None

    # ---- public forms -------------------------------------------------------------------
    def stream_wait(self, stream: Any) -> Any:
        """Order ``stream`` (rather than the current stream) after the event."""
        if self.event is None:
            raise RuntimeError("The event has already been released")
        return self._attach(stream)

    def current_stream_wait(self, release_handle: bool = False) -> Any:
        if self.event is None:
            raise RuntimeError("The event has already been released")
        outcome = self._attach(torch.cuda.current_stream())
        if release_handle:
            self._spend()
        return outcome

    wait = current_stream_wait

    def register_hook_after_wait(self, hook_after_wait: Callable[[], Any]) -> None:
        if self.hook_after_wait is not None:
            raise RuntimeError("An epilogue hook is already registered")
        self.hook_after_wait = hook_after_wait

    def __call__(self, release_handle: bool = False) -> "EventOverlap":
        """``with overlap(release_handle=True): ...`` releases when the block is left."""
        self._release_when_left = bool(release_handle)
        return self

    def __enter__(self) -> "EventOverlap":
        return self

    def __exit__(self, *exc_info: Any) -> None:
        release, self._release_when_left = self._release_when_left, False
        if self.event is not None:  # a spent object leaves silently
            self.current_stream_wait(release)

"""Streams restricted to a subset of the compute units.

The dispatch kernels poll and move rows for milliseconds on a few dozen
wavefronts.  A compute kernel that runs meanwhile and spreads persistently over
all compute units waits for the few units it shares with those wavefronts.  HIP
can confine a stream's kernels to a set of compute units
(``hipExtStreamCreateWithCUMask``); giving the dispatch one set and the compute
stream the complement removes the interaction.  The reference has no
counterpart (its answer to the same concern is a small SM footprint,
docs/pcie-ep/dispatch-profiling-20261029.md:103).

The mask is a bit array over the device's compute units; the driver deals the
bits round-robin over the XCDs and shader engines, so a run of N consecutive
bits is spread evenly over the chip.
"""

from __future__ import annotations

import ctypes as C
from typing import Any, Tuple

import torch

_hip = None


def _runtime() -> C.CDLL:
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so")
        _hip.hipExtStreamCreateWithCUMask.restype = C.c_int
        _hip.hipExtStreamCreateWithCUMask.argtypes = [C.POINTER(C.c_void_p), C.c_uint32, C.POINTER(C.c_uint32)]
    return _hip


class MaskedStream:
    """A HIP stream whose kernels run only on compute units ``[first, first + count)``
    of the mask order; ``.stream`` is usable wherever a ``torch.cuda.Stream`` is.

    The HIP stream is created once per (device, range) and lives until the
    process ends.  It must not be destroyed earlier: PyTorch's caching allocator
    remembers every stream a tensor was recorded on or allocated on and records
    an event on it when the tensor is freed, which may be long after the code
    that used the stream is done; on a destroyed stream that call crashes."""

    _cache: dict = {}

    def __new__(cls, device: int, count: int, first: int = 0) -> "MaskedStream":
        key = (device, first, count)
        existing = cls._cache.get(key)
        if existing is not None:
            return existing
        instance = super().__new__(cls)
        instance._create(device, count, first)
        cls._cache[key] = instance
        return instance

    def _create(self, device: int, count: int, first: int) -> None:
        total = torch.cuda.get_device_properties(device).multi_processor_count
        if not isinstance(count, int) or not isinstance(first, int) or count < 1 or first < 0 or first + count > total:
            raise ValueError(f"compute-unit range [{first}, {first + count}) does not fit the device's {total} units")
        words = (total + 31) // 32
        mask = (C.c_uint32 * words)()
        for unit in range(first, first + count):
            mask[unit // 32] |= 1 << (unit % 32)
        handle = C.c_void_p()
        with torch.cuda.device(device):
            status = _runtime().hipExtStreamCreateWithCUMask(C.byref(handle), words, mask)
        if status != 0 or not handle.value:
            raise RuntimeError(f"hipExtStreamCreateWithCUMask failed with status {status}")
        self._handle = handle
        self.units: Tuple[int, int] = (first, first + count)
        self.stream: Any = torch.cuda.ExternalStream(handle.value, device=torch.device("cuda", device))

    def close(self) -> None:
        """Wait for the stream's work; the stream itself stays (see the class comment)."""
        self.stream.synchronize()


def masked_stream(count: int, first: int = 0, device: Any = None) -> MaskedStream:
    """A stream on ``count`` compute units starting at ``first`` (mask order) of the current device."""
    index = torch.cuda.current_device() if device is None else torch.device(device).index
    return MaskedStream(index, count, first)

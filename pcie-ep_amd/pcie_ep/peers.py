"""Python face of the host peer emulator: the CPU threads that play the other
logical ranks on the pinned rings.  It has no counterpart in the reference's
Python package (its peers are other processes); tests and benchmarks use it to
feed and drain the one real GPU."""

from __future__ import annotations

import ctypes as C
from typing import Dict, Optional

import numpy as np
import torch

from . import _native

(FAULT_NONE, FAULT_NO_COUNTS_READY, FAULT_NO_COUNTS_CONSUMED, FAULT_NO_LAST_ACK, FAULT_WRONG_SEQUENCE, FAULT_RANK_ORDINAL,
 FAULT_EXPERT_ORDINAL, FAULT_SLOT_RANGE) = range(8)


class PeerGroup:
    def __init__(self, runtime) -> None:
        self._runtime = runtime
        self._lib = _native.library()

    def set_source(self, rank: int, x: torch.Tensor, topk_idx: torch.Tensor, topk_weights: Optional[torch.Tensor] = None) -> None:
        """Inputs of logical rank ``rank`` for the following epochs (CPU tensors, copied)."""
        x = x.detach().cpu().contiguous()
        idx = topk_idx.detach().cpu().contiguous()
        if x.dtype != torch.bfloat16 or idx.dtype != torch.int64:
            raise ValueError("peer inputs must be BF16 payload and int64 routes")
        weights = topk_weights.detach().cpu().contiguous().float() if topk_weights is not None else None
        _native.check(self._lib.pcie_ep_peer_set_source(
            self._runtime.handle, rank, C.c_void_p(x.data_ptr()), C.c_void_p(idx.data_ptr()),
            C.c_void_p(weights.data_ptr()) if weights is not None else None, int(x.shape[0])))

    def start(self, epochs: int = 1, capture: bool = False, restage: bool = False, read_rows: bool = False) -> None:
        """Serve the next ``epochs`` dispatches.  ``capture`` keeps what the GPU sent,
        ``restage`` rewrites every source slot in every epoch (unchanged rows are
        otherwise left in place), ``read_rows`` makes the receivers read whole rows."""
        flags = (1 if capture else 0) | (2 if restage else 0) | (4 if read_rows else 0)
        _native.check(self._lib.pcie_ep_peers_start(self._runtime.handle, epochs, flags), invalid=RuntimeError)

    def wait_staged(self, timeout_ms: int = 60_000) -> None:
        _native.check(self._lib.pcie_ep_peers_wait_staged(self._runtime.handle, timeout_ms), invalid=RuntimeError)

    def wait(self, timeout_ms: int = 60_000) -> None:
        _native.check(self._lib.pcie_ep_peers_wait(self._runtime.handle, timeout_ms), invalid=RuntimeError)

    def cancel(self) -> None:
        _native.check(self._lib.pcie_ep_peers_cancel(self._runtime.handle))

    def inject_fault(self, rank: int, fault: int) -> None:
        _native.check(self._lib.pcie_ep_peers_inject_fault(self._runtime.handle, rank, fault))

    def captured(self, rank: int) -> Dict[str, np.ndarray]:
        """Rows rank ``rank`` received from the GPU during the last served epoch."""
        count = C.c_int64()
        _native.check(self._lib.pcie_ep_peer_captured_count(self._runtime.handle, rank, C.byref(count)))
        n, k = int(count.value), self._runtime.topk
        payload_bytes = int(self._runtime.sizes.payload_bytes)
        out = {
            "tokens": np.zeros(n, np.int32), "rank_ordinals": np.zeros(n, np.int32), "payload": np.zeros((n, payload_bytes), np.uint8),
            "scales": np.zeros(n, np.float32), "expert_idx": np.zeros((n, k), np.int32), "expert_ordinals": np.zeros((n, k), np.int32),
            "weights": np.zeros((n, k), np.float32), "masks": np.zeros(n, np.uint32),
        }
        order = ("tokens", "rank_ordinals", "payload", "scales", "expert_idx", "expert_ordinals", "weights", "masks")
        pointers = [C.c_void_p(out[name].ctypes.data) for name in order]
        _native.check(self._lib.pcie_ep_peer_captured_copy(self._runtime.handle, rank, *pointers))
        return out

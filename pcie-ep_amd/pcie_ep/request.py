"""Admission of one dispatch call: every check on the caller's arguments, done
once, for the eager path and for graph capture alike.

Only tensor *metadata* is looked at (device, dtype, shape, contiguity, version
counter); GPU memory is never read and nothing waits for the GPU.  What is
rejected, with which exception type and message, is the reference's contract
for ``dispatch`` (pcie_ep/buffers/ep.py:283-360) and ``capture_dispatch``
(pcie_ep/graph.py:116-170); the two differ in a few messages and in the upper
bound on the alignment, which is what ``_WORDING`` captures.

The outcome is a ``DispatchRequest``: the normalised inputs plus the native plan
of a cached layout (or ``None``), ready to be handed to the runtime.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import torch

# Per-mode wording and limits.
_WORDING = {
    "eager": {
        "alignment": (lambda a: a >= 1, "expert_alignment must be a positive integer"),
        "padding": "do_zero_padding is valid only with do_expand=True",
        "capacity": "Input token count exceeds the prepared capacity",
    },
    "graph": {
        "alignment": (lambda a: 1 <= a <= 256, "expert_alignment must be in [1,256]"),
        "padding": "do_zero_padding requires do_expand=True",
        "capacity": "Graph input exceeds the prepared capacity",
    },
}


@dataclass
class DispatchRequest:
    x: torch.Tensor
    routes: torch.Tensor
    weights: Optional[torch.Tensor]
    alignment: int
    expand: bool
    zero_padding: bool
    cached: Any            # the handle / cached layout the caller supplied, or None
    plan: Any              # its native plan, or None: the routing is computed by this dispatch
    stats_out: Optional[torch.Tensor] = None

    @property
    def inputs(self) -> tuple:
        return (self.x, self.routes, self.weights)


def require_tensor(tensor: Any, name: str, device: int, dtype: torch.dtype, shape: tuple) -> None:
    """``shape`` entries of ``None`` are free."""
    if not isinstance(tensor, torch.Tensor):
        raise TypeError(f"{name} must be a torch Tensor")
    if not tensor.is_cuda or tensor.device.index != device:
        raise ValueError(f"{name} must be on this buffer's CUDA device")
    if tensor.dtype != dtype or not tensor.is_contiguous():
        raise ValueError(f"{name} must be contiguous with dtype {dtype}")
    if tensor.ndim != len(shape) or any(want is not None and have != want for have, want in zip(tensor.shape, shape)):
        raise ValueError(f"{name} has shape {tuple(tensor.shape)}, expected {tuple(shape)}")


def admit(buffer: Any, mode: str, x: Any, topk_idx: Any, topk_weights: Any, *, handle: Any = None,
          expert_alignment: Optional[int] = None, do_expand: bool = False, do_zero_padding: bool = False,
          stats_out: Any = None) -> DispatchRequest:
    """Validate one call against ``buffer``'s prepared dimensions."""
    wording = _WORDING[mode]
    if handle is not None:
        if topk_idx is not None:
            raise ValueError("topk_idx must be None when a cached handle is supplied")
        topk_idx = handle.topk_idx  # raises when the routes were edited in place
    alignment = expert_alignment if expert_alignment is not None else (handle.expert_alignment if handle is not None else 1)
    alignment_ok, alignment_message = wording["alignment"]
    if not isinstance(alignment, int) or isinstance(alignment, bool) or not alignment_ok(alignment):
        raise ValueError(alignment_message)
    if do_zero_padding and not do_expand:
        raise ValueError(wording["padding"])
    require_tensor(x, "x", buffer.device, torch.bfloat16, (None, buffer.hidden))
    require_tensor(topk_idx, "topk_idx", buffer.device, torch.int64, (x.shape[0], buffer.num_topk))
    if x.shape[0] > buffer.num_max_tokens_per_rank:
        raise ValueError(wording["capacity"])
    if topk_weights is not None:
        require_tensor(topk_weights, "topk_weights", buffer.device, torch.float32, tuple(topk_idx.shape))
    if stats_out is not None:
        require_tensor(stats_out, "cumulative_local_expert_recv_stats", buffer.device, torch.int32,
                       (buffer.num_experts // buffer.num_ranks,))
    plan = handle.validate_cached(buffer, x, alignment, bool(do_expand)) if handle is not None else None
    return DispatchRequest(x, topk_idx, topk_weights, alignment, bool(do_expand), bool(do_zero_padding), handle, plan, stats_out)

"""FP8 wire helpers running the same gfx950 device code as the dispatch
(per-token amax/448 scale with a 2^-126 floor, E4M3FN round-to-nearest-even).
The reference ships CPU validation functions under this module name
(pcie_ep/quantization.py); here they are GPU entry points, and the CPU
restatement used for checking lives with the tests."""

from __future__ import annotations

import ctypes as C
from typing import Tuple

import torch

from . import _native


def quantize_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """BF16 [T,H] on the GPU -> (uint8 codes [T,H], float32 scales [T])."""
    if x.ndim != 2 or x.dtype != torch.bfloat16 or not x.is_cuda or not x.is_contiguous():
        raise ValueError("FP8 quantization expects a contiguous CUDA BF16 [T,H] tensor")
    codes = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    scales = torch.empty(x.shape[0], dtype=torch.float32, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    _native.check(_native.library().pcie_ep_quantize_fp8(
        C.c_void_p(x.data_ptr()), C.c_void_p(codes.data_ptr()), C.c_void_p(scales.data_ptr()), x.shape[0], x.shape[1],
        C.c_void_p(stream)))
    return codes, scales


def dequantize_fp8(codes: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    if codes.dtype != torch.uint8 or codes.ndim != 2 or not codes.is_cuda or not codes.is_contiguous():
        raise ValueError("FP8 codes must be a contiguous CUDA uint8 [T,H] tensor")
    if scales.shape != codes.shape[:1] or scales.dtype != torch.float32 or not scales.is_contiguous():
        raise ValueError("FP8 scales must be FP32 [T]")
    out = torch.empty(codes.shape, dtype=torch.bfloat16, device=codes.device)
    stream = torch.cuda.current_stream(codes.device).cuda_stream
    _native.check(_native.library().pcie_ep_dequantize_fp8(
        C.c_void_p(codes.data_ptr()), C.c_void_p(scales.data_ptr()), C.c_void_p(out.data_ptr()), codes.shape[0], codes.shape[1],
        C.c_void_p(stream)))
    return out

"""CPU oracle for the per-token FP8 (E4M3FN) wire format.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline``
leg may import this module; the product path never does.

Two independent restatements are kept so that each pins the other:

* ``quantize`` / ``dequantize`` / ``roundtrip`` follow the reference's PyTorch
  validation functions (pcie_ep/quantization.py:14-44): FP32 amax per row,
  ``scale = 1`` for an all-zero row else ``max(amax/448, FLT_MIN)``, multiply
  by the FP32 reciprocal of the scale, clamp to ±448, cast to
  ``torch.float8_e4m3fn`` (round to nearest even).
* ``encode_e4m3_bits`` / ``decode_e4m3_bits`` implement OCP E4M3FN in integer
  arithmetic on the FP32 bit pattern (no torch cast), the arithmetic the
  reference kernel gets from ``__nv_cvt_float_to_fp8(.., __NV_SATFINITE,
  __NV_E4M3)`` (csrc/kernels/host_staged/quantization.cuh:16-24).

Pins (tests/test_oracle_fp8.py): the reference's own known-answer tests
(tests/test_s7.py:41-84 — zero rows, ``scale == amax/448`` on 16 log-spaced rows
with seed 71, exact round trip of [0, 1, -1, 448, -448], empty shapes, the BF16
numeric-corner bit patterns with their scale floor and error bound); exhaustive
agreement of the integer encoder with the library cast over all 2^16 BF16 bit
patterns times several scales; decode of all 256 codes against the closed form
``(-1)^s 2^(e-7) (1 + m/8)``.
"""

from __future__ import annotations

import numpy as np
import torch

E4M3_MAX = 448.0
SCALE_FLOOR = float(np.finfo(np.float32).tiny)  # 2**-126


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits_rne(values: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even FP32 → BF16 for finite inputs (quantization.cuh:23)."""
    raw = np.asarray(values, dtype=np.float32).view(np.uint32)
    rounding = np.uint32(0x7FFF) + ((raw >> np.uint32(16)) & np.uint32(1))
    return ((raw + rounding) >> np.uint32(16)).astype(np.uint16)


def quantize(x: torch.Tensor):
    """pcie_ep/quantization.py:14-30 restated.  Returns (codes uint8 [T,H], scales f32 [T])."""
    if x.ndim != 2 or not x.is_floating_point():
        raise ValueError("expects a floating [T,H] tensor")
    values = x.float()
    amax = values.abs().amax(dim=1) if values.shape[1] else torch.zeros(values.shape[0])
    floor = torch.tensor(SCALE_FLOOR, dtype=torch.float32)
    scales = torch.where(amax == 0, torch.ones_like(amax), torch.maximum(amax / E4M3_MAX, floor))
    scaled = values * (1.0 / scales).unsqueeze(1)
    codes = scaled.clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn).view(torch.uint8)
    return codes, scales


def dequantize(codes: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """pcie_ep/quantization.py:33-39 restated: decode, multiply by the scale in
    FP32 and round to BF16."""
    if codes.dtype != torch.uint8 or codes.ndim != 2:
        raise ValueError("codes must be uint8 [T,H]")
    if scales.shape != codes.shape[:1] or scales.dtype != torch.float32:
        raise ValueError("scales must be FP32 [T]")
    return (codes.view(torch.float8_e4m3fn).float() * scales.unsqueeze(1)).to(torch.bfloat16)


def roundtrip(x: torch.Tensor) -> torch.Tensor:
    """Expected remote BF16 row on an FP8 wire (pcie_ep/quantization.py:42-44)."""
    return dequantize(*quantize(x))


def encode_e4m3_bits(values: np.ndarray) -> np.ndarray:
    """Integer-ALU E4M3FN encoder: round to nearest even, saturate finite
    values to ±448 (0x7E), NaN → 0x7F.  Input FP32, output uint8."""
    raw = np.asarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    sign = ((raw >> np.uint64(24)) & np.uint64(0x80)).astype(np.uint8)
    magnitude = raw & np.uint64(0x7FFFFFFF)
    exponent = (magnitude >> np.uint64(23)).astype(np.int64)  # biased by 127
    mantissa = (magnitude & np.uint64(0x7FFFFF)).astype(np.int64)
    result = np.zeros(raw.shape, dtype=np.int64)
    is_nan = magnitude > np.uint64(0x7F800000)
    # Normal E4M3 range: unbiased exponent -6..8 -> FP32 biased 121..135.
    normal = exponent >= 121
    # Normal: keep 3 mantissa bits; RNE on the 20 dropped bits.
    keep = mantissa >> 20
    rest = mantissa & 0xFFFFF
    round_up = (rest > 0x80000) | ((rest == 0x80000) & ((keep & 1) == 1))
    code_normal = ((exponent - 120) << 3) + keep + round_up.astype(np.int64)
    # Subnormal E4M3: value = m * 2^-9, m in 0..7 (reaching 8 rounds into the
    # first normal).  significand = 1.mantissa * 2^(exponent-127).
    significand = mantissa | (1 << 23)
    shift = np.clip(121 - exponent, 0, 40) + 20  # bits to drop to reach units of 2^-9
    shift = np.minimum(shift, 62)
    keep_sub = significand >> shift
    rest_sub = significand & ((np.int64(1) << shift) - 1)
    half = np.int64(1) << (shift - 1)
    round_up_sub = (rest_sub > half) | ((rest_sub == half) & ((keep_sub & 1) == 1))
    code_sub = keep_sub + round_up_sub.astype(np.int64)
    code_sub = np.where(exponent == 0, 0, code_sub)  # FP32 zero / subnormal inputs are far below 2^-10
    result = np.where(normal, code_normal, code_sub)
    result = np.where(result > 0x7E, 0x7E, result)  # satfinite (also infinities)
    result = np.where(is_nan, 0x7F, result)
    return (result.astype(np.uint8) | sign).astype(np.uint8)


def decode_e4m3_bits(codes: np.ndarray) -> np.ndarray:
    """Closed-form E4M3FN decode to FP32 (NaN for 0x7F / 0xFF)."""
    codes = np.asarray(codes, dtype=np.uint8).astype(np.int64)
    sign = np.where(codes & 0x80, -1.0, 1.0)
    exponent = (codes >> 3) & 0xF
    mantissa = codes & 0x7
    normal = np.ldexp(1.0 + mantissa / 8.0, exponent - 7)
    subnormal = np.ldexp(mantissa / 8.0, -6)
    value = np.where(exponent == 0, subnormal, normal)
    value = np.where((codes & 0x7F) == 0x7F, np.nan, value)
    return (sign * value).astype(np.float32)


def quantize_bits(x_bits: np.ndarray):
    """NumPy-only restatement of the kernel arithmetic (quantization.cuh:34-71)
    on raw BF16 bit rows: returns (codes uint8 [T,H], scales f32 [T])."""
    values = bf16_bits_to_f32(x_bits)
    amax = np.abs(values).max(axis=1) if values.shape[1] else np.zeros(values.shape[0], np.float32)
    amax = amax.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        scales = np.where(amax == 0, np.float32(1.0), np.maximum(amax / np.float32(E4M3_MAX), np.float32(SCALE_FLOOR))).astype(np.float32)
        inverse = (np.float32(1.0) / scales).astype(np.float32)
        scaled = (values * inverse[:, None]).astype(np.float32)
    return encode_e4m3_bits(scaled), scales


def dequantize_bits(codes: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """NumPy-only decode to BF16 bits (quantization.cuh:21-24)."""
    decoded = decode_e4m3_bits(codes) * np.asarray(scales, dtype=np.float32)[:, None]
    return f32_to_bf16_bits_rne(decoded.astype(np.float32))


def e4m3_ulp(values: np.ndarray) -> np.ndarray:
    """Spacing of E4M3FN at |value| (value already divided by the row scale):
    2^(e-3) for normals with unbiased exponent e >= -6, 2^-9 below."""
    magnitude = np.abs(np.asarray(values, dtype=np.float64))
    exponent = np.floor(np.log2(np.maximum(magnitude, 2.0**-6)))
    exponent = np.clip(exponent, -6, 8)
    return np.ldexp(1.0, (exponent - 3).astype(np.int64))

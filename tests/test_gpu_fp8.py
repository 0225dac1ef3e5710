"""FP8 (E4M3FN + per-token FP32 scale) wire: GPU kernels against the oracle.

Bytes and scales must equal the reference encoding (pcie_ep/quantization.py:14-30)
bit for bit; dequantised remote rows must equal the oracle round trip and lie
within one E4M3 ulp times the row scale of the input; local rows stay the
original BF16 (tests/test_s7.py:154-157 of the reference)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import fp8_oracle
from helpers import make_inputs, run_dispatch, verify_captured, verify_dispatch
from test_gpu_dispatch import make_buffer
from test_oracle_fp8 import numeric_corner_bits

pytestmark = pytest.mark.gpu


def _heavy_tailed(tokens, hidden, seed):
    generator = torch.Generator().manual_seed(seed)
    x = torch.randn(tokens, hidden, generator=generator)
    channels = torch.randperm(hidden, generator=generator)[: max(1, hidden // 100)]
    x[:, channels] *= 50.0
    return x.to(torch.bfloat16)


@pytest.mark.parametrize("hidden", [7168, 128, 129, 40])
def test_quantize_kernel_bytes_match_reference_encoding(hidden):
    from pcie_ep.quantization import dequantize_fp8, quantize_fp8

    rows = [_heavy_tailed(96, hidden, 5), torch.zeros(3, hidden, dtype=torch.bfloat16),
            (torch.randn(16, hidden, generator=torch.Generator().manual_seed(71)) * torch.logspace(-3, 3, 16).unsqueeze(1)).to(torch.bfloat16)]
    if hidden % 8 == 0:
        rows.append(numeric_corner_bits(hidden))
    x = torch.cat(rows)
    codes, scales = quantize_fp8(x.cuda())
    want_codes, want_scales = fp8_oracle.quantize(x)
    assert torch.equal(scales.cpu().view(torch.int32), want_scales.view(torch.int32)), "scales differ"
    assert torch.equal(codes.cpu(), want_codes), "E4M3 bytes differ from the reference encoding"
    decoded = dequantize_fp8(codes, scales).cpu()
    assert torch.equal(decoded.view(torch.int16), fp8_oracle.dequantize(want_codes, want_scales).view(torch.int16))
    # Tolerance the task states: within one E4M3 ulp times the row scale.
    normalised = x.double() / want_scales.double().unsqueeze(1)
    ulp = torch.from_numpy(fp8_oracle.e4m3_ulp(normalised.numpy()))
    assert torch.all((decoded.double() - x.double()).abs() <= ulp * want_scales.double().unsqueeze(1))


def test_quantize_kernel_all_bf16_bit_patterns():
    """Every finite BF16 value, in rows of mixed magnitude so many scales occur."""
    from pcie_ep.quantization import quantize_fp8

    bits = torch.arange(65536, dtype=torch.int32)
    finite = ((bits >> 7) & 0xFF) != 0xFF
    values = bits[finite].to(torch.int16).view(torch.bfloat16)
    pad = (-values.numel()) % 256
    values = torch.cat([values, torch.zeros(pad, dtype=torch.bfloat16)])
    x = values[torch.randperm(values.numel(), generator=torch.Generator().manual_seed(3))].view(-1, 256)
    sorted_rows = values.view(-1, 256)  # monotone rows: small-amax rows exercise tiny scales
    x = torch.cat([x, sorted_rows]).contiguous()
    codes, scales = quantize_fp8(x.cuda())
    want_codes, want_scales = fp8_oracle.quantize(x)
    assert torch.equal(scales.cpu().view(torch.int32), want_scales.view(torch.int32))
    assert torch.equal(codes.cpu(), want_codes)


@pytest.mark.parametrize("hidden,channels", [(7168, 8), (136, 2), (129, 2)])
def test_fp8_wire_dispatch(hidden, channels):
    world, experts, topk = 8, 256, 8
    with make_buffer(hidden=hidden, channels=channels, stage=7, wire_dtype="fp8_e4m3", payload_slots=3, descriptor_slots=2) as buffer:
        for expand in (True, False):
            print(f"case: fp8 hidden={hidden} expand={expand}", flush=True)
            inputs = make_inputs(world, [61] * world, hidden, experts, topk, "random", seed=11, gaussian=True, heavy_tail=True)
            result, _ = run_dispatch(buffer, inputs, expand=expand, zero_padding=expand, alignment=8 if expand else 1, capture=True)
            verify_dispatch(result, inputs, 0, world, experts, topk, expand, 8 if expand else 1, expand, fp8_wire=True)
            verify_captured(buffer.peers, inputs, 0, world, experts, topk, fp8_wire=True)
            del result


def test_fp8_wire_numeric_corners():
    """Zero rows, BF16 subnormals, tiny normals and finite maxima through the wire."""
    world, experts, topk, hidden = 8, 256, 8, 128
    corners = numeric_corner_bits(hidden)
    with make_buffer(hidden=hidden, channels=2, stage=7, wire_dtype="fp8_e4m3") as buffer:
        inputs = make_inputs(world, [corners.shape[0]] * world, hidden, experts, topk, "random", seed=13)
        inputs = [(corners.clone(), idx, w) for _, idx, w in inputs]
        result, _ = run_dispatch(buffer, inputs, expand=True, capture=True)
        verify_dispatch(result, inputs, 0, world, experts, topk, True, 1, False, fp8_wire=True)
        verify_captured(buffer.peers, inputs, 0, world, experts, topk, fp8_wire=True)

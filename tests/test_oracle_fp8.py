"""Pin the FP8 wire oracle: the reference's own known-answer tests plus an
independent integer encoder checked exhaustively against the library cast."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import fp8_oracle as fp8


def numeric_corner_bits(hidden: int) -> torch.Tensor:
    """BF16 bit patterns of tests/test_s7.py:21-37 of the reference (data):
    zero, signed subnormals, tiny normals and finite maxima."""
    patterns = torch.tensor(
        [
            [0, 0, 0, 0, 0, 0, 0, 0],
            [0x0001, 0x8001, 0, 0x0002, 0x8002, 0x0007, 0x8007, 0],
            [0x007F, 0x807F, 0x0080, 0x8080, 0x0040, 0x8040, 0, 0x0001],
            [0x0200, 0x8200, 0x0300, 0x8300, 0x0400, 0x8400, 0, 0x0080],
            [0x7F7F, 0xFF7F, 0x7E80, 0xFE80, 0, 0x3F80, 0xBF80, 0x0080],
        ],
        dtype=torch.int32,
    ).to(torch.int16).view(torch.bfloat16)
    return patterns.repeat(1, hidden // patterns.shape[1])


def test_zero_rows_use_scale_one():
    x = torch.zeros(3, 7168, dtype=torch.bfloat16)
    codes, scales = fp8.quantize(x)
    assert torch.equal(scales, torch.ones(3))
    assert not torch.count_nonzero(codes)
    assert torch.equal(fp8.dequantize(codes, scales), x)


def test_scales_are_amax_over_448_and_error_is_bounded():
    generator = torch.Generator().manual_seed(71)
    x = (torch.randn(16, 7168, generator=generator) * torch.logspace(-3, 3, 16).unsqueeze(1)).to(torch.bfloat16)
    codes, scales = fp8.quantize(x)
    assert codes.dtype == torch.uint8 and scales.dtype == torch.float32
    assert torch.equal(scales, x.float().abs().amax(1) / 448.0)
    decoded = fp8.dequantize(codes, scales)
    error = (decoded.float() - x.float()).abs().amax(1)
    assert torch.all(error <= x.float().abs().amax(1) * 0.041 + 1e-7)


def test_fp8_max_and_signs_round_trip_exactly():
    x = torch.tensor([[0, 1, -1, 448, -448]], dtype=torch.bfloat16)
    assert torch.equal(fp8.roundtrip(x), x)
    codes, scales = fp8.quantize(x)
    assert codes.tolist() == [[0x00, 0x38, 0xB8, 0x7E, 0xFE]] and scales.tolist() == [1.0]


def test_empty_input_preserves_shapes():
    codes, scales = fp8.quantize(torch.empty(0, 128, dtype=torch.bfloat16))
    assert codes.shape == (0, 128) and scales.shape == (0,)


def test_numeric_corners_keep_finite_decode_and_bounded_error():
    x = numeric_corner_bits(128)
    codes, scales = fp8.quantize(x)
    decoded = fp8.dequantize(codes, scales)
    assert torch.isfinite(scales).all() and torch.isfinite(scales.reciprocal()).all()
    assert torch.isfinite(decoded).all()
    assert torch.equal(scales[1:4], torch.full((3,), torch.finfo(torch.float32).tiny))
    assert torch.equal(decoded[0], x[0]) and torch.equal(decoded[1], x[1])
    maximum = x.double().abs().amax(1)
    error = (decoded.double() - x.double()).abs().amax(1)
    assert torch.all(error <= maximum * 0.07 + 2.0**-133)


def test_decode_table_matches_closed_form_and_library():
    codes = np.arange(256, dtype=np.uint8)
    mine = fp8.decode_e4m3_bits(codes)
    library = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    finite = ~np.isnan(library)
    assert np.array_equal(np.isnan(mine), np.isnan(library))
    assert np.array_equal(mine[finite].view(np.uint32), library[finite].view(np.uint32))
    assert mine[0x7E] == 448.0 and mine[0x38] == 1.0 and mine[0x01] == 2.0**-9 and mine[0x08] == 2.0**-6


@pytest.mark.parametrize("inverse_scale", [1.0, 448.0 / 3.0, 0.37, 2.0**100, 1.0 / 3.1e-5, 2.0**126])
def test_integer_encoder_matches_library_cast_exhaustively(inverse_scale):
    """All 2^16 BF16 bit patterns (finite ones), multiplied by a scale
    reciprocal and clamped as the reference does, encode identically through
    the integer-ALU encoder and through torch's float8_e4m3fn cast."""
    bits = np.arange(65536, dtype=np.uint16)
    values = fp8.bf16_bits_to_f32(bits)
    finite = np.isfinite(values)
    with np.errstate(over="ignore", invalid="ignore"):
        scaled = (values[finite] * np.float32(inverse_scale)).astype(np.float32)
    scaled = np.clip(scaled, -448.0, 448.0).astype(np.float32)
    library = torch.from_numpy(scaled).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(fp8.encode_e4m3_bits(scaled), library)


def test_integer_encoder_ties_and_saturation():
    # Halfway cases: 1 + 1/16 is a tie between 1.0 (even) and 1.125; 1.1875 ties to 1.25 (even mantissa 2).
    values = np.array([1.0625, 1.1875, 2.0**-10, 3 * 2.0**-10, 2.0**-9 * 7.5, 464.0, 1e9, -1e9, 0.0, -0.0], dtype=np.float32)
    expected = [0x38, 0x3A, 0x00, 0x02, 0x08, 0x7E, 0x7E, 0xFE, 0x00, 0x80]
    assert fp8.encode_e4m3_bits(values).tolist() == expected


def test_numpy_kernel_restatement_equals_torch_restatement():
    """quantize_bits (kernel arithmetic on raw bits) == quantize (reference
    Python arithmetic) on heavy-tailed rows, corner rows and zero rows."""
    generator = torch.Generator().manual_seed(5)
    x = torch.randn(64, 512, generator=generator)
    x[:, ::97] *= 50.0
    x = torch.cat([x.to(torch.bfloat16), numeric_corner_bits(512), torch.zeros(2, 512, dtype=torch.bfloat16)])
    codes, scales = fp8.quantize(x)
    bits = x.view(torch.int16).numpy().view(np.uint16)
    codes_np, scales_np = fp8.quantize_bits(bits)
    assert np.array_equal(scales_np.view(np.uint32), scales.numpy().view(np.uint32))
    assert np.array_equal(codes_np, codes.numpy())
    decoded = fp8.dequantize(codes, scales).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(fp8.dequantize_bits(codes_np, scales_np), decoded)


def test_roundtrip_within_one_ulp_times_scale():
    generator = torch.Generator().manual_seed(9)
    x = torch.randn(32, 1024, generator=generator)
    x[:, ::101] *= 50.0
    x = x.to(torch.bfloat16)
    codes, scales = fp8.quantize(x)
    decoded = fp8.dequantize(codes, scales).double()
    normalised = x.double() / scales.double().unsqueeze(1)
    ulp = torch.from_numpy(fp8.e4m3_ulp(normalised.numpy()))
    assert torch.all((decoded - x.double()).abs() <= ulp * scales.double().unsqueeze(1))

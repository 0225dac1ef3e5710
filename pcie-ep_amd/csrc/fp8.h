// E4M3FN wire arithmetic shared by the gfx950 kernels and the host peer
// emulator.  The host side is integer ALU on FP32 bit patterns; the kernels use
// gfx950's conversion instructions (OCP E4M3FN <-> FP32, FP32 -> BF16, all round
// to nearest even), which produce the same bytes for every finite input:
//   scale  = amax == 0 ? 1 : max(amax / 448, 2^-126)
//   code   = e4m3_rne_satfinite(clamp(x * (1 / scale), -448, 448))
//   decode = bf16_rne(float(e4m3(code)) * scale)
// (reference: pcie_ep/quantization.py:14-44, csrc/kernels/host_staged/quantization.cuh:13-24, :58-70).
#pragma once

#include <cstdint>
#include <cstring>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define PCIE_EP_FP8_HD __host__ __device__ __forceinline__
#else
#define PCIE_EP_FP8_HD inline
#endif

namespace pcie_ep {

constexpr float kE4M3Max = 448.0f;
constexpr float kScaleFloor = 1.17549435e-38f;  // 2^-126, the FP32 normal minimum

PCIE_EP_FP8_HD uint32_t float_bits(float value) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __float_as_uint(value);
#else
    uint32_t bits;
    std::memcpy(&bits, &value, 4);
    return bits;
#endif
}
PCIE_EP_FP8_HD float bits_float(uint32_t bits) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __uint_as_float(bits);
#else
    float value;
    std::memcpy(&value, &bits, 4);
    return value;
#endif
}

PCIE_EP_FP8_HD float bf16_to_float(uint16_t bits) { return bits_float(uint32_t(bits) << 16); }

// Round to nearest even; inputs are finite.
PCIE_EP_FP8_HD uint16_t float_to_bf16_rne(float value) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(value));
#else
    const uint32_t raw = float_bits(value);
    return uint16_t((raw + 0x7FFFu + ((raw >> 16) & 1u)) >> 16);
#endif
}
#if defined(__HIPCC__)
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
// Two FP32 -> two BF16 in one word (first element in the low half), one instruction.
__device__ __forceinline__ uint32_t float2_to_bf16x2_rne(float first, float second) {
    const f32x2 pair = {first, second};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
}
#endif

PCIE_EP_FP8_HD float fp8_scale_from_amax(float amax) {
    if (amax == 0.0f) return 1.0f;
    const float scale = amax / kE4M3Max;
    return scale < kScaleFloor ? kScaleFloor : scale;
}

// FP32 -> E4M3FN, round to nearest even, finite values saturate to 0x7E.
PCIE_EP_FP8_HD uint8_t e4m3_encode(float value) {
#if defined(__HIP_DEVICE_COMPILE__)
    // |value| <= 448 or NaN here (the caller clamps): nothing for the instruction to saturate.
    return uint8_t(__builtin_amdgcn_cvt_pk_fp8_f32(value, 0.0f, 0, false));
#endif
    const uint32_t raw = float_bits(value);
    const uint32_t sign = (raw >> 24) & 0x80u;
    const uint32_t magnitude = raw & 0x7FFFFFFFu;
    if (magnitude > 0x7F800000u) return uint8_t(sign | 0x7Fu);  // NaN (outside the wire contract)
    const uint32_t exponent = magnitude >> 23;  // biased by 127
    uint32_t code;
    if (exponent >= 121u) {
        // Normal E4M3 (unbiased exponent >= -6): keep three mantissa bits.
        const uint32_t mantissa = magnitude & 0x7FFFFFu;
        const uint32_t keep = mantissa >> 20;
        const uint32_t rest = mantissa & 0xFFFFFu;
        const uint32_t up = (rest > 0x80000u) || (rest == 0x80000u && (keep & 1u));
        code = ((exponent - 120u) << 3) + keep + up;
        if (code > 0x7Eu) code = 0x7Eu;
    } else if (exponent < 110u) {
        code = 0;  // below a quarter of the smallest subnormal (2^-9)
    } else {
        // Subnormal E4M3: integer multiples of 2^-9.
        const uint32_t significand = (magnitude & 0x7FFFFFu) | 0x800000u;
        const uint32_t shift = 141u - exponent;  // 21..31
        const uint32_t keep = significand >> shift;
        const uint32_t rest = significand & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1u);
        code = keep + ((rest > half) || (rest == half && (keep & 1u)));
    }
    return uint8_t(sign | code);
}

// E4M3FN -> FP32, exact.
PCIE_EP_FP8_HD float e4m3_decode(uint8_t code) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_cvt_f32_fp8(int(code), 0);
#endif
    if ((code & 0x7Fu) == 0x7Fu) return bits_float(0x7FC00000u);  // NaN (outside the wire contract)
    const uint32_t sign = uint32_t(code & 0x80u) << 24;
    const uint32_t exponent = (code >> 3) & 0xFu;
    const uint32_t mantissa = code & 0x7u;
    if (exponent == 0) {
        // mantissa * 2^-9: the FP32 of a small integer times an exact power of two.
        const float magnitude = float(mantissa) * 0.001953125f;
        return bits_float(float_bits(magnitude) | sign);
    }
    return bits_float(sign | ((exponent + 120u) << 23) | (mantissa << 20));
}

PCIE_EP_FP8_HD uint8_t fp8_quantize_element(uint16_t bf16_bits, float inverse_scale) {
    float scaled = bf16_to_float(bf16_bits) * inverse_scale;
    scaled = scaled > kE4M3Max ? kE4M3Max : (scaled < -kE4M3Max ? -kE4M3Max : scaled);
    return e4m3_encode(scaled);
}

PCIE_EP_FP8_HD uint16_t fp8_dequantize_element(uint8_t code, float scale) {
    return float_to_bf16_rne(e4m3_decode(code) * scale);
}

#if defined(__HIPCC__)
__device__ __forceinline__ float fp8_clamp(float scaled) { return scaled > kE4M3Max ? kE4M3Max : (scaled < -kE4M3Max ? -kE4M3Max : scaled); }
// Four BF16 (two words, elements in order) -> four codes in one word.
__device__ __forceinline__ uint32_t fp8_quantize_word(uint32_t first, uint32_t second, float inverse_scale) {
    const float a = fp8_clamp(bits_float(first << 16) * inverse_scale), b = fp8_clamp(bits_float(first & 0xFFFF0000u) * inverse_scale);
    const float c = fp8_clamp(bits_float(second << 16) * inverse_scale), d = fp8_clamp(bits_float(second & 0xFFFF0000u) * inverse_scale);
    int codes = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    codes = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, codes, true);
    return uint32_t(codes);
}
// Four codes of one word -> four BF16 (two words, elements in order).
__device__ __forceinline__ void fp8_dequantize_word(uint32_t codes, float scale, uint32_t& first, uint32_t& second) {
    const f32x2 low = __builtin_amdgcn_cvt_pk_f32_fp8(int(codes), false), high = __builtin_amdgcn_cvt_pk_f32_fp8(int(codes), true);
    first = float2_to_bf16x2_rne(low[0] * scale, low[1] * scale);
    second = float2_to_bf16x2_rne(high[0] * scale, high[1] * scale);
}
#endif

}  // namespace pcie_ep

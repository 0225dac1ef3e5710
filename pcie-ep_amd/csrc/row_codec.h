// Whole-row helpers executed by one 64-lane wavefront: plain copy, FP8 wire
// quantisation (per-token amax -> scale -> E4M3FN codes) and de-quantisation.
// The quantiser restates quantize_transport_payload of the reference
// (csrc/kernels/host_staged/quantization.cuh:34-71) for one wavefront per token.
#pragma once

#include "device_common.h"

namespace pcie_ep {

__device__ __forceinline__ float wave_max(float value) {
    for (int offset = 32; offset > 0; offset >>= 1) value = fmaxf(value, __shfl_xor(value, offset));
    return value;
}

// BF16 row copy.  kVector requires hidden % 8 == 0 and 16-byte aligned rows.
template <bool kVector, bool kStreamOut>
__device__ __forceinline__ void copy_row(const uint16_t* input, uint16_t* output, int hidden, int lane) {
    if constexpr (kVector) {
        const int vectors = hidden / 8;
        const u32x4* source = reinterpret_cast<const u32x4*>(input);
        u32x4* destination = reinterpret_cast<u32x4*>(output);
        for (int first = 0; first < vectors; first += kPassItems * kWave) {
            RowVectors row;
            row_load_vectors<true>(row, source, first, vectors, lane);
            row_store_vectors<kStreamOut>(row, destination, first, vectors, lane);
        }
    } else {
        for (int index = lane; index < hidden; index += kWave) output[index] = input[index];
    }
}

// Where a quantised row goes: device memory, or a host slot through buffer
// stores with the system-scope cache policy.
struct DeviceCodes {
    uint8_t* output;
    __device__ __forceinline__ void vector(int group, u32x4 codes) const { reinterpret_cast<u32x4*>(output)[group] = codes; }
    __device__ __forceinline__ void single(int index, uint8_t code) const { output[index] = code; }
};
struct HostCodes {
    __amdgpu_buffer_rsrc_t slot;
    __device__ __forceinline__ void vector(int group, u32x4 codes) const { host_store_b128(slot, uint32_t(group) * 16u, codes); }
    __device__ __forceinline__ void single(int index, uint8_t code) const { host_store_b8(slot, uint32_t(index), code); }
};

// BF16 row from device memory into a host slot.
template <bool kVector>
__device__ __forceinline__ void copy_row_to_host(const uint16_t* input, __amdgpu_buffer_rsrc_t slot, int hidden, int lane) {
    if constexpr (kVector) {
        const int vectors = hidden / 8;
        const u32x4* source = reinterpret_cast<const u32x4*>(input);
        for (int first = 0; first < vectors; first += kPassItems * kWave) {
            RowVectors row;
            row_load_vectors<true>(row, source, first, vectors, lane);
#pragma unroll
            for (int j = 0; j < kPassItems; ++j) {
                const int index = first + j * kWave + lane;
                if (index < vectors) host_store_b128(slot, uint32_t(index) * 16u, row.v[j]);
            }
        }
    } else {
        for (int index = lane; index < hidden; index += kWave) host_store_b16(slot, uint32_t(index) * 2u, input[index]);
    }
}

// Returns the row scale.  kVector requires hidden % 16 == 0.
template <bool kVector, typename Sink>
__device__ __forceinline__ float quantize_row(const uint16_t* input, const Sink& sink, int hidden, int lane) {
    // Sweep 1: row amax in FP32.  Sweep 2 re-reads the row (it is L2 resident).
    float amax = 0.0f;
    if constexpr (kVector) {
        const int vectors = hidden / 8;
        const u32x4* source = reinterpret_cast<const u32x4*>(input);
        for (int index = lane; index < vectors; index += kWave) {
            const u32x4 v = source[index];
#pragma unroll
            for (int word = 0; word < 4; ++word) {
                amax = fmaxf(amax, fabsf(bf16_to_float(uint16_t(v[word] & 0xFFFFu))));
                amax = fmaxf(amax, fabsf(bf16_to_float(uint16_t(v[word] >> 16))));
            }
        }
    } else {
        for (int index = lane; index < hidden; index += kWave) amax = fmaxf(amax, fabsf(bf16_to_float(input[index])));
    }
    amax = wave_max(amax);
    const float scale = fp8_scale_from_amax(amax);
    // Multiply by the correctly rounded FP32 reciprocal, as the reference does
    // (quantization.cuh:66; pcie_ep/quantization.py:27-29), not a division per element.
    const float inverse = 1.0f / scale;
    if constexpr (kVector) {
        // 16 elements (two 16-byte loads) -> 16 codes (one 16-byte store) per lane.
        const int groups = hidden / 16;
        const u32x4* source = reinterpret_cast<const u32x4*>(input);
        for (int group = lane; group < groups; group += kWave) {
            const u32x4 lo = source[group * 2], hi = source[group * 2 + 1];
            u32x4 codes;
#pragma unroll
            for (int word = 0; word < 4; ++word) {
                const uint32_t a = word < 2 ? lo[word * 2] : hi[(word - 2) * 2];
                const uint32_t b = word < 2 ? lo[word * 2 + 1] : hi[(word - 2) * 2 + 1];
                codes[word] = fp8_quantize_word(a, b, inverse);
            }
            sink.vector(group, codes);
        }
    } else {
        for (int index = lane; index < hidden; index += kWave) sink.single(index, fp8_quantize_element(input[index], inverse));
    }
    return scale;
}

// 16 codes -> two 16-byte vectors of BF16 (elements in order).
__device__ __forceinline__ void dequantize_vector(const u32x4& codes, float scale, u32x4& lo, u32x4& hi) {
#pragma unroll
    for (int word = 0; word < 4; ++word) {
        const uint32_t c = codes[word];
        uint32_t a, b;
        fp8_dequantize_word(c, scale, a, b);
        if (word < 2) {
            lo[word * 2] = a;
            lo[word * 2 + 1] = b;
        } else {
            hi[(word - 2) * 2] = a;
            hi[(word - 2) * 2 + 1] = b;
        }
    }
}

template <bool kVector>
__device__ __forceinline__ void dequantize_row(const uint8_t* codes, float scale, uint16_t* output, int hidden, int lane) {
    if constexpr (kVector) {
        const int groups = hidden / 16;
        const u32x4* source = reinterpret_cast<const u32x4*>(codes);
        u32x4* destination = reinterpret_cast<u32x4*>(output);
        for (int group = lane; group < groups; group += kWave) {
            u32x4 lo, hi;
            dequantize_vector(source[group], scale, lo, hi);
            destination[group * 2] = lo;
            destination[group * 2 + 1] = hi;
        }
    } else {
        for (int index = lane; index < hidden; index += kWave) output[index] = fp8_dequantize_element(codes[index], scale);
    }
}

// Store one BF16 row (already read into registers pass by pass) to every
// destination row named by the lanes whose `my_row >= 0`.
template <bool kVector>
__device__ __forceinline__ void scatter_row(const uint16_t* input, uint16_t* output_base, int hidden, int64_t my_row, int lane) {
    const uint64_t destinations = __ballot(my_row >= 0);
    if (!destinations) return;
    if constexpr (kVector) {
        const int vectors = hidden / 8;
        const u32x4* source = reinterpret_cast<const u32x4*>(input);
        for (int first = 0; first < vectors; first += kPassItems * kWave) {
            RowVectors row;
            row_load_vectors<true>(row, source, first, vectors, lane);
            uint64_t remaining = destinations;
            while (remaining) {
                const int owner = __builtin_ctzll(remaining);
                remaining &= remaining - 1;
                const int64_t out_row = __shfl(my_row, owner);
                row_store_vectors<true>(row, reinterpret_cast<u32x4*>(output_base + size_t(out_row) * hidden), first, vectors, lane);
            }
        }
    } else {
        for (int first = 0; first < hidden; first += kPassScalars * kWave) {
            RowScalars items;
#pragma unroll
            for (int j = 0; j < kPassScalars; ++j) {
                const int index = first + j * kWave + lane;
                if (index < hidden) items.v[j] = input[index];
            }
            uint64_t remaining = destinations;
            while (remaining) {
                const int owner = __builtin_ctzll(remaining);
                remaining &= remaining - 1;
                uint16_t* output = output_base + size_t(__shfl(my_row, owner)) * hidden;
#pragma unroll
                for (int j = 0; j < kPassScalars; ++j) {
                    const int index = first + j * kWave + lane;
                    if (index < hidden) output[index] = items.v[j];
                }
            }
        }
    }
}

template <bool kVector>
__device__ __forceinline__ void zero_row(uint16_t* output, int hidden, int lane) {
    if constexpr (kVector) {
        u32x4* destination = reinterpret_cast<u32x4*>(output);
        const u32x4 zero = {0u, 0u, 0u, 0u};
        for (int index = lane; index < hidden / 8; index += kWave) __builtin_nontemporal_store(zero, destination + index);
    } else {
        for (int index = lane; index < hidden; index += kWave) output[index] = 0;
    }
}

// Alignment gap of one local expert, rows [offset + count, next offset):
// payload 0, expert -1, weight 0, metadata -1 (advanced_layout.cuh:250-265).
// The prefixes are read with device-scope loads: inside the transport kernel
// they were written by another wavefront of the same launch.
template <bool kVector>
__device__ __forceinline__ void zero_padding_of_expert(const DeviceState& state, int expert, int lane) {
    const int hidden = state.z.dims.hidden;
    const int64_t next = device_load(state.expert_offsets + expert + 1);
    const int64_t end = next < state.expanded_capacity ? next : state.expanded_capacity;
    for (int64_t row = device_load(state.expert_prefix + expert); row < end; ++row) {
        zero_row<kVector>(state.expanded_payload + size_t(row) * hidden, hidden, lane);
        if (lane == 0) {
            state.expanded_expert_idx[row] = -1;
            state.expanded_weights[row] = 0.0f;
            state.expanded_source_meta[row * 3] = state.expanded_source_meta[row * 3 + 1] = state.expanded_source_meta[row * 3 + 2] = -1;
        }
    }
}

// Local bypass of one own token: it never touches the host ring and keeps the
// original BF16 even on an FP8 wire (advanced_layout.cuh:217-248).  Returns
// false when a destination row lies beyond the expanded capacity.
template <bool kVector>
__device__ __forceinline__ bool local_token_rows(const DeviceState& state, int token, int lane) {
    const SegmentLayout& z = state.z;
    const int ranks = z.dims.num_ranks, topk = z.dims.topk, me = state.local_rank, local = z.local_experts;
    const int hidden = z.dims.hidden;
    if (!((state.plan_mask[token] >> me) & 1u)) return true;
    const uint16_t* input = state.x + size_t(token) * hidden;
    float weight = 1.0f;
    int expert_global = -1, ordinal = -1;
    if (lane < topk) {
        expert_global = state.plan_exp_idx[size_t(token) * topk + lane];
        ordinal = state.plan_exp_ord[size_t(token) * topk + lane];
        if (state.topk_weights) weight = state.topk_weights[size_t(token) * topk + lane];
    }
    const int expert = expert_global - me * local;
    const bool is_local = expert_global >= 0 && expert >= 0 && expert < local;
    if (state.expand && state.fuse_expand) {
        int64_t my_row = -1;
        if (is_local)
            my_row = int64_t(device_load(state.expert_offsets + expert)) + device_load(state.source_expert_prefix + me * local + expert) + ordinal;
        if (__any(my_row >= state.expanded_capacity)) return false;
        scatter_row<kVector>(input, state.expanded_payload, hidden, my_row, lane);
        if (my_row >= 0) {
            state.expanded_expert_idx[my_row] = expert;
            state.expanded_weights[my_row] = weight;
            state.expanded_source_meta[my_row * 3] = me;
            state.expanded_source_meta[my_row * 3 + 1] = token;
            state.expanded_source_meta[my_row * 3 + 2] = lane;
        }
    } else {
        const int64_t row = int64_t(device_load(state.source_offsets + me)) + state.plan_rank_ord[size_t(token) * ranks + me];
        copy_row<kVector, true>(input, state.unique_payload + size_t(row) * hidden, hidden, lane);
        if (lane < topk) {
            state.unique_topk_idx[row * topk + lane] = is_local ? expert : -1;
            state.unique_topk_weights[row * topk + lane] = is_local ? weight : 0.0f;
            state.unique_expert_ordinals[row * topk + lane] = ordinal;
        }
        if (lane == 0) {
            state.unique_source_meta[row * 3] = me;
            state.unique_source_meta[row * 3 + 1] = token;
            state.unique_source_meta[row * 3 + 2] = -1;
        }
    }
    return true;
}

}  // namespace pcie_ep

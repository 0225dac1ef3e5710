// HBM-bound stand-alone kernels: the expand of unique rows into expert-major
// rows, the FP8 wire kernels and the calibration copies.  One wavefront moves
// one row: all 16-byte loads of the row are in flight before the first store,
// the row is read once and stored to every destination with streaming 16-byte
// stores.
//
// Replaces scatter_expert_inputs (csrc/kernels/host_staged/dispatch.cuh:8-65) and
// quantize_transport_payload (quantization.cuh:34-71).  The reference copies 2
// bytes per thread here.
#include "device_common.h"
#include "launch.h"
#include "row_codec.h"

namespace pcie_ep {

namespace {

// Stand-alone expand: unique rows -> expert-major rows (dispatch.cuh:8-65).
// Algorithmic HBM traffic: unique_count rows read + expanded_count rows written
// (+ 36 bytes of row metadata per expanded row).
// This version serves rows that are not whole 16-byte vectors (2-byte items,
// one wavefront per row); expand_pieces_kernel below is the one for vector rows.
__global__ void __launch_bounds__(kRowKernelThreads) expand_rows_kernel(DeviceState state) {
    if (load_error_code(state)) return;
    const SegmentLayout& z = state.z;
    const int lane = threadIdx.x % kWave;
    const int waves_per_block = blockDim.x / kWave;
    const int global_wave = blockIdx.x * waves_per_block + threadIdx.x / kWave;
    const int total_waves = gridDim.x * waves_per_block;
    const int topk = z.dims.topk, local = z.local_experts, hidden = z.dims.hidden;
    const int64_t unique = *state.unique_count;
    for (int64_t row = global_wave; row < unique; row += total_waves) {
        const int source = int(state.unique_source_meta[row * 3]);
        const int token = int(state.unique_source_meta[row * 3 + 1]);
        int expert = -1;
        int64_t my_row = -1;
        float weight = 0.0f;
        if (lane < topk) {
            expert = int(state.unique_topk_idx[row * topk + lane]);
            weight = state.unique_topk_weights[row * topk + lane];
            if (expert >= 0)
                my_row = int64_t(state.expert_offsets[expert]) + state.source_expert_prefix[source * local + expert] +
                         state.unique_expert_ordinals[row * topk + lane];
        }
        if (__any(my_row >= state.expanded_capacity)) {
            if (lane == 0) record_error(state, kErrExpandedCapacity);
            return;
        }
        scatter_row<false>(state.unique_payload + size_t(row) * hidden, state.expanded_payload, hidden, my_row, lane);
        if (my_row >= 0) {
            state.expanded_expert_idx[my_row] = expert;
            state.expanded_weights[my_row] = weight;
            state.expanded_source_meta[my_row * 3] = source;
            state.expanded_source_meta[my_row * 3 + 1] = token;
            state.expanded_source_meta[my_row * 3 + 2] = lane;
        }
    }
    if (state.zero_padding)
        for (int expert = global_wave; expert < local; expert += total_waves) zero_padding_of_expert<false>(state, expert, lane);
}

// The same expand for rows of whole 16-byte vectors, shaped for HBM: a workgroup
// of two wavefronts moves ONE 2 KiB piece of a row (one vector per thread) to every
// destination of the row and ends.  Measured on MI355X with the traffic mix of a
// top-8 dispatch (one row read, 1.5 written): pieces that stay inside one aligned
// 2 KiB block, moved by workgroups that live for one piece, reach 5.8 TB/s, a
// wavefront (or workgroup) per 14 KiB row 5.2-5.5 TB/s, looping wavefronts less.
// The row count is only known on the device and a workgroup without a row still
// costs its dispatch (0.2 ns: 34 us for the unused third of a 65 536-row pool),
// so the grid is FOLDED: workgroup (group, piece) serves rows group, group + span,
// group + 2 span ... while they exist.  With two or three rows per workgroup at
// most, every workgroup of a well-filled pool has work and a sparsely filled pool
// pays for a fraction of its capacity only.
// Such a wavefront lives for a few microseconds and a compute unit holds 32 of
// them, so what a piece costs in LATENCY bounds the throughput: everything a piece
// needs is requested at once - the payload vector, the row's routes, and the two
// small prefix tables (expert offsets, per-source expert prefixes), which go to LDS
// so that the destination rows follow from one round of loads instead of two
// dependent ones.
constexpr int kPieceThreads = 128;
constexpr int kPieceTableEntries = 2048;  // expert_offsets[local + 1] + source_expert_prefix[P * local]; larger tables are read from memory
__global__ void __launch_bounds__(kPieceThreads) expand_pieces_kernel(DeviceState state, int pieces, int span) {
    __shared__ int table[kPieceTableEntries];
    const SegmentLayout& z = state.z;
    const int lane = threadIdx.x % kWave;
    const int topk = z.dims.topk, local = z.local_experts, hidden = z.dims.hidden;
    const int group = blockIdx.x / pieces, piece = blockIdx.x % pieces;
    const uint32_t at = uint32_t(piece * kPieceThreads + int(threadIdx.x)) * 16u;  // beyond the row: reads zero, stores dropped
    const uint32_t row_bytes = uint32_t(hidden) * 2u;
    const int entries = local + 1 + z.dims.num_ranks * local;
    const bool tabled = entries <= kPieceTableEntries;
    // Row `group` exists in the pool whether or not it is in use: its loads are issued
    // before anything is known, beside the loads of the count and the tables.  (The grid
    // may be wider than the pool where it is sized by the padding work: a workgroup
    // beyond the pool loads row 0 instead and never uses it.)
    int64_t row = group;
    const int64_t first = row < unique_capacity(z.dims) ? row : 0;
    u32x4 value = stream_load_b128(device_resource(state.unique_payload + size_t(first) * hidden, row_bytes), at);
    int source = int(state.unique_source_meta[first * 3]);
    int expert = lane < topk ? int(state.unique_topk_idx[first * topk + lane]) : -1;
    int ordinal = lane < topk ? state.unique_expert_ordinals[first * topk + lane] : 0;
    // Never beyond the pool, whatever count the sources announced.
    const int64_t announced = *state.unique_count, unique = announced < unique_capacity(z.dims) ? announced : unique_capacity(z.dims);
    const bool failed = load_error_code(state) != 0;
    if (tabled) {
        for (int index = threadIdx.x; index < entries; index += kPieceThreads)
            table[index] = index <= local ? state.expert_offsets[index] : state.source_expert_prefix[index - local - 1];
        __syncthreads();
    }
    if (failed) return;
    while (row < unique) {
        int64_t my_row = -1;
        if (expert >= 0) {
            if (tabled) my_row = int64_t(table[expert]) + table[local + 1 + source * local + expert] + ordinal;
            else my_row = int64_t(state.expert_offsets[expert]) + state.source_expert_prefix[source * local + expert] + ordinal;
        }
        if (__any(my_row >= state.expanded_capacity)) {
            if (lane == 0) record_error(state, kErrExpandedCapacity);
            return;
        }
        uint64_t remaining = __ballot(my_row >= 0);
        while (remaining) {
            const int owner = __builtin_ctzll(remaining);
            remaining &= remaining - 1;
            const int64_t out_row = __shfl(my_row, owner);
            stream_store_b128(device_resource(state.expanded_payload + size_t(out_row) * hidden, row_bytes), at, value);
        }
        // Row metadata once per row: the first wavefront of the row's first piece.
        if (piece == 0 && threadIdx.x < kWave && my_row >= 0) {
            state.expanded_expert_idx[my_row] = expert;
            state.expanded_weights[my_row] = state.unique_topk_weights[row * topk + lane];
            state.expanded_source_meta[my_row * 3] = source;
            state.expanded_source_meta[my_row * 3 + 1] = int(state.unique_source_meta[row * 3 + 1]);
            state.expanded_source_meta[my_row * 3 + 2] = lane;
        }
        row += span;
        if (row >= unique) break;
        value = stream_load_b128(device_resource(state.unique_payload + size_t(row) * hidden, row_bytes), at);
        source = int(state.unique_source_meta[row * 3]);
        expert = lane < topk ? int(state.unique_topk_idx[row * topk + lane]) : -1;
        ordinal = lane < topk ? state.unique_expert_ordinals[row * topk + lane] : 0;
    }
    if (state.zero_padding) {
        const int global_wave = blockIdx.x * (kPieceThreads / kWave) + threadIdx.x / kWave;
        if (global_wave < local) zero_padding_of_expert<true>(state, global_wave, lane);
    }
}

template <bool kVector>
__global__ void __launch_bounds__(kRowKernelThreads) quantize_kernel(const uint16_t* x, uint8_t* codes, float* scales, int tokens, int hidden) {
    const int lane = threadIdx.x % kWave;
    const int waves_per_block = blockDim.x / kWave;
    const int total_waves = gridDim.x * waves_per_block;
    for (int token = blockIdx.x * waves_per_block + threadIdx.x / kWave; token < tokens; token += total_waves) {
        const float scale = quantize_row<kVector>(x + size_t(token) * hidden, DeviceCodes{codes + size_t(token) * hidden}, hidden, lane);
        if (lane == 0) scales[token] = scale;
    }
}

template <bool kVector>
__global__ void __launch_bounds__(kRowKernelThreads) dequantize_kernel(const uint8_t* codes, const float* scales, uint16_t* out, int tokens, int hidden) {
    const int lane = threadIdx.x % kWave;
    const int waves_per_block = blockDim.x / kWave;
    const int total_waves = gridDim.x * waves_per_block;
    for (int token = blockIdx.x * waves_per_block + threadIdx.x / kWave; token < tokens; token += total_waves)
        dequantize_row<kVector>(codes + size_t(token) * hidden, scales[token], out + size_t(token) * hidden, hidden, lane);
}

// Plain device copy: every wavefront moves one contiguous 8 KiB (8 x 16-byte
// vectors per lane) and ends - the fastest copy shape measured on this part
// (6.3 TB/s read + write; 16 KiB per wavefront 6.1, wavefronts that loop over
// several pieces 5.6-5.8, the copy engine behind hipMemcpy 5.2).  It exists to
// calibrate measurements: the practical HBM ceiling of a read+write stream, and
// the scale of the memory traffic counters for a kernel whose traffic is known.
constexpr int kCopyItems = 8;
__global__ void __launch_bounds__(kRowKernelThreads) hbm_copy_kernel(const u32x4* source, u32x4* destination, int64_t vectors) {
    const int lane = threadIdx.x % kWave;
    const int64_t first = (int64_t(blockIdx.x) * (kRowKernelThreads / kWave) + threadIdx.x / kWave) * (kCopyItems * kWave);
    if (first >= vectors) return;
    const int64_t left = vectors - first;
    const uint32_t bytes = uint32_t(left < kCopyItems * kWave ? left : kCopyItems * kWave) * 16u;
    const __amdgpu_buffer_rsrc_t from = device_resource(source + first, bytes), to = device_resource(destination + first, bytes);
    u32x4 piece[kCopyItems];
#pragma unroll
    for (int j = 0; j < kCopyItems; ++j) piece[j] = stream_load_b128(from, uint32_t(j * kWave + lane) * 16u);
#pragma unroll
    for (int j = 0; j < kCopyItems; ++j) stream_store_b128(to, uint32_t(j * kWave + lane) * 16u, piece[j]);
}

// The same copy between pinned host memory and HBM, through the buffer accesses
// with the system-scope cache policy that the transport kernel uses for host
// slots.  A fixed number of wavefronts loops over the 16 KiB pieces, so the bytes
// in flight are wavefronts x 16 KiB as in the transport kernel.  It calibrates
// what a kernel (as opposed to the copy engine behind hipMemcpy) can pull over
// the host link, and the scale of the host-traffic counters.
template <bool kToDevice>
__global__ void __launch_bounds__(kRowKernelThreads) host_copy_kernel(char* host, u32x4* device, int64_t vectors) {
    const int lane = threadIdx.x % kWave;
    const int waves_per_block = blockDim.x / kWave;
    const int64_t total_waves = int64_t(gridDim.x) * waves_per_block;
    const int64_t chunk = int64_t(kPassItems) * kWave;
    for (int64_t first = (int64_t(blockIdx.x) * waves_per_block + threadIdx.x / kWave) * chunk; first < vectors; first += total_waves * chunk) {
        const int count = int(vectors - first < chunk ? vectors - first : chunk);
        const __amdgpu_buffer_rsrc_t piece = host_resource(host + first * 16, uint32_t(count) * 16u);
        RowVectors row;
        if constexpr (kToDevice) {
#pragma unroll
            for (int j = 0; j < kPassItems; ++j) row.v[j] = host_load_b128(piece, uint32_t(j * kWave + lane) * 16u);  // out of range reads 0
            row_store_vectors<true>(row, device + first, 0, count, lane);
        } else {
            row_load_vectors<true>(row, device + first, 0, count, lane);
#pragma unroll
            for (int j = 0; j < kPassItems; ++j)
                if (j * kWave + lane < count) host_store_b128(piece, uint32_t(j * kWave + lane) * 16u, row.v[j]);
        }
    }
}

// Plain fill: the clearing step of callers that may be under graph capture,
// where a memset node is not wanted.
__global__ void __launch_bounds__(kRowKernelThreads) zero_kernel(u32x4* destination, size_t vectors) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x; index < vectors; index += size_t(gridDim.x) * blockDim.x)
        destination[index] = zero;
}

// Calibration of the expand kernel's traffic SHAPE: every wavefront reads one row
// and writes it once, and a given fraction of the rows twice, with no metadata
// and no dependent loads.  The destination order is linear, `streams`
// interleaved sequential streams (what expert-major placement of source-ordered
// rows produces), or hashed; patterns 3 and 4 only read / only write the rows.
// What this reaches is the practical HBM ceiling
// for a write-heavy row scatter; the expand kernel is compared with it.
__global__ void __launch_bounds__(kRowKernelThreads) row_scatter_kernel(const u32x4* source, u32x4* destination, int rows, int row_vectors,
                                                                         int extra_per_1024, int pattern, int streams) {
    const int lane = threadIdx.x % kWave;
    const int waves_per_block = blockDim.x / kWave;
    const int total_waves = gridDim.x * waves_per_block;
    for (int row = blockIdx.x * waves_per_block + threadIdx.x / kWave; row < rows; row += total_waves) {
        int out = row;
        if (pattern == 1) {
            const int stream = row % streams, position = row / streams, per_stream = rows / streams;
            if (position < per_stream) out = stream * per_stream + position;
        } else if (pattern == 2) {
            out = int(uint64_t(row) * 2654435761ull % uint64_t(rows));
        }
        const u32x4* from = source + size_t(row) * row_vectors;
        for (int first = 0; first < row_vectors; first += kPassItems * kWave) {
            RowVectors pass;
            if (pattern == 4) {  // write only
#pragma unroll
                for (int j = 0; j < kPassItems; ++j) pass.v[j] = u32x4{uint32_t(row), uint32_t(j), uint32_t(lane), 1u};
            } else {
                row_load_vectors<true>(pass, from, first, row_vectors, lane);
            }
            if (pattern == 3) {  // read only: fold the row so the loads cannot be dropped
                uint32_t fold = 0;
#pragma unroll
                for (int j = 0; j < kPassItems; ++j)
                    if (first + j * kWave + lane < row_vectors) fold += pass.v[j][0] ^ pass.v[j][1] ^ pass.v[j][2] ^ pass.v[j][3];
                if (fold == 0x9E3779B9u) destination[0] = pass.v[0];
                continue;
            }
            row_store_vectors<true>(pass, destination + size_t(out) * row_vectors, first, row_vectors, lane);
            if (pattern < 3 && (row & 1023) * extra_per_1024 / 1024 != ((row & 1023) + 1) * extra_per_1024 / 1024)
                row_store_vectors<true>(pass, destination + size_t(rows + out) * row_vectors, first, row_vectors, lane);
        }
    }
}

int row_grid(int64_t rows, int64_t cap = 8192) {
    // Four wavefronts per workgroup, one row per wavefront, capped so that the
    // grid-stride loop still spreads over all 256 CUs several times.
    int64_t blocks = (rows + 3) / 4;
    if (blocks < 1) blocks = 1;
    if (blocks > cap) blocks = cap;
    return int(blocks);
}

}  // namespace

hipError_t launch_expand(const DeviceState& state, hipStream_t stream) {
    const int64_t capacity = unique_capacity(state.z.dims);
    if (state.z.dims.hidden % 8 == 0) {
        // 2 KiB pieces, one workgroup each; the grid is folded so that it has about
        // 150 000 workgroups at most (a third of a 65 536-row pool of 14 KiB rows)
        // and at least one workgroup per piece of every local expert's padding.
        const int64_t pieces = (state.z.dims.hidden / 8 + kPieceThreads - 1) / kPieceThreads;
        constexpr int64_t kTargetWorkgroups = 152922;
        const int64_t fold = (capacity * pieces + kTargetWorkgroups - 1) / kTargetWorkgroups;
        int64_t span = (capacity + fold - 1) / fold;
        const int64_t padding_groups = (state.z.local_experts + 1) / 2;  // two wavefronts per workgroup
        if (span * pieces < padding_groups) span = (padding_groups + pieces - 1) / pieces;
        if (span * pieces > (int64_t(1) << 30)) return hipErrorInvalidValue;  // cannot happen within the supported dimensions
        hipLaunchKernelGGL(expand_pieces_kernel, dim3(unsigned(span * pieces)), dim3(kPieceThreads), 0, stream, state, int(pieces), int(span));
        return hipGetLastError();
    }
    // Rows that are not whole vectors: one wavefront per possible unique row up to 65 536 rows.
    const dim3 grid(row_grid(capacity, 16384)), block(kRowKernelThreads);
    hipLaunchKernelGGL(expand_rows_kernel, grid, block, 0, stream, state);
    return hipGetLastError();
}

hipError_t launch_zero(void* destination, size_t bytes, hipStream_t stream) {
    if (bytes % 16 || reinterpret_cast<uintptr_t>(destination) % 16) return hipErrorInvalidValue;
    const size_t vectors = bytes / 16;
    if (!vectors) return hipSuccess;
    const size_t blocks = (vectors + kRowKernelThreads - 1) / kRowKernelThreads;
    hipLaunchKernelGGL(zero_kernel, dim3(unsigned(blocks < 1024 ? blocks : 1024)), dim3(kRowKernelThreads), 0, stream, static_cast<u32x4*>(destination), vectors);
    return hipGetLastError();
}

hipError_t launch_row_scatter(const void* source, void* destination, int rows, int row_bytes, int extra_per_1024, int pattern, int streams,
                              hipStream_t stream) {
    if (rows <= 0 || row_bytes <= 0 || row_bytes % 16 || extra_per_1024 < 0 || extra_per_1024 > 1024 || pattern < 0 || pattern > 4 || streams < 1)
        return hipErrorInvalidValue;
    const dim3 grid(row_grid(rows, 16384)), block(kRowKernelThreads);
    hipLaunchKernelGGL(row_scatter_kernel, grid, block, 0, stream, static_cast<const u32x4*>(source), static_cast<u32x4*>(destination), rows,
                       row_bytes / 16, extra_per_1024, pattern, streams);
    return hipGetLastError();
}

hipError_t launch_copy(const void* source, void* destination, int64_t bytes, hipStream_t stream) {
    const int64_t vectors = bytes / 16;
    if (vectors <= 0) return hipSuccess;
    const int64_t per_block = int64_t(kCopyItems) * kWave * (kRowKernelThreads / kWave);
    const int64_t blocks = (vectors + per_block - 1) / per_block;
    if (blocks > (int64_t(1) << 30)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(hbm_copy_kernel, dim3(unsigned(blocks)), dim3(kRowKernelThreads), 0, stream, static_cast<const u32x4*>(source),
                       static_cast<u32x4*>(destination), vectors);
    return hipGetLastError();
}

hipError_t launch_host_copy(void* host, void* device, int64_t bytes, bool to_device, int wavefronts, hipStream_t stream) {
    const int64_t vectors = bytes / 16;
    if (vectors <= 0) return hipSuccess;
    const dim3 grid(wavefronts < 4 ? 1 : wavefronts / 4), block(kRowKernelThreads);
    if (to_device) hipLaunchKernelGGL(host_copy_kernel<true>, grid, block, 0, stream, static_cast<char*>(host), static_cast<u32x4*>(device), vectors);
    else hipLaunchKernelGGL(host_copy_kernel<false>, grid, block, 0, stream, static_cast<char*>(host), static_cast<u32x4*>(device), vectors);
    return hipGetLastError();
}

hipError_t launch_quantize(const uint16_t* x, uint8_t* codes, float* scales, int tokens, int hidden, hipStream_t stream) {
    if (tokens <= 0) return hipSuccess;
    const dim3 grid(row_grid(tokens)), block(kRowKernelThreads);
    if (hidden % 16 == 0) hipLaunchKernelGGL(quantize_kernel<true>, grid, block, 0, stream, x, codes, scales, tokens, hidden);
    else hipLaunchKernelGGL(quantize_kernel<false>, grid, block, 0, stream, x, codes, scales, tokens, hidden);
    return hipGetLastError();
}

hipError_t launch_dequantize(const uint8_t* codes, const float* scales, uint16_t* out, int tokens, int hidden, hipStream_t stream) {
    if (tokens <= 0) return hipSuccess;
    const dim3 grid(row_grid(tokens)), block(kRowKernelThreads);
    if (hidden % 16 == 0) hipLaunchKernelGGL(dequantize_kernel<true>, grid, block, 0, stream, codes, scales, out, tokens, hidden);
    else hipLaunchKernelGGL(dequantize_kernel<false>, grid, block, 0, stream, codes, scales, out, tokens, hidden);
    return hipGetLastError();
}

}  // namespace pcie_ep

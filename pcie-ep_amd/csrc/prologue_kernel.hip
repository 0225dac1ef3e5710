// Prologue kernel: the dispatch prologue (prologue_body.h) as a launch of its own,
// one workgroup per chunk of up to 16 wavefronts of tokens, in front of the
// transport kernel.  Used when the prologue cannot ride in the transport kernel's
// launch (the runtime decides at create time: `fused` in runtime.hip), or when the caller asks for it.
#include "prologue_body.h"

namespace pcie_ep {

template <int kTopk>
__global__ void __launch_bounds__(kPrologueMaxThreads) prologue_kernel(DeviceState state, int chunk_waves, int chunks) {
    extern __shared__ __align__(16) unsigned char lds[];
    prologue_chunk<kTopk, false>(state, lds, chunk_waves, chunks, int(blockIdx.x));
}

size_t prologue_lds_bytes(const SegmentLayout& z, int chunk_waves) {
    const size_t bins = size_t(z.dims.num_ranks) + z.dims.num_experts;
    return bins * chunk_waves * 10 + bins * 4 + size_t(z.dims.channels) * z.dims.num_ranks * 4 +
           size_t(z.dims.channels) * (1 + z.dims.domains) * 4 + 64;
}

// The largest chunk whose tables fit the 64 KiB of LDS every workgroup may use
// without opting in to more: 16 wavefronts up to 390 bins, 1 wavefront (14 bytes
// per bin: 57.6 KB) at the maximum of 16 + 4096 bins.
int prologue_chunk_waves(const SegmentLayout& z) {
    int waves = 16;
    while (waves > 1 && prologue_lds_bytes(z, waves) > 64 * 1024) waves /= 2;
    return waves;
}

int prologue_chunks(const SegmentLayout& z, int tokens, int chunk_waves) {
    const int chunk_tokens = (chunk_waves > 0 ? chunk_waves : prologue_chunk_waves(z)) * kWave;
    return (tokens + chunk_tokens - 1) / chunk_tokens;
}

// Whether the prologue can run as workgroups of the transport launch (blocks of
// `block_threads`): its chunks are then that workgroup's wavefronts.  The route
// ids of a token stay in registers (top-k up to 8 only: more would raise the
// register count of the whole transport kernel), the layout tables share the LDS
// with the transport roles, and all chunks of a full batch must be resident beside them.
constexpr int kFusedChunkWaves = 4;
constexpr int kFusedMaxChunks = 64;
bool fused_prologue_fits(const SegmentLayout& z, int block_threads, int max_tokens) {
    return z.dims.topk <= 8 && block_threads == kFusedChunkWaves * kWave && prologue_lds_bytes(z, kFusedChunkWaves) <= 40 * 1024 &&
           prologue_chunks(z, max_tokens, kFusedChunkWaves) <= kFusedMaxChunks;
}

// Chunk flags and records are sized for the smaller of the two chunk shapes.
static int most_chunks(const SegmentLayout& z) {
    const int waves = prologue_chunk_waves(z) < kFusedChunkWaves ? prologue_chunk_waves(z) : kFusedChunkWaves;
    return prologue_chunks(z, z.dims.max_tokens, waves);
}

size_t prologue_flag_bytes(const SegmentLayout& z) { return align_up(size_t(most_chunks(z)) * 8, 256); }

size_t prologue_scratch_bytes(const SegmentLayout& z) {
    const ChunkRecord record{z.dims.num_ranks + z.dims.num_experts, z.dims.channels, z.dims.num_ranks, z.dims.domains};
    return prologue_flag_bytes(z) + size_t(most_chunks(z)) * record.stride() * 4;
}

hipError_t launch_prologue(const DeviceState& state, hipStream_t stream) {
    const int waves = prologue_chunk_waves(state.z);
    const size_t bytes = prologue_lds_bytes(state.z, waves);
    const bool narrow = state.z.dims.topk <= 8;
    if (bytes > 64 * 1024) return hipErrorInvalidValue;  // cannot happen within the supported dimensions
    // At least 256 threads so the clear / publish loops stay short.
    const int threads = waves * kWave < 256 ? 256 : waves * kWave;
    if (threads > kPrologueMaxThreads) return hipErrorInvalidValue;
    const int chunks = state.reuse_plan ? 0 : prologue_chunks(state.z, state.num_tokens, waves);
    const dim3 grid(chunks > 1 ? chunks : 1);
    if (narrow) hipLaunchKernelGGL(prologue_kernel<8>, grid, dim3(threads), bytes, stream, state, waves, chunks);
    else hipLaunchKernelGGL(prologue_kernel<kMaxTopk>, grid, dim3(threads), bytes, stream, state, waves, chunks);
    return hipGetLastError();
}

}  // namespace pcie_ep

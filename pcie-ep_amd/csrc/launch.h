// Host-callable launchers of the gfx950 kernels (one translation unit each).
#pragma once

#include <hip/hip_runtime.h>

#include <string>

#include "../../include/pcie_ep_amd.h"

#include "device_common.h"

namespace pcie_ep {

// Payload workgroups of the transport kernel (after the C control workgroups)
// and the payload wavefronts each of them carries (tx_waves + rx_waves: which
// direction a wavefront serves is decided row by row inside the kernel, so only
// the sum of the two numbers matters).  Every wavefront has one row in flight, so
// their number sets the bytes outstanding on the host link.  The default keeps
// kBytesInFlight outstanding whatever the row size is: 48 workgroups of four
// wavefronts for 14 KB rows (BF16, hidden 7168), 96 for 7 KB rows (the FP8 wire:
// measured 1.5 % faster than 64) and for anything shorter.  More wavefronts than
// that buy nothing on the link (48 to 96 workgroups are within 0.2 % of each
// other for 14 KB rows) and take compute units from kernels running beside the
// dispatch.
constexpr int64_t kBytesInFlight = 2736 << 10;
constexpr int kMinDefaultWorkerGroups = 16, kMaxDefaultWorkerGroups = 96;
constexpr int kDefaultTxWaves = 2;
constexpr int kDefaultRxWaves = 2;
constexpr int kMaxTxWaves = 4;
constexpr int kMaxRxWaves = 6;
// Upper bound of the payload workgroups: with at most 32 control and 32 local-bypass workgroups the grid then has at
// most 256 workgroups of at most 768 threads, and an MI355X (256 compute units, each able to hold at least one such
// workgroup next to other work) keeps all of them resident at once.  The roles wait for each other through device
// memory, so the control workgroups must be running while payload wavefronts wait for tickets: with the whole grid
// resident that holds without any assumption about the order in which workgroups are started.  On a smaller
// partition the control workgroups still carry the lowest indices and are started first; should a payload wavefront
// ever wait for a control workgroup that is not running, its bounded wait ends the dispatch with code 15.
constexpr int kMaxWorkerGroups = 192;

// Workgroup sizes.  Each constant is used twice: as the __launch_bounds__ of the
// kernel and by its launcher, so a launch shape can never exceed what the kernel
// was compiled for (a block larger than the bound fails at launch).
constexpr int kRowKernelThreads = 256;       // expand, FP8 wire, copy and fill kernels: four wavefronts
constexpr int kTransportMaxThreads = 768;    // 2 control + at most 10 payload wavefronts
constexpr int kPrologueMaxThreads = 1024;    // 16 wavefronts per token chunk
static_assert((2 + kMaxTxWaves + kMaxRxWaves) * kWave <= kTransportMaxThreads, "transport workgroup exceeds its launch bound");

// Epoch begin + layout + count publication (one workgroup per chunk of tokens).
// The layout scratch holds prologue_flag_bytes() of zero-initialised chunk
// flags followed by the per-chunk records.
hipError_t launch_prologue(const DeviceState& state, hipStream_t stream);
size_t prologue_flag_bytes(const SegmentLayout& z);
size_t prologue_scratch_bytes(const SegmentLayout& z);
size_t prologue_lds_bytes(const SegmentLayout& z, int chunk_waves);
int prologue_chunk_waves(const SegmentLayout& z);
// Chunks of `tokens` tokens at `chunk_waves` wavefronts per chunk (0: the prologue kernel's own shape).
int prologue_chunks(const SegmentLayout& z, int tokens, int chunk_waves);
// Whether the prologue can run inside the transport launch (workgroups of `block_threads` threads);
// launch_transport runs it there when DeviceState::fused is set, and launch_prologue is then not called.
bool fused_prologue_fits(const SegmentLayout& z, int block_threads, int max_tokens);
// Channel transport: control / TX / RX-scatter wavefront roles, the local bypass,
// alignment-gap zeroing and the statistics reduction.
hipError_t launch_transport(const DeviceState& state, hipStream_t stream);
int transport_threads(const DeviceState& state);
// Transport workgroups (of the instantiation `state` selects) that one compute unit holds at once.
hipError_t transport_workgroups_per_unit(const DeviceState& state, int* per_unit);
// Stand-alone expand of unique rows into expert-major rows (+ padding).
hipError_t launch_expand(const DeviceState& state, hipStream_t stream);
// Plain device-to-device copy of `bytes` (multiple of 16) with the row movers' access shape.
hipError_t launch_copy(const void* source, void* destination, int64_t bytes, hipStream_t stream);
// One row read, one row written (and `extra_per_1024` of every 1024 rows written a second time into the upper half of
// `destination`, which holds 2 * rows rows): pattern 0 linear, 1 `streams` interleaved sequential streams, 2 hashed, 3 read only, 4 write only.
hipError_t launch_row_scatter(const void* source, void* destination, int rows, int row_bytes, int extra_per_1024, int pattern, int streams,
                              hipStream_t stream);
// Zero `bytes` (a multiple of 16) of device memory at a 16-byte aligned address with a fill kernel.
hipError_t launch_zero(void* destination, size_t bytes, hipStream_t stream);
// Kernel-driven copy between pinned host memory and HBM with `wavefronts` wavefronts in flight.
hipError_t launch_host_copy(void* host, void* device, int64_t bytes, bool to_device, int wavefronts, hipStream_t stream);
// Publication / acknowledgement litmus on pinned host memory (litmus.hip); 0 or a PCIE_EP_E_* code.
int run_litmus(int device, int mode, int64_t iterations, int payload_bytes, int writer_delay_ns, int reader_delay_ns, int timeout_ms,
               pcie_ep_litmus_result* out, std::string& error);
// Stand-alone FP8 wire kernels.
hipError_t launch_quantize(const uint16_t* x, uint8_t* codes, float* scales, int tokens, int hidden, hipStream_t stream);
hipError_t launch_dequantize(const uint8_t* codes, const float* scales, uint16_t* out, int tokens, int hidden, hipStream_t stream);

}  // namespace pcie_ep

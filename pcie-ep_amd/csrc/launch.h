// Host-callable launchers of the gfx950 kernels (one translation unit each).
#pragma once

#include <hip/hip_runtime.h>

#include "device_common.h"

namespace pcie_ep {

constexpr int kDefaultTxWaves = 2;
constexpr int kDefaultRxWaves = 4;
constexpr int kMaxTxWaves = 4;
constexpr int kMaxRxWaves = 6;

// Epoch begin + layout + count publication (one workgroup).
hipError_t launch_prologue(const DeviceState& state, hipStream_t stream);
// Channel transport: control / TX / RX-scatter wavefront roles, one workgroup per channel.
hipError_t launch_transport(const DeviceState& state, hipStream_t stream);
int transport_threads(int tx_waves, int rx_waves);
// Local bypass copy, alignment-gap zeroing and statistics reduction.
hipError_t launch_epilogue(const DeviceState& state, hipStream_t stream);
// Stand-alone expand of unique rows into expert-major rows (+ padding).
hipError_t launch_expand(const DeviceState& state, hipStream_t stream);
// Stand-alone FP8 wire kernels.
hipError_t launch_quantize(const uint16_t* x, uint8_t* codes, float* scales, int tokens, int hidden, hipStream_t stream);
hipError_t launch_dequantize(const uint8_t* codes, const float* scales, uint16_t* out, int tokens, int hidden, hipStream_t stream);

}  // namespace pcie_ep

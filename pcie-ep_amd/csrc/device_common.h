// Device-side state, synchronisation primitives and wavefront row movers for
// the gfx950 dispatch kernels.  Wave size is 64 throughout.
#pragma once

#include <hip/hip_runtime.h>

#include "fp8.h"
#include "wire.h"

namespace pcie_ep {

constexpr int kWave = 64;

// Per-role timing records, compiled in only with -DPCIE_EP_ENABLE_PROFILING=1 (the
// reference's switch of the same name: csrc/kernels/host_staged/advanced_common.cuh:
// 126-181, docs/pcie-ep/profiling-instrumentation.md).  A default build contains
// none of it: the macro below expands to nothing and DeviceState has no field for it.
#ifndef PCIE_EP_ENABLE_PROFILING
#define PCIE_EP_ENABLE_PROFILING 0
#endif
#if PCIE_EP_ENABLE_PROFILING
#define PCIE_EP_PROFILE(...) __VA_ARGS__
#else
#define PCIE_EP_PROFILE(...)
#endif
constexpr int kProfileFields = 32;
constexpr int kProfileSampleStride = 8;  // every 8th row of a payload wavefront is timed in detail

constexpr uint64_t kPrefixFailed = ~uint64_t(0);
// Set in the claim word of the receive prefixes once their producer has put its
// reads of the count mailboxes on the host link.
constexpr uint64_t kPrefixRequested = uint64_t(1) << 63;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Work queues of the transport kernel, in device memory.  Control wavefronts
// (one TX and one RX control per channel) produce tickets into two global
// rings; payload wavefronts of ANY workgroup, and therefore of any XCD, claim
// them.  A row is thus moved by whichever wavefront is free: channels are load
// balanced against each other, every channel is served by all eight XCDs (the
// XCDs get unequal shares of the host link), and the number of rows in flight
// - which sets the latency every control-path read sees - is chosen by the
// number of worker wavefronts, not by the number of channels.
// All fields are accessed with device-scope (cross-XCD coherent) operations;
// the per-entry tags carry the epoch, so the rings need no clearing.
constexpr int kRing = 2048;

struct alignas(16) RxEntry {
    int32_t source;
    int32_t slot;
    int32_t token;
    int32_t channel;
    uint64_t payload_sequence;
    int32_t channel_ordinal;  // position among the channel's receive tickets of this dispatch
    int32_t replica;          // 1: `slot` is a replica slot of this rank's domain (relay mode)
};
struct alignas(16) TxEntry {
    int32_t token;
    int32_t ordinal;  // position among this channel's remote tokens
    uint32_t endpoints;  // destination ranks of the own domain and, in relay mode, relay endpoints P + domain
    int32_t channel;
    int32_t descriptor_ordinal[kMaxEndpoints];
};
static_assert(sizeof(RxEntry) == 32 && sizeof(TxEntry) == 112, "queue entry layout");

struct alignas(128) QueueCounter {
    uint32_t value;
    int32_t total;  // -1 until the number of tickets is known
    char pad[120];
};

struct alignas(256) TransportQueues {
    QueueCounter rx_tail, tx_tail;  // tickets reserved by producers (fetch-add)
    QueueCounter rx_head, tx_head;  // tickets claimed by workers (fetch-add); .total = tickets of this dispatch
    QueueCounter abort;             // value != 0: every role exits
    QueueCounter local_head;        // own tokens (then padding gaps) claimed for the local bypass
    QueueCounter finished;          // role wavefronts that have ended; the last one reduces the statistics
    // Prologue inside the transport launch: value = epoch_flag(epoch) once the epoch begin has cleared the
    // diagnostics and reset the queues (begun) / has found no abort word set and the previous count mailbox
    // consumed (verdict) / the leader has published the counts and the whole plan is in memory (plan_ready);
    // plan_chunks counts the chunks other than the leader's whose part of the plan is in memory.
    QueueCounter begun, verdict, plan_ready, plan_chunks;
    QueueCounter rx_retired[kMaxChannels], tx_retired[kMaxChannels], rx_finished[kMaxChannels];
    uint64_t rx_ready[kRing], rx_taken[kRing];  // sequence(epoch, n): entry n % kRing holds / has been copied out
    uint64_t tx_ready[kRing], tx_taken[kRing];
    RxEntry rx[kRing];
    TxEntry tx[kRing];
};

// Launch argument of every kernel: this rank's device pointers, the device
// aliases of the pinned host segments and the plan/output pool of one dispatch
// (the role of AdvancedDeviceState: csrc/kernels/host_staged/advanced_common.cuh:86-129).
struct DeviceState {
    SegmentLayout z;
    char* seg[kMaxRanks];
    char* replica_in[kMaxRanks];  // relay mode: replica payload region of every source for this rank's domain
    int local_rank;
    int fuse_expand;  // receive waves scatter straight into expert rows
    int expand;
    int alignment;
    int num_tokens;
    int zero_padding;
    int reuse_plan;
    int counts_ack_skip_source;
    int overlap_diagnostic;  // fill receive_expand_overlap (count, completion watermark); 0 leaves it zero
    int fused;               // 1: the prologue runs as the first workgroups of the transport launch
    int prologue_chunks;     // token chunks of this dispatch's layout (0 when a cached plan is reused)
    uint64_t timeout_ticks;
    uint64_t clock_khz;  // rate of wall_clock64() on this device (hipDeviceAttributeWallClockRate)
    uint64_t* epoch;

    const uint16_t* x;
    const int64_t* topk_idx;
    const float* topk_weights;

    // Route plan (immutable once built; a cached layout pins it).
    uint32_t* plan_mask;      // [Tmax]
    int32_t* plan_rank_ord;   // [Tmax, P]
    int32_t* plan_exp_idx;    // [Tmax, K]
    int32_t* plan_exp_ord;    // [Tmax, K]
    int32_t* plan_counts;     // [P + E]
    int32_t* plan_chan_counts;// [C, P]
    int32_t* plan_chan_remote;// [C]
    int32_t* plan_chan_relay; // [C, N]: own tokens of each channel bound for each other domain (relay mode)

    int32_t* chan_remote_tokens;  // scratch [C, ceil(Tmax / C)]: ring history for slot reuse
    TransportQueues* queues;
    uint64_t* layout_flags;       // prologue scratch: one epoch-tagged flag per token chunk
    int32_t* layout_records;      // prologue scratch: per-chunk bin totals
    int worker_groups;            // payload workgroups after the C control workgroups (spread over the XCDs)
    int tx_waves, rx_waves;       // payload wavefronts per payload workgroup
    int local_groups;             // workgroups after those, for the local bypass and padding (>= 1)

    uint16_t* unique_payload;
    int64_t* unique_topk_idx;
    float* unique_topk_weights;
    int64_t* unique_source_meta;
    int32_t* unique_expert_ordinals;
    uint16_t* expanded_payload;
    int64_t* expanded_expert_idx;
    float* expanded_weights;
    int64_t* expanded_source_meta;
    int64_t expanded_capacity;
    int64_t* unique_count;
    int64_t* expanded_count;
    int32_t* expert_prefix;
    int32_t* expert_counts;
    int32_t* expert_offsets;
    int32_t* source_offsets;
    int32_t* source_expert_prefix;
    int64_t* errors;
    int64_t* stats;
    int64_t* transport_timestamps_ns;
    int32_t* expected_receive_counts;
    int64_t* channel_stats;
    int64_t* channel_timestamps_ns;
    int64_t* receive_expand_overlap;
    uint64_t* receive_prefix_state;
    int64_t* prefix_tx_timestamps_ns;

#if PCIE_EP_ENABLE_PROFILING
    int64_t* profiling;  // [profile_rows(...)][kProfileFields], one row per role wavefront (profiling builds only)
#endif

    // Test hooks, in clock ticks (advanced_common.cuh:118-124).
    uint64_t metadata_delay;
    uint64_t tx_delay;
    uint64_t rx_delay;
    uint64_t scatter_delay;
    uint64_t prefix_delay;
    uint64_t control_abort_after;
};

// ---- clocks and back-off ---------------------------------------------------

__device__ __forceinline__ uint64_t now_ticks() { return wall_clock64(); }
// ticks * 1e6 / kHz without overflowing on absolute clock values.
__device__ __forceinline__ int64_t ticks_to_ns(const DeviceState& state, uint64_t ticks) {
    const uint64_t khz = state.clock_khz;
    return int64_t(ticks / khz * 1000000ull + ticks % khz * 1000000ull / khz);
}
__device__ __forceinline__ void backoff() { __builtin_amdgcn_s_sleep(8); }
// Epoch of the running dispatch.  With the prologue in a launch of its own the epoch word has been advanced when
// the transport kernel starts; inside one launch it still holds the previous epoch until the last role ends.
__device__ __forceinline__ uint64_t dispatch_epoch(const DeviceState& state) { return *state.epoch + uint64_t(state.fused); }
// Workgroups in front of the transport roles when the prologue rides in the transport launch: the epoch begin and one
// per chunk of tokens (one, the leader, also when there is nothing to lay out).
__host__ __device__ __forceinline__ int fused_prologue_groups(const DeviceState& state) {
    return state.fused ? 1 + (state.prologue_chunks > 1 ? state.prologue_chunks : 1) : 0;
}
// Which workgroup runs where.  Consecutive workgroup ids go to consecutive XCDs (eight of them), and everything a
// wavefront sends to memory passes through its XCD's L2 queues, where a host read stays for as long as the host link
// needs for all the bytes requested before it.  A control path that shares an XCD with payload wavefronts therefore
// sees every one of its device-memory operations take that long too - tickets, prefixes and flags arrive tens of
// microseconds late as soon as rows are in flight.  With payload workgroups of their own, the launch therefore
// gives the first kControlXcds XCDs to the control class (epoch begin, layout chunks, channel controls) and the
// other six to the payload class (payload and local-bypass workgroups): workgroup id = row * 8 + XCD; ids that fall
// behind the end of their class are fillers that end at once.  Without payload workgroups the ids are linear.
constexpr int kXcds = 8, kControlXcds = 2;
// Channel control workgroups: one per channel (both of its controls) without payload workgroups of their own;
// with them, one per direction and pair of channels.
__host__ __device__ __forceinline__ int control_groups(const DeviceState& state) {
    const int channels = state.z.dims.channels;
    return state.worker_groups > 0 ? (channels + 1) / 2 * 2 : channels;
}
struct TransportGrid {
    int control_class;   // epoch begin + layout chunks (prologue in this launch) + channel control workgroups
    int payload_class;   // payload workgroups + local-bypass workgroups
    int rows;            // 0: linear ids (control class first)
    int blocks;
};
__host__ __device__ __forceinline__ TransportGrid transport_grid(const DeviceState& state) {
    TransportGrid grid;
    const int payload_groups = state.worker_groups > 0 ? state.worker_groups : 0;
    grid.control_class = fused_prologue_groups(state) + control_groups(state);
    grid.payload_class = payload_groups + state.local_groups;
    if (!payload_groups) {
        grid.rows = 0;
        grid.blocks = grid.control_class + grid.payload_class;
        return grid;
    }
    const int control_rows = (grid.control_class + kControlXcds - 1) / kControlXcds;
    const int payload_rows = (grid.payload_class + kXcds - kControlXcds - 1) / (kXcds - kControlXcds);
    grid.rows = control_rows > payload_rows ? control_rows : payload_rows;
    grid.blocks = grid.rows * kXcds;
    return grid;
}
// Logical index of a workgroup id (control class first, then the payload class), -1 for a filler.
__host__ __device__ __forceinline__ int transport_block(const TransportGrid& grid, int id) {
    if (!grid.rows) return id;
    const int xcd = id % kXcds, row = id / kXcds;
    if (xcd < kControlXcds) {
        const int index = row * kControlXcds + xcd;
        return index < grid.control_class ? index : -1;
    }
    const int index = row * (kXcds - kControlXcds) + xcd - kControlXcds;
    return index < grid.payload_class ? grid.control_class + index : -1;
}
// 32-bit value an epoch-tagged flag word carries (epochs stay below 2^32; the one beyond, which only ends in error 20, still gets a value of its own).
__device__ __forceinline__ uint32_t epoch_flag(uint64_t epoch) { return uint32_t(epoch) + uint32_t(epoch >> 32) * 0x9E3779B9u; }

#if PCIE_EP_ENABLE_PROFILING
// Fields of one role's record.  Times are nanoseconds of the device's wall clock
// (absolute stamps end in Ns, accumulated intervals in Sum); a zero stamp means
// the event did not happen.  Each record has one writer (lane 0 of the role's
// wavefront), is kept in registers and written once when the role ends: no reset
// kernel, fence, barrier or atomic is added (as in the reference).  Intervals of
// different roles overlap and must not be added up.
enum ProfileField : int {
    kProfileEnterNs = 0, kProfileExitNs, kProfileTotalNs, kProfileItems,
    // ---- control wavefronts (rows [0, 2C)) ----
    kProfileFirstTicketNs = 4,   // TX control: first ticket handed out; RX control: first descriptor accepted
    kProfileLastTicketNs,        // ... and the last one
    kProfileWorkersDoneNs,       // TX control: all own rows written and published; RX control: all rows scattered
    kProfileDrainedNs,           // TX control: last payload ACK seen
    kProfileFinishedNs,          // both directions of the channel complete (TX control) / rx_finished stored (RX control)
    kProfilePolls,               // TX control: ACK drain passes; RX control: descriptor polls
    kProfilePollMisses,          // ... that found nothing new
    kProfilePollSum,             // time inside those polls
    kProfileHealthScans, kProfileHealthSum,
    kProfileCountsKnownNs,       // RX control: receive prefixes seen
    kProfileControlSpare,        // (not used)
    // receive-prefix producer (in the record of the RX control that was elected)
    kProfilePrefixEnterNs = 16, kProfilePrefixCountsReadyNs, kProfilePrefixMailboxNs, kProfilePrefixPublishedNs,
    // ---- payload wavefronts (rows [2C, 2C + W)); field 3 = rows moved ----
    kProfileFirstClaimNs = 4,
    kProfileLastRowNs,           // end of this wavefront's last row
    kProfileTxRows, kProfileRxRows,
    kProfileSampledTxRows, kProfileSampledRxRows,  // rows timed in detail (every kProfileSampleStride-th)
    kProfileTicketWaitSum,       // claim -> ticket marked ready (all rows)
    kProfileIdleSum,             // time with nothing to claim
    kProfileTxFlowWaitSum,       // sampled: slot ACK / descriptor credit wait
    kProfileTxCopySum,           // sampled: row + metadata stores issued -> acknowledged by the host
    kProfileRxRequestSum,        // sampled: row loads issued -> metadata and payload returned
    kProfileRxPrefixWaitSum,     // sampled: waiting for the receive prefixes (first rows only)
    kProfileRxScatterSum,        // sampled: row loads issued -> destination rows' stores issued
    kProfileGateOpenNs,          // first received row: the gate in front of the row requests seen open
    // The way of this wavefront's first row, as points in time:
    kProfileFirstLookNs,         // the look at the queues that found the row's ticket
    kProfileFirstTaggedNs,       // ticket claimed and its tag seen ready
    kProfileFirstEntryNs,        // ticket entry read (receive side)
    kProfileFirstRequestNs,      // metadata and first payload loads issued (receive side)
    kProfileFirstDataNs,         // metadata back (receive side)
};
// Record of the prologue's leader workgroup (thread 0), stored behind the payload wavefronts' records.
enum PrologueProfileField : int {
    kPrologueLayoutNs = 4,     // own chunk's ordinals written
    kPrologueTotalsNs,         // totals of all chunks summed
    kPrologueVerdictNs,        // abort words and counts_consumed (host loads issued at entry) looked at
    kPrologueMailboxFreeNs,    // previous count mailbox seen consumed by every peer
    kPrologueMailboxAckedNs,   // count mailbox stores acknowledged by the host
    kPrologueCountsReadyNs,    // counts_ready stored
    kPrologueBegunNs,          // diagnostics cleared, queues reset (and, inside the transport launch, announced)
    kPrologueRoutesNs,         // route ids loaded and checked, hit masks requested
    kPrologueMasksNs,          // hit masks and channel counts of the chunk complete
    kPrologueChunkTotalsNs,    // chunk totals stored (single chunk: the plan's totals)
    kProloguePlanReadyNs,      // inside the transport launch: plan_ready announced
};
// Rows of the table: TX controls [0, C), RX controls [C, 2C), payload wavefronts, prologue leader, epoch begin
// (a record of its own only where the prologue rides in the transport launch; otherwise the leader's holds its stamps),
// producer of the receive prefixes (a record of its own only where it is a wavefront of its own; otherwise the
// prefix fields of the elected RX control's record hold its stamps).
__host__ __device__ inline int profile_rows(int channels, int payload_wavefronts) { return 2 * channels + payload_wavefronts + 3; }
struct RoleProfile {
    uint64_t values[kProfileFields] = {};
    uint64_t khz;
    __device__ explicit RoleProfile(uint64_t clock_khz) : khz(clock_khz) { values[kProfileEnterNs] = now(); }
    __device__ __forceinline__ uint64_t now() const {
        const uint64_t ticks = wall_clock64();
        asm volatile("" ::: "memory");
        return ticks / khz * 1000000ull + ticks % khz * 1000000ull / khz;
    }
    __device__ __forceinline__ void first(int field) { if (!values[field]) values[field] = now(); }
    __device__ __forceinline__ void last(int field) { values[field] = now(); }
    __device__ __forceinline__ void add(int field, uint64_t amount = 1) { values[field] += amount; }
    __device__ void save(int64_t* table, int row, int lane) {
        values[kProfileExitNs] = now();
        values[kProfileTotalNs] = values[kProfileExitNs] - values[kProfileEnterNs];
        if (lane == 0 && table)
            for (int field = 0; field < kProfileFields; ++field) table[size_t(row) * kProfileFields + field] = int64_t(values[field]);
    }
};
#endif

__device__ __forceinline__ void test_delay(uint64_t ticks) {
    if (!ticks) return;
    const uint64_t start = now_ticks();
    while (now_ticks() - start < ticks) __builtin_amdgcn_s_sleep(16);
}

// ---- pinned, fine-grained host memory -----------------------------------------------
// Ordinary loads and stores to the host segments may be served from / parked in
// the GPU's L2 and only become coherent with the CPU through the cache
// write-back and invalidate that full system-scope release / acquire fences
// perform.  On a kernel that is streaming hundreds of MB of expert rows into
// HBM that write-back costs microseconds per signal.  The hot path therefore
// gives every access to host memory the system-scope cache policy (sc0 sc1:
// write-through, never served from a GPU cache):
//   * payload and metadata move through buffer instructions with that policy
//     (host_resource / host_load_* / host_store_*); out-of-range lanes are
//     dropped by the buffer bounds check, so rows need no per-lane predicate;
//   * signals and descriptor fields use system-scope relaxed atomics, which get
//     the same policy;
//   * host_store_release waits until every earlier load has returned and every
//     earlier store has been acknowledged (the counters are wave-wide) and then
//     stores the signal; host_load is a relaxed load whose dependants are issued
//     after it returned.
// The full-fence versions remain for the once-per-dispatch paths (count
// mailbox, receive prefixes), where plain accesses are used.

constexpr int kHostPolicy = 17;  // sc0 | sc1
__device__ __forceinline__ __amdgpu_buffer_rsrc_t host_resource(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, int(bytes), 0x00020000);
}
__device__ __forceinline__ u32x4 host_load_b128(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset) {
    return __builtin_amdgcn_raw_buffer_load_b128(resource, int(byte_offset), 0, kHostPolicy);
}
__device__ __forceinline__ void host_store_b128(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset, u32x4 value) {
    __builtin_amdgcn_raw_buffer_store_b128(value, resource, int(byte_offset), 0, kHostPolicy);
}
__device__ __forceinline__ uint32_t host_load_b32(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset) {
    return __builtin_amdgcn_raw_buffer_load_b32(resource, int(byte_offset), 0, kHostPolicy);
}
__device__ __forceinline__ void host_store_b32(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset, uint32_t value) {
    __builtin_amdgcn_raw_buffer_store_b32(value, resource, int(byte_offset), 0, kHostPolicy);
}
__device__ __forceinline__ uint16_t host_load_b16(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset) {
    return __builtin_amdgcn_raw_buffer_load_b16(resource, int(byte_offset), 0, kHostPolicy);
}
__device__ __forceinline__ void host_store_b16(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset, uint16_t value) {
    __builtin_amdgcn_raw_buffer_store_b16(value, resource, int(byte_offset), 0, kHostPolicy);
}
__device__ __forceinline__ uint8_t host_load_b8(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset) {
    return __builtin_amdgcn_raw_buffer_load_b8(resource, int(byte_offset), 0, kHostPolicy);
}
__device__ __forceinline__ void host_store_b8(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset, uint8_t value) {
    __builtin_amdgcn_raw_buffer_store_b8(value, resource, int(byte_offset), 0, kHostPolicy);
}
template <typename T>
__device__ __forceinline__ T host_field_load(const T* address) {
    return __hip_atomic_load(address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
// The same for an address the compiler cannot trace back to a kernel argument
// (one rebuilt from lane shuffles, say): stating the global address space keeps
// the access a global load instead of a flat one.
__device__ __forceinline__ uint64_t host_load_global(const uint64_t* address) {
    typedef const uint64_t __attribute__((address_space(1))) * GlobalWord;
    return __hip_atomic_load((GlobalWord)address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ int32_t host_field_load_global(const int32_t* address) {
    typedef const int32_t __attribute__((address_space(1))) * GlobalWord;
    return __hip_atomic_load((GlobalWord)address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
template <typename T>
__device__ __forceinline__ void host_field_store(T* address, T value) {
    __hip_atomic_store(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// One 16-byte load from host memory at a per-lane address with the system-scope
// policy, complete on return.  Lanes that read neighbouring entries of a packed
// queue are served by one request per line; a buffer load would need one
// instruction per distinct queue base.
__device__ __forceinline__ u32x4 host_load_b128_at(const void* address) {
    u32x4 value;
    asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(value) : "v"(address) : "memory");
    return value;
}

__device__ __forceinline__ void wait_memory_ops() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void compiler_barrier() { asm volatile("" ::: "memory"); }

__device__ __forceinline__ uint64_t host_load(const uint64_t* address) {
    const uint64_t value = __hip_atomic_load(address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    compiler_barrier();
    return value;
}
__device__ __forceinline__ void host_store_release(uint64_t* address, uint64_t value) {
    wait_memory_ops();
    __hip_atomic_store(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ uint64_t load_acquire_system(const uint64_t* address) {
    return __hip_atomic_load(address, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void store_release_system(uint64_t* address, uint64_t value) {
    __hip_atomic_store(address, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void fence_acquire_system() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, ""); }

// ---- workgroup-scope hand-off through LDS -----------------------------------
// Role wavefronts of one workgroup exchange tickets and counters through LDS.
// The fences are restricted to the LDS address space: a wavefront that has
// megabytes of global loads/stores in flight must not drain them just to bump
// a counter.  Global data handed over together with a ticket is made visible
// explicitly by its writer (wait_memory_ops) and read with device-scope loads.

__device__ __forceinline__ void fence_lds() { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup", "local"); }
__device__ __forceinline__ int lds_load(const int* address) {
    const int value = __hip_atomic_load(address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    return value;
}
__device__ __forceinline__ void lds_store(int* address, int value) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __hip_atomic_store(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// Device-scope (cross-XCD coherent) accesses.  As with host memory, data that
// crosses workgroups is always accessed with the coherent cache policy and
// ordered with wait_memory_ops(), never with cache write-back fences.
constexpr int kDevicePolicy = 16;  // sc1
template <typename T>
__device__ __forceinline__ T device_load(const T* address) {
    return __hip_atomic_load(address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
__device__ __forceinline__ void device_store(T* address, T value) {
    __hip_atomic_store(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The same for an address the compiler cannot trace back to a kernel argument
// (one rebuilt from lane shuffles, say): stating the global address space keeps
// the access a global load instead of a flat one, which would be waited for on
// both memory counters before anything else is issued.
__device__ __forceinline__ int32_t device_load_global(const int32_t* address) {
    typedef const int32_t __attribute__((address_space(1))) * GlobalWord;
    return __hip_atomic_load((GlobalWord)address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t device_add(uint32_t* address, uint32_t value) {
    return __hip_atomic_fetch_add(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t device_resource(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, int(bytes), 0x00020000);
}
__device__ __forceinline__ uint32_t device_load_b32(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset) {
    return __builtin_amdgcn_raw_buffer_load_b32(resource, int(byte_offset), 0, kDevicePolicy);
}
__device__ __forceinline__ void device_store_b32(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset, uint32_t value) {
    __builtin_amdgcn_raw_buffer_store_b32(value, resource, int(byte_offset), 0, kDevicePolicy);
}
// Sixteen bytes as one write-through transaction where four 4-byte ones would each travel to memory alone.
__device__ __forceinline__ void device_store_b128(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset, u32x4 value) {
    __builtin_amdgcn_raw_buffer_store_b128(value, resource, int(byte_offset), 0, kDevicePolicy);
}
__device__ __forceinline__ void plain_store_b128(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset, u32x4 value) {
    __builtin_amdgcn_raw_buffer_store_b128(value, resource, int(byte_offset), 0, 0);
}

// Streaming row accesses in device memory: buffer instructions with the non-temporal
// policy.  Lanes beyond the resource's size read zero / are dropped, so rows need no
// per-lane predicate, and the instruction stream of a row is branch-free.
constexpr int kStreamPolicy = 2;  // nt
__device__ __forceinline__ u32x4 stream_load_b128(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset) {
    return __builtin_amdgcn_raw_buffer_load_b128(resource, int(byte_offset), 0, kStreamPolicy);
}
__device__ __forceinline__ void stream_store_b128(__amdgpu_buffer_rsrc_t resource, uint32_t byte_offset, u32x4 value) {
    __builtin_amdgcn_raw_buffer_store_b128(value, resource, int(byte_offset), 0, kStreamPolicy);
}

// ---- device-scope flags in HBM -----------------------------------------------

__device__ __forceinline__ uint64_t load_acquire_device(const uint64_t* address) {
    return __hip_atomic_load(address, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_release_device(uint64_t* address, uint64_t value) {
    __hip_atomic_store(address, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}
// Relaxed: an acquire here would invalidate caches in every wavefront that
// merely checks whether the dispatch already failed.
__device__ __forceinline__ int64_t load_error_code(const DeviceState& state) {
    return __hip_atomic_load(state.errors, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// First error wins; context fields follow the reference
// (advanced_common.cuh:289-295: errors[1] = local rank, errors[2] = epoch).
__device__ __forceinline__ void record_error(const DeviceState& state, int code, int64_t context = -1, int64_t detail = -1) {
    unsigned long long expected = 0;
    if (atomicCAS(reinterpret_cast<unsigned long long*>(state.errors), expected, static_cast<unsigned long long>(code)) == 0ull) {
        state.errors[1] = context >= 0 ? context : state.local_rank;
        state.errors[2] = detail >= 0 ? detail : int64_t(dispatch_epoch(state));
    }
}

// ---- lane helpers ---------------------------------------------------------------

__device__ __forceinline__ int lane_id() { return int(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u))); }
__device__ __forceinline__ uint64_t lanes_below(int lane) { return lane >= 64 ? ~0ull : ((1ull << lane) - 1ull); }
__device__ __forceinline__ int broadcast_first(int value) { return __builtin_amdgcn_readfirstlane(value); }

// ---- abort flags on the host segments ----------------------------------------------
// Flags per rank: abort, channel_abort[C] and, in relay mode, relay_failed[C][N].
// All 64 lanes load in parallel (the reference scans 32 at a time:
// advanced_common.cuh:350-378).  A scan may be restricted to the flags whose
// index is congruent to `slice` modulo `slices`.
__device__ __forceinline__ int abort_flags_per_rank(const SegmentLayout& z) { return 1 + z.dims.channels * (1 + z.dims.domains); }
__device__ __forceinline__ const uint64_t* abort_flag_at(const SegmentLayout& z, char* segment, int flag) {
    if (flag == 0) return signal_at(segment, z.abort_offset);
    if (flag <= z.dims.channels) return signal_at(segment, z.channel_abort_offset, flag - 1);
    return signal_at(segment, z.relay_failed_offset, flag - 1 - z.dims.channels);
}
__device__ __forceinline__ bool any_abort_wave(const DeviceState& state, int lane, int slice = 0, int slices = 1) {
    const int per_rank = abort_flags_per_rank(state.z);
    const int flags = state.z.dims.num_ranks * per_rank;
    bool aborted = false;
    for (int index = lane; index < flags; index += kWave) {
        if (index % slices != slice) continue;
        aborted |= host_load(abort_flag_at(state.z, state.seg[index / per_rank], index % per_rank)) != 0;
    }
    return __any(aborted);
}

// Bounded failure detection: the local timeout is checked on every call, the
// remote flags at most every min(1 ms, timeout / 8) (advanced_common.cuh:380-429).
// Waits for one named signal (counts_ready, the count mailbox) use the plain
// timeout and report their own code; generic progress waits (ring progress,
// ticket hand-off) add a quarter, so that when a named signal is missing the
// specific code is recorded first rather than whichever wait started earliest.
//
// The C channel guardians of the transport kernel share one device-side abort
// word, so they also share the scanning: guardian `member` of `members` reads
// one slice of the P * (1 + C) flags per scan and moves to the next slice on the
// next scan.  Every flag is still read once per interval while all guardians
// run, and by every surviving guardian within `members` intervals, but the
// host-link reads spent on scanning shrink by the number of channels (at 32
// channels and 8 ranks: 17 KB instead of 540 KB per millisecond).
__device__ __forceinline__ uint64_t progress_timeout_ticks(const DeviceState& state) {
    return state.timeout_ticks + state.timeout_ticks / 4;
}
struct HealthCheck {
    uint64_t start;
    uint64_t next_scan;
    uint64_t interval;
    uint64_t limit;
    int member, members, scans;
    __device__ __forceinline__ HealthCheck(const DeviceState& state, uint64_t begin, bool progress_wait = false, int member_ = 0, int members_ = 1)
        : start(begin), member(member_), members(members_), scans(0) {
        const uint64_t cap = state.clock_khz;  // one millisecond
        const uint64_t eighth = state.timeout_ticks / 8;
        interval = eighth < cap ? eighth : cap;
        next_scan = begin + interval;
        limit = progress_wait ? progress_timeout_ticks(state) : state.timeout_ticks;
    }
    __device__ __forceinline__ bool poll(const DeviceState& state, int lane) {
        const uint64_t now = now_ticks();
        if (now - start > limit) return true;
        // `now` differs slightly per lane; take lane 0's verdict for the scan.
        const int scan = broadcast_first(now >= next_scan ? 1 : 0);
        if (!scan) return false;
        const bool failed = any_abort_wave(state, lane, (member + scans) % members, members);
        ++scans;
        next_scan = now_ticks() + interval;
        return failed;
    }
};

// ---- wavefront row movers ----------------------------------------------------------
// One wavefront moves a whole row: every lane keeps up to kPassItems 16-byte
// vectors in registers, all loads of a pass are issued before the first use,
// so a 14 336-byte BF16 row is 14 loads in flight per lane and is read once
// however many expert rows it is scattered to.
constexpr int kPassItems = 16;

struct RowVectors {
    u32x4 v[kPassItems];
};

// Vector index of item j for this lane: j * 64 + lane (consecutive lanes touch
// consecutive 16-byte vectors: 1 KiB contiguous per instruction).
template <bool kNonTemporal>
__device__ __forceinline__ void row_load_vectors(RowVectors& row, const u32x4* source, int first, int count, int lane) {
#pragma unroll
    for (int j = 0; j < kPassItems; ++j) {
        const int index = first + j * kWave + lane;
        if (index < count) row.v[j] = kNonTemporal ? __builtin_nontemporal_load(source + index) : source[index];
    }
}
template <bool kNonTemporal>
__device__ __forceinline__ void row_store_vectors(const RowVectors& row, u32x4* destination, int first, int count, int lane) {
#pragma unroll
    for (int j = 0; j < kPassItems; ++j) {
        const int index = first + j * kWave + lane;
        if (index < count) {
            if (kNonTemporal) __builtin_nontemporal_store(row.v[j], destination + index);
            else destination[index] = row.v[j];
        }
    }
}

// Scalar fall-back for rows whose byte length is not a multiple of 16: the
// same structure with 2-byte items (the reference also falls back to scalar
// copies for such hidden sizes: csrc/kernels/host_staged/fused_receive.cuh:116-126).
constexpr int kPassScalars = 32;
struct RowScalars {
    uint16_t v[kPassScalars];
};

}  // namespace pcie_ep

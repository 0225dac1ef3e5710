// Host side of the runtime and its C ABI (include/pcie_ep_amd.h).
//
// Replaces the host half of the reference's native extension: AdvancedRuntime
// (csrc/buffers/advanced.hpp:44-552), the segment creation / first touch /
// registration helpers (csrc/comm/advanced_shared_memory.hpp:143-288) and the
// pybind module (csrc/runtime.cu:8-29).  Tensor allocation and pool ownership
// live in the caller; this library owns the pinned segments, a few KB of device
// workspace and the host peer emulator.
#include <hip/hip_runtime.h>

#include <linux/mempolicy.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <cctype>
#include <cerrno>
#include <vector>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <algorithm>
#include <memory>
#include <mutex>
#include <string>

#include "../../include/pcie_ep_amd.h"
#include "launch.h"
#include "peers.h"
#include "relay.h"

using namespace pcie_ep;

struct pcie_ep_runtime;

namespace {

thread_local std::string g_last_error;

int set_error(int code, const char* format, ...) {
    char buffer[1024];
    va_list arguments;
    va_start(arguments, format);
    vsnprintf(buffer, sizeof buffer, format, arguments);
    va_end(arguments);
    g_last_error = buffer;
    return code;
}

#define HIP_TRY(expression)                                                                                   \
    do {                                                                                                      \
        hipError_t status_ = (expression);                                                                    \
        if (status_ != hipSuccess)                                                                            \
            return set_error(PCIE_EP_E_HIP, "%s failed: %s", #expression, hipGetErrorString(status_));        \
    } while (0)

// Plan blob sub-layout (the tensors of AdvancedLayout: advanced.hpp:21-41).
struct PlanLayout {
    size_t mask, rank_ord, exp_idx, exp_ord, counts, chan_counts, chan_remote, chan_relay, bytes;
};

PlanLayout plan_layout(const Dimensions& d) {
    PlanLayout p{};
    size_t cursor = 0;
    auto reserve = [&](size_t bytes) {
        const size_t offset = cursor;
        cursor += align_up(bytes, 256);
        return offset;
    };
    const size_t tokens = size_t(d.max_tokens);
    p.mask = reserve(tokens * 4);
    p.rank_ord = reserve(tokens * d.num_ranks * 4);
    p.exp_idx = reserve(tokens * d.topk * 4);
    p.exp_ord = reserve(tokens * d.topk * 4);
    p.counts = reserve(size_t(d.num_ranks + d.num_experts) * 4);
    p.chan_counts = reserve(size_t(d.channels) * d.num_ranks * 4);
    p.chan_remote = reserve(size_t(d.channels) * 4);
    p.chan_relay = reserve(size_t(d.channels) * (d.domains ? d.domains : 1) * 4);
    p.bytes = cursor;
    return p;
}

// Domains of a relay configuration: the distinct known nodes of the ranks in
// ascending order (one placeholder domain when none is known); a rank of unknown
// node belongs to domain 0 (advanced_shared_memory.hpp:98-105).
int numa_domains(const pcie_ep_config& c, int* nodes, int* rank_domain) {
    int count = 0;
    for (int rank = 0; rank < c.num_ranks; ++rank) {
        const int node = c.rank_numa_nodes[rank];
        if (node >= 0 && std::find(nodes, nodes + count, node) == nodes + count) nodes[count++] = node;
    }
    if (!count) nodes[count++] = 0;
    std::sort(nodes, nodes + count);
    for (int rank = 0; rank < c.num_ranks; ++rank) {
        const int* found = std::find(nodes, nodes + count, c.rank_numa_nodes[rank]);
        rank_domain[rank] = found == nodes + count ? 0 : int(found - nodes);
    }
    return count;
}

int check_config(const pcie_ep_config* c, Dimensions& dims) {
    if (!c) return set_error(PCIE_EP_E_INVALID, "config is NULL");
    // advanced.hpp:110-112
    if (!(c->num_ranks >= 1 && c->num_ranks <= kMaxRanks && c->local_rank >= 0 && c->local_rank < c->num_ranks && c->max_tokens > 0 &&
          c->hidden > 0 && c->topk > 0 && c->topk <= kMaxTopk && c->num_experts >= c->num_ranks && c->num_experts <= kMaxExperts &&
          c->num_experts % c->num_ranks == 0))
        return set_error(PCIE_EP_E_INVALID, "unsupported advanced dimensions");
    // advanced_shared_memory.hpp:106-111
    if (c->channels < 1 || c->channels > kMaxChannels) return set_error(PCIE_EP_E_INVALID, "channels must be 1..32");
    if (c->payload_slots <= 0 || c->descriptor_slots <= 0 || c->timeout_ms <= 0)
        return set_error(PCIE_EP_E_INVALID, "invalid advanced capacity or timeout");
    if (c->tx_waves < 0 || c->tx_waves > kMaxTxWaves || c->rx_waves < 0 || c->rx_waves > kMaxRxWaves)
        return set_error(PCIE_EP_E_INVALID, "tx_waves must be 0..%d and rx_waves 0..%d", kMaxTxWaves, kMaxRxWaves);
    if (c->worker_groups < -1 || c->worker_groups > kMaxWorkerGroups)
        return set_error(PCIE_EP_E_INVALID, "worker_groups must be -1..%d", kMaxWorkerGroups);
    if (c->receive_expand_mode < 0 || c->receive_expand_mode > 2) return set_error(PCIE_EP_E_INVALID, "receive_expand_mode must be 0 (pipelined), 1 (vectorized) or 2 (scalar)");
    // Row bytes, slot offsets and the prologue's token keys are 32-bit quantities.
    if (c->hidden > (1 << 24) || c->max_tokens > (1 << 24)) return set_error(PCIE_EP_E_INVALID, "hidden and max_tokens must not exceed 2^24");
    if (c->peer_threads < 0) return set_error(PCIE_EP_E_INVALID, "peer_threads must be non-negative");
    if (c->staging_numa_node < -1 || c->staging_numa_node >= 1024) return set_error(PCIE_EP_E_INVALID, "staging_numa_node must be -1..1023");
    dims = Dimensions{c->num_ranks, c->max_tokens, c->hidden, c->topk, c->num_experts, c->channels, c->payload_slots, c->descriptor_slots,
                      c->wire_fp8 ? 1 : 0};
    if (c->numa_mode != 0 && c->numa_mode != 1) return set_error(PCIE_EP_E_INVALID, "invalid NUMA mode");
    if (c->numa_mode == 1) {
        // advanced_shared_memory.hpp:96-111
        if (c->replica_slots <= 0) return set_error(PCIE_EP_E_INVALID, "invalid advanced capacity or timeout");
        if (c->relay_workers_per_numa < 1 || c->relay_workers_per_numa > c->channels) return set_error(PCIE_EP_E_INVALID, "invalid relay worker count");
        if (c->relay_cpu_count < 0 || c->relay_cpu_count > 64) return set_error(PCIE_EP_E_INVALID, "relay_cpu_count must be 0..64");
        int nodes[kMaxRanks];
        const int count = numa_domains(*c, nodes, dims.rank_domain);
        if (count > kMaxDomains) return set_error(PCIE_EP_E_INVALID, "too many NUMA domains");
        dims.domains = count;
        dims.replica_slots = c->replica_slots;
    }
    return 0;
}

// Launch shape of the transport kernel: explicit values win, 0 selects the
// defaults.  The default number of payload workgroups follows from the row size
// alone (a fixed number of bytes in flight on the host link), in steps of eight
// so that every XCD gets the same number.
struct LaunchShape {
    int tx_waves, rx_waves, worker_groups;
};
LaunchShape resolve_launch_shape(const pcie_ep_config& c) {
    LaunchShape shape{};
    shape.tx_waves = c.tx_waves ? c.tx_waves : kDefaultTxWaves;
    shape.rx_waves = c.rx_waves ? c.rx_waves : kDefaultRxWaves;
    if (c.worker_groups < 0) shape.worker_groups = 0;
    else if (c.worker_groups) shape.worker_groups = c.worker_groups;
    else {
        const int64_t row_bytes = int64_t(c.hidden) * (c.wire_fp8 ? 1 : 2) + 256;  // payload + slot metadata, roughly
        const int64_t waves = (kBytesInFlight + row_bytes - 1) / row_bytes;
        const int64_t per_group = shape.tx_waves + shape.rx_waves;
        int64_t groups = ((waves + per_group - 1) / per_group + 7) / 8 * 8;
        groups = groups < kMinDefaultWorkerGroups ? kMinDefaultWorkerGroups : groups;
        shape.worker_groups = int(groups > kMaxDefaultWorkerGroups ? kMaxDefaultWorkerGroups : groups);
    }
    return shape;
}

// ---- static scratch of the allocation-free dispatch --------------------------------
// One array per GPU, resident from the moment the library's code object is
// loaded until the process ends.  In host code the array's name is only a
// stand-in for the symbol: its device address is looked up once per device
// (static_scratch_of) and every use below goes through that address.
constexpr size_t kStaticScratchBytes = size_t(4) << 20;
constexpr int kStaticScratchDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

std::mutex g_scratch_guard;
unsigned char* g_scratch_address[kStaticScratchDevices] = {};
// The runtime whose dispatch used this GPU's array last; its `scratch_done` event
// says whether that dispatch has finished.
pcie_ep_runtime* g_scratch_user[kStaticScratchDevices] = {};

// Device address of `scratch` on `device`, which must be the current device.
int static_scratch_of(int device, unsigned char** address) {
    if (device < 0 || device >= kStaticScratchDevices)
        return set_error(PCIE_EP_E_INVALID, "device %d is beyond the %d devices the static scratch table covers", device, kStaticScratchDevices);
    std::lock_guard<std::mutex> lock(g_scratch_guard);
    if (!g_scratch_address[device]) {
        void* pointer = nullptr;
        const hipError_t status = hipGetSymbolAddress(&pointer, HIP_SYMBOL(scratch));
        if (status != hipSuccess || !pointer)
            return set_error(PCIE_EP_E_HIP, "hipGetSymbolAddress(scratch) failed on device %d: %s", device, hipGetErrorString(status));
        g_scratch_address[device] = static_cast<unsigned char*>(pointer);
    }
    *address = g_scratch_address[device];
    return 0;
}

// Carve-out of the transport scratch inside one contiguous block: ticket queues,
// prologue flags + records, ring history.  Everything from the start of the
// block up to `clear_bytes` carries epoch-tagged words and must start at zero
// when the block may have been used by another runtime.
struct ScratchCarve {
    size_t queues, layout, history, clear_bytes, bytes;
};
ScratchCarve carve_scratch(const SegmentLayout& z) {
    ScratchCarve c{};
    c.queues = 0;
    c.layout = align_up(sizeof(TransportQueues), 256);
    c.clear_bytes = c.layout + align_up(prologue_flag_bytes(z), 256);
    c.history = c.layout + align_up(prologue_scratch_bytes(z), 256);
    const size_t per_channel = size_t(z.dims.max_tokens + z.dims.channels - 1) / z.dims.channels;
    c.bytes = c.history + align_up(size_t(z.dims.channels) * per_channel * 4, 256);
    return c;
}

// One pinned, fine-grained, GPU-mapped allocation, first touched (and zeroed)
// under a bind policy for `node` when node >= 0.
int pinned_zeroed(size_t bytes, int node, char** out, const char* what) {
    unsigned long node_mask[16] = {};
    const bool bind = node >= 0;
    if (bind) {
        if (node >= 1024) return set_error(PCIE_EP_E_INVALID, "NUMA node %d is out of range", node);
        node_mask[node / 64] = 1ul << (node % 64);
        if (syscall(SYS_set_mempolicy, MPOL_BIND, node_mask, sizeof(node_mask) * 8) != 0)
            return set_error(PCIE_EP_E_INVALID, "set_mempolicy(MPOL_BIND, node %d) failed", node);
    }
    void* pointer = nullptr;
    const unsigned flags = hipHostMallocCoherent | hipHostMallocMapped | hipHostMallocPortable | (bind ? hipHostMallocNumaUser : 0u);
    const hipError_t allocated = hipHostMalloc(&pointer, bytes, flags);
    if (allocated == hipSuccess) std::memset(pointer, 0, bytes);
    if (bind) syscall(SYS_set_mempolicy, MPOL_DEFAULT, nullptr, 0);
    if (allocated != hipSuccess) return set_error(PCIE_EP_E_HIP, "hipHostMalloc of a %zu-byte %s failed: %s", bytes, what, hipGetErrorString(allocated));
    *out = static_cast<char*>(pointer);
    return 0;
}

}  // namespace

struct pcie_ep_runtime {
    pcie_ep_config config{};
    SegmentLayout z{};
    PlanLayout plan{};
    char* segments[kMaxRanks] = {};
    uint64_t* epoch = nullptr;
    int32_t* chan_remote_tokens = nullptr;
    int tx_waves = kDefaultTxWaves, rx_waves = kDefaultRxWaves, worker_groups = kMinDefaultWorkerGroups;
    TransportQueues* queues = nullptr;
    char* layout_scratch = nullptr;
    uint64_t metadata_delay = 0, tx_delay = 0, rx_delay = 0, scatter_delay = 0, prefix_delay = 0, control_abort_after = 0;
    int counts_ack_skip_source = -1;
    // Relay mode: replica payload regions [rank][domain], each bound to its
    // domain's node when that node exists here, and this rank's relay workers.
    char* replica[kMaxRanks * kMaxDomains] = {};
    bool owns_segments = true;  // false: attached to segments of a pcie_ep_segments set, which outlives this runtime
    int domain_node[kMaxDomains] = {};
    bool domain_bound[kMaxDomains] = {};
    std::unique_ptr<NumaRelay> relay;
    std::unique_ptr<PeerEmulator> peers;
    uint64_t clock_khz = 100000;  // wall clock of the device, queried at creation
    unsigned char* static_scratch = nullptr;  // device address of `scratch` on this runtime's GPU
    bool fused = false;  // the prologue rides in the transport launch (one kernel per dispatch)
    bool closed = false;
    uint64_t ticks_of_ns(uint64_t ns) const { return ns / 1000000 * clock_khz + ns % 1000000 * clock_khz / 1000000; }
    // Optional per-kernel timing with HIP events on the launch stream.
    bool timing = false;
    bool timing_valid = false;
    bool timing_expand = false;
    bool timing_split = false;  // the timed dispatch ran the prologue as a kernel of its own
    hipEvent_t marks[4] = {};
    // Recorded behind every dispatch through the static scratch (created with the runtime:
    // that entry point must not allocate).
    hipEvent_t scratch_done = nullptr;
    // Profiling builds: [profile_rows][kProfileFields] records in device memory.
    int64_t* profiling = nullptr;
    int profile_row_count = 0;
};

namespace {



int build_state(pcie_ep_runtime* rt, const pcie_ep_dispatch_args* a, DeviceState& s) {
    const Dimensions& d = rt->z.dims;
    if (rt->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    if (!a) return set_error(PCIE_EP_E_INVALID, "dispatch args are NULL");
    // advanced.hpp:367-380
    if (a->num_tokens < 0 || a->num_tokens > d.max_tokens || (a->num_tokens > 0 && (!a->x || !a->topk_idx)))
        return set_error(PCIE_EP_E_INVALID, "bad advanced input");
    if (a->alignment < 1 || a->alignment > 256) return set_error(PCIE_EP_E_INVALID, "alignment must be in [1,256]");
    if (!a->plan) return set_error(PCIE_EP_E_INVALID, "route plan storage is NULL");
    if (a->zero_padding && !a->expand) return set_error(PCIE_EP_E_INVALID, "zero padding requires expand");
    const void* required[] = {a->unique_payload, a->unique_topk_idx, a->unique_topk_weights, a->unique_source_meta, a->unique_expert_ordinals,
                              a->expanded_payload, a->expanded_expert_idx, a->expanded_weights, a->expanded_source_meta, a->unique_count,
                              a->expanded_count, a->expert_prefix, a->expert_counts, a->expert_offsets, a->source_offsets,
                              a->source_expert_prefix, a->errors, a->stats, a->transport_timestamps_ns, a->expected_receive_counts,
                              a->channel_stats, a->channel_timestamps_ns, a->receive_expand_overlap, a->receive_prefix_state,
                              a->prefix_tx_timestamps_ns};
    for (const void* pointer : required)
        if (!pointer) return set_error(PCIE_EP_E_INVALID, "an output pool pointer is NULL");
    if (a->expanded_capacity_rows <= 0) return set_error(PCIE_EP_E_INVALID, "expanded capacity must be positive");
    // The kernels move rows as 16-byte vectors when the row length allows it and
    // use 8-byte accesses for the 64-bit outputs: refuse pointers they would fault on.
    auto misaligned = [](const void* pointer, uintptr_t alignment) { return pointer && reinterpret_cast<uintptr_t>(pointer) % alignment != 0; };
    const uintptr_t row_alignment = d.hidden % 8 == 0 ? 16 : 2;
    if (misaligned(a->x, row_alignment) || misaligned(a->unique_payload, row_alignment) || misaligned(a->expanded_payload, row_alignment))
        return set_error(PCIE_EP_E_INVALID, "payload pointers must be %d-byte aligned for hidden=%d", int(row_alignment), d.hidden);
    const void* words64[] = {a->topk_idx, a->unique_topk_idx, a->unique_source_meta, a->expanded_expert_idx, a->expanded_source_meta,
                             a->unique_count, a->expanded_count, a->errors, a->stats, a->transport_timestamps_ns, a->channel_stats,
                             a->channel_timestamps_ns, a->receive_expand_overlap, a->receive_prefix_state, a->prefix_tx_timestamps_ns};
    for (const void* pointer : words64)
        if (misaligned(pointer, 8)) return set_error(PCIE_EP_E_INVALID, "a 64-bit array pointer is not 8-byte aligned");
    const void* words32[] = {a->topk_weights, a->unique_topk_weights, a->unique_expert_ordinals, a->expanded_weights, a->expert_prefix,
                             a->expert_counts, a->expert_offsets, a->source_offsets, a->source_expert_prefix, a->expected_receive_counts};
    for (const void* pointer : words32)
        if (misaligned(pointer, 4)) return set_error(PCIE_EP_E_INVALID, "a 32-bit array pointer is not 4-byte aligned");
    if (misaligned(a->plan, 256)) return set_error(PCIE_EP_E_INVALID, "route plan storage must be 256-byte aligned");

    std::memset(&s, 0, sizeof s);
    s.z = rt->z;
    for (int rank = 0; rank < d.num_ranks; ++rank) {
        s.seg[rank] = rt->segments[rank];
        if (d.domains) s.replica_in[rank] = rt->replica[rank * kMaxDomains + d.rank_domain[rt->config.local_rank]];
    }
    s.local_rank = rt->config.local_rank;
    s.queues = rt->queues;
    s.worker_groups = rt->worker_groups;
    s.tx_waves = rt->tx_waves;
    s.rx_waves = rt->rx_waves;
    // One local-bypass wavefront per ~8 own tokens, at most 32 workgroups: the work
    // (HBM only) then ends long before the host link has moved the remote rows.
    {
        const int waves_per_group = transport_threads(s) / kWave;
        const int wanted = (a->num_tokens / 8 + waves_per_group) / waves_per_group;
        s.local_groups = wanted < 1 ? 1 : (wanted > 32 ? 32 : wanted);
    }
    s.fuse_expand = rt->config.fuse_receive_expand ? 1 : 0;
    s.expand = a->expand ? 1 : 0;
    s.alignment = a->alignment;
    s.num_tokens = a->num_tokens;
    s.zero_padding = a->zero_padding ? 1 : 0;
    s.reuse_plan = a->reuse_plan ? 1 : 0;
    s.counts_ack_skip_source = rt->counts_ack_skip_source;
    s.overlap_diagnostic = s.fuse_expand && s.expand && rt->config.receive_expand_mode == 0;
    s.fused = rt->fused ? 1 : 0;
    s.prologue_chunks = (rt->fused && !a->reuse_plan) ? prologue_chunks(rt->z, a->num_tokens, transport_threads(s) / kWave) : 0;
    s.timeout_ticks = uint64_t(rt->config.timeout_ms) * rt->clock_khz;
    s.clock_khz = rt->clock_khz;
    s.epoch = rt->epoch;
    s.x = static_cast<const uint16_t*>(a->x);
    s.topk_idx = a->topk_idx;
    s.topk_weights = a->topk_weights;
    char* plan = static_cast<char*>(a->plan);
    s.plan_mask = reinterpret_cast<uint32_t*>(plan + rt->plan.mask);
    s.plan_rank_ord = reinterpret_cast<int32_t*>(plan + rt->plan.rank_ord);
    s.plan_exp_idx = reinterpret_cast<int32_t*>(plan + rt->plan.exp_idx);
    s.plan_exp_ord = reinterpret_cast<int32_t*>(plan + rt->plan.exp_ord);
    s.plan_counts = reinterpret_cast<int32_t*>(plan + rt->plan.counts);
    s.plan_chan_counts = reinterpret_cast<int32_t*>(plan + rt->plan.chan_counts);
    s.plan_chan_remote = reinterpret_cast<int32_t*>(plan + rt->plan.chan_remote);
    s.plan_chan_relay = reinterpret_cast<int32_t*>(plan + rt->plan.chan_relay);
    s.chan_remote_tokens = rt->chan_remote_tokens;
    s.layout_flags = reinterpret_cast<uint64_t*>(rt->layout_scratch);
    s.layout_records = reinterpret_cast<int32_t*>(rt->layout_scratch + prologue_flag_bytes(rt->z));
    s.unique_payload = static_cast<uint16_t*>(a->unique_payload);
    s.unique_topk_idx = a->unique_topk_idx;
    s.unique_topk_weights = a->unique_topk_weights;
    s.unique_source_meta = a->unique_source_meta;
    s.unique_expert_ordinals = a->unique_expert_ordinals;
    s.expanded_payload = static_cast<uint16_t*>(a->expanded_payload);
    s.expanded_expert_idx = a->expanded_expert_idx;
    s.expanded_weights = a->expanded_weights;
    s.expanded_source_meta = a->expanded_source_meta;
    s.expanded_capacity = a->expanded_capacity_rows;
    s.unique_count = a->unique_count;
    s.expanded_count = a->expanded_count;
    s.expert_prefix = a->expert_prefix;
    s.expert_counts = a->expert_counts;
    s.expert_offsets = a->expert_offsets;
    s.source_offsets = a->source_offsets;
    s.source_expert_prefix = a->source_expert_prefix;
    s.errors = a->errors;
    s.stats = a->stats;
    s.transport_timestamps_ns = a->transport_timestamps_ns;
    s.expected_receive_counts = a->expected_receive_counts;
    s.channel_stats = a->channel_stats;
    s.channel_timestamps_ns = a->channel_timestamps_ns;
    s.receive_expand_overlap = a->receive_expand_overlap;
    s.receive_prefix_state = a->receive_prefix_state;
    s.prefix_tx_timestamps_ns = a->prefix_tx_timestamps_ns;
#if PCIE_EP_ENABLE_PROFILING
    s.profiling = rt->profiling;
#endif
    s.metadata_delay = rt->metadata_delay;
    s.tx_delay = rt->tx_delay;
    s.rx_delay = rt->rx_delay;
    s.scatter_delay = rt->scatter_delay;
    s.prefix_delay = rt->prefix_delay;
    s.control_abort_after = rt->control_abort_after;
    return 0;
}

}  // namespace

extern "C" {

int pcie_ep_abi_version(void) { return PCIE_EP_ABI_VERSION; }

const char* pcie_ep_last_error(void) { return g_last_error.c_str(); }

int pcie_ep_query_sizes(const pcie_ep_config* config, pcie_ep_sizes* sizes) {
    Dimensions dims;
    if (int status = check_config(config, dims)) return status;
    if (!sizes) return set_error(PCIE_EP_E_INVALID, "sizes is NULL");
    const SegmentLayout z = make_segment_layout(dims);
    std::memset(sizes, 0, sizeof *sizes);
    sizes->unique_rows = unique_capacity(dims);
    sizes->expanded_rows = expanded_capacity(dims);
    sizes->plan_bytes = int64_t(plan_layout(dims).bytes);
    sizes->segment_bytes = int64_t(z.size_bytes);
    sizes->slot_stride = int64_t(z.slot_stride);
    sizes->local_experts = z.local_experts;
    sizes->payload_bytes = z.payload_bytes;
    sizes->meta_bytes = z.meta_bytes;
    sizes->mailbox_dwords = z.mailbox_dwords;
    DeviceState probe{};
    const LaunchShape shape = resolve_launch_shape(*config);
    probe.tx_waves = shape.tx_waves;
    probe.rx_waves = shape.rx_waves;
    probe.worker_groups = shape.worker_groups;
    sizes->transport_threads = transport_threads(probe);
    sizes->transport_workgroups = config->channels + probe.worker_groups;
    sizes->num_domains = dims.domains;
    sizes->replica_region_bytes = dims.domains ? int64_t(z.replica_region_bytes) : 0;
    return 0;
}

namespace {

// Allocates the pinned segments of every rank (and, in relay mode, the replica
// regions): first touch by this thread under the requested NUMA policy, then
// zeroed - a zero sequence word means "never written".  A rank's segment belongs
// on the rank's own node and each replica payload region on the node of the
// domain it serves (advanced_shared_memory.hpp:214-262); a node that this machine
// does not have leaves the memory where first touch puts it.
int allocate_segments(const pcie_ep_config& config, const Dimensions& dims, const SegmentLayout& z, char** segments, char** replica,
                      int* domain_node, bool* domain_bound) {
    int status = 0;
    if (dims.domains) {
        int rank_domain[kMaxRanks];
        numa_domains(config, domain_node, rank_domain);
    }
    for (int rank = 0; rank < dims.num_ranks && !status; ++rank) {
        int node = config.staging_numa_node;
        if (node < 0 && dims.domains && numa_node_exists(config.rank_numa_nodes[rank])) node = config.rank_numa_nodes[rank];
        status = pinned_zeroed(z.size_bytes, node, &segments[rank], "source segment");
        for (int domain = 0; domain < dims.domains && !status; ++domain) {
            const bool present = numa_node_exists(domain_node[domain]);
            domain_bound[domain] = present;
            status = pinned_zeroed(z.replica_region_bytes, present ? domain_node[domain] : -1, &replica[rank * kMaxDomains + domain], "replica region");
        }
    }
    return status;
}

int free_segments(char** segments, char** replica) {
    int status = 0;
    for (int rank = 0; rank < kMaxRanks; ++rank) {
        if (segments[rank] && hipHostFree(segments[rank]) != hipSuccess) status = set_error(PCIE_EP_E_HIP, "hipHostFree of a source segment failed");
        segments[rank] = nullptr;
    }
    for (int index = 0; index < kMaxRanks * kMaxDomains; ++index) {
        if (replica[index] && hipHostFree(replica[index]) != hipSuccess) status = set_error(PCIE_EP_E_HIP, "hipHostFree of a replica region failed");
        replica[index] = nullptr;
    }
    return status;
}

int create_runtime(const pcie_ep_config* config, const pcie_ep_segments* attached, pcie_ep_runtime** out);

}  // namespace

int pcie_ep_runtime_create(const pcie_ep_config* config, pcie_ep_runtime** out) { return create_runtime(config, nullptr, out); }

int pcie_ep_runtime_attach(const pcie_ep_config* config, const pcie_ep_segments* segments, pcie_ep_runtime** out) {
    if (!segments) return set_error(PCIE_EP_E_INVALID, "segments is NULL");
    return create_runtime(config, segments, out);
}

int pcie_ep_segments_create(const pcie_ep_config* config, pcie_ep_segments* out) {
    Dimensions dims;
    if (int status = check_config(config, dims)) return status;
    if (!out) return set_error(PCIE_EP_E_INVALID, "segments output pointer is NULL");
    int device_count = 0;
    if (hipGetDeviceCount(&device_count) != hipSuccess || device_count <= config->device)
        return set_error(PCIE_EP_E_HIP, "no HIP device %d is available: the host-staged runtime needs a GPU", config->device);
    HIP_TRY(hipSetDevice(config->device));
    std::memset(out, 0, sizeof *out);
    static_assert(sizeof(out->segment) / sizeof(void*) == kMaxRanks && sizeof(out->replica) / sizeof(void*) == kMaxRanks * kMaxDomains,
                  "pcie_ep_segments is sized by the wire limits");
    const SegmentLayout z = make_segment_layout(dims);
    int domain_node[kMaxDomains] = {};
    bool domain_bound[kMaxDomains] = {};
    const int status = allocate_segments(*config, dims, z, reinterpret_cast<char**>(out->segment), reinterpret_cast<char**>(out->replica), domain_node,
                                         domain_bound);
    if (status) (void)free_segments(reinterpret_cast<char**>(out->segment), reinterpret_cast<char**>(out->replica));
    return status;
}

int pcie_ep_segments_destroy(pcie_ep_segments* segments) {
    if (!segments) return 0;
    return free_segments(reinterpret_cast<char**>(segments->segment), reinterpret_cast<char**>(segments->replica));
}

namespace {

int create_runtime(const pcie_ep_config* config, const pcie_ep_segments* attached, pcie_ep_runtime** out) {
    Dimensions dims;
    if (int status = check_config(config, dims)) return status;
    if (!out) return set_error(PCIE_EP_E_INVALID, "runtime output pointer is NULL");
    *out = nullptr;
    int device_count = 0;
    if (hipGetDeviceCount(&device_count) != hipSuccess || device_count <= config->device)
        return set_error(PCIE_EP_E_HIP, "no HIP device %d is available: the host-staged runtime needs a GPU", config->device);
    HIP_TRY(hipSetDevice(config->device));
    auto rt = std::make_unique<pcie_ep_runtime>();
    rt->config = *config;
    // Once per device, with that device current: where this GPU keeps its copy of the static scratch.
    if (int status = static_scratch_of(config->device, &rt->static_scratch)) return status;
    // Every device-side timeout, back-off period and timestamp is derived from the
    // rate of the constant wall clock the kernels read.
    int clock_khz = 0;
    HIP_TRY(hipDeviceGetAttribute(&clock_khz, hipDeviceAttributeWallClockRate, config->device));
    if (clock_khz <= 0) return set_error(PCIE_EP_E_HIP, "device %d reports no wall clock rate", config->device);
    rt->clock_khz = uint64_t(clock_khz);
    rt->z = make_segment_layout(dims);
    rt->plan = plan_layout(dims);
    const LaunchShape shape = resolve_launch_shape(*config);
    rt->tx_waves = shape.tx_waves;
    rt->rx_waves = shape.rx_waves;
    rt->worker_groups = shape.worker_groups;
    {
        DeviceState probe{};
        probe.z = rt->z;
        probe.tx_waves = rt->tx_waves;
        probe.rx_waves = rt->rx_waves;
        probe.worker_groups = rt->worker_groups;
        // One launch per dispatch wherever the prologue fits into the transport launch and the whole grid
        // (epoch begin, prologue chunks of a full batch, control, payload and local-bypass workgroups) is resident at once.
        const int block_threads = transport_threads(probe);
        rt->fused = !config->split_launch && fused_prologue_fits(rt->z, block_threads, dims.max_tokens) &&
                    1 + prologue_chunks(rt->z, dims.max_tokens, block_threads / kWave) + control_groups(probe) + (rt->worker_groups > 0 ? rt->worker_groups : 0) + 32 <= 256;
    }

    // Pinned, fine-grained, GPU-mapped segments (the reference registers
    // /dev/shm mappings: advanced_shared_memory.hpp:264-288): this runtime's own, or
    // those of a set that several runtimes share (advanced_shared_memory.hpp:235-262:
    // attach validates the header a creator wrote; here the creator's struct is the
    // proof, and what is checked is that every pointer this rank will use is there).
    int status = 0;
    if (attached) {
        if (config->peer_threads > 0)
            return set_error(PCIE_EP_E_INVALID, "an attached runtime has real peers: peer_threads must be 0");
        rt->owns_segments = false;
        if (dims.domains) {
            int rank_domain[kMaxRanks];
            numa_domains(*config, rt->domain_node, rank_domain);
        }
        for (int rank = 0; rank < dims.num_ranks; ++rank) {
            rt->segments[rank] = static_cast<char*>(attached->segment[rank]);
            if (!rt->segments[rank]) return set_error(PCIE_EP_E_INVALID, "segment of rank %d is NULL", rank);
            for (int domain = 0; domain < dims.domains; ++domain) {
                rt->replica[rank * kMaxDomains + domain] = static_cast<char*>(attached->replica[rank * kMaxDomains + domain]);
                if (!rt->replica[rank * kMaxDomains + domain]) return set_error(PCIE_EP_E_INVALID, "replica region %d of rank %d is NULL", domain, rank);
            }
        }
    } else {
        status = allocate_segments(*config, dims, rt->z, rt->segments, rt->replica, rt->domain_node, rt->domain_bound);
    }
    if (!status) {
        const size_t history = size_t(dims.channels) * ((dims.max_tokens + dims.channels - 1) / dims.channels) * 4;
        hipError_t error = hipMalloc(reinterpret_cast<void**>(&rt->epoch), 256);
        if (error == hipSuccess) error = hipMemset(rt->epoch, 0, 256);
        if (error == hipSuccess) error = hipMalloc(reinterpret_cast<void**>(&rt->chan_remote_tokens), history);
        if (error == hipSuccess) error = hipMemset(rt->chan_remote_tokens, 0, history);
        if (error == hipSuccess) error = hipMalloc(reinterpret_cast<void**>(&rt->queues), sizeof(TransportQueues));
        if (error == hipSuccess) error = hipMemset(rt->queues, 0, sizeof(TransportQueues));
        if (error == hipSuccess) error = hipMalloc(reinterpret_cast<void**>(&rt->layout_scratch), prologue_scratch_bytes(rt->z));
        if (error == hipSuccess) error = hipMemset(rt->layout_scratch, 0, prologue_scratch_bytes(rt->z));
        if (error == hipSuccess) error = hipEventCreateWithFlags(&rt->scratch_done, hipEventDisableTiming);
#if PCIE_EP_ENABLE_PROFILING
        rt->profile_row_count = profile_rows(dims.channels, (rt->worker_groups > 0 ? rt->worker_groups : dims.channels) * (rt->tx_waves + rt->rx_waves));
        const size_t profile_bytes = size_t(rt->profile_row_count) * kProfileFields * sizeof(int64_t);
        if (error == hipSuccess) error = hipMalloc(reinterpret_cast<void**>(&rt->profiling), profile_bytes);
        if (error == hipSuccess) error = hipMemset(rt->profiling, 0, profile_bytes);
#endif
        if (error == hipSuccess) error = hipDeviceSynchronize();
        if (error != hipSuccess) status = set_error(PCIE_EP_E_HIP, "device workspace allocation failed: %s", hipGetErrorString(error));
    }
    if (status) {
        if (rt->owns_segments) (void)free_segments(rt->segments, rt->replica);
        if (rt->epoch) (void)hipFree(rt->epoch);
        if (rt->chan_remote_tokens) (void)hipFree(rt->chan_remote_tokens);
        if (rt->queues) (void)hipFree(rt->queues);
        if (rt->layout_scratch) (void)hipFree(rt->layout_scratch);
        if (rt->scratch_done) (void)hipEventDestroy(rt->scratch_done);
        if (rt->profiling) (void)hipFree(rt->profiling);
        return status;
    }
    RelayOptions relay_options;
    relay_options.workers_per_domain = config->relay_workers_per_numa > 0 ? config->relay_workers_per_numa : 1;
    relay_options.timeout_ms = config->timeout_ms;
    relay_options.delay_ns = config->relay_delay_ns;
    relay_options.cpus.assign(config->relay_cpus, config->relay_cpus + (dims.domains ? config->relay_cpu_count : 0));
    std::copy(rt->domain_node, rt->domain_node + kMaxDomains, relay_options.domain_node);
    // This rank's relay workers start before the first dispatch and wait for
    // epoch 1 (advanced.hpp:113-115).
    if (dims.domains)
        rt->relay = std::make_unique<NumaRelay>(rt->z, config->local_rank, rt->segments, rt->replica + config->local_rank * kMaxDomains, relay_options);
    if (config->peer_threads > 0 && dims.num_ranks > 1)
        rt->peers = std::make_unique<PeerEmulator>(rt->z, config->local_rank, rt->segments, rt->replica, config->peer_threads, config->timeout_ms,
                                                   relay_options);
    *out = rt.release();
    return 0;
}

}  // namespace

int pcie_ep_runtime_destroy(pcie_ep_runtime* rt) {
    if (!rt) return 0;
    rt->closed = true;
    // Tell the relay workers of every rank to stop before their memory goes away
    // (the reference's destructor raises relay_failed = 199: advanced.hpp:256-262).
    if (rt->relay) rt->relay->stop_and_join();
    rt->peers.reset();  // joins the emulator threads before the segments go away
    rt->relay.reset();
    int status = 0;
    if (rt->owns_segments) status = free_segments(rt->segments, rt->replica);
    if (rt->epoch) (void)hipFree(rt->epoch);
    if (rt->chan_remote_tokens) (void)hipFree(rt->chan_remote_tokens);
    if (rt->queues) (void)hipFree(rt->queues);
    if (rt->layout_scratch) (void)hipFree(rt->layout_scratch);
    for (hipEvent_t mark : rt->marks)
        if (mark) (void)hipEventDestroy(mark);
    {
        std::lock_guard<std::mutex> lock(g_scratch_guard);
        for (pcie_ep_runtime*& user : g_scratch_user)
            if (user == rt) user = nullptr;
    }
    if (rt->scratch_done) (void)hipEventDestroy(rt->scratch_done);
    if (rt->profiling) (void)hipFree(rt->profiling);
    delete rt;
    return status;
}

int pcie_ep_dispatch(pcie_ep_runtime* rt, const pcie_ep_dispatch_args* args, void* stream_handle) {
    if (!rt) return set_error(PCIE_EP_E_INVALID, "runtime is NULL");
    DeviceState state;
    if (int status = build_state(rt, args, state)) return status;
    hipStream_t stream = static_cast<hipStream_t>(stream_handle);
    // Kernel sequence of launch_dispatch (advanced.hpp:472-523), two launches:
    //   prologue  = begin_epoch + route_flags + stable_ordinals + prepare_channels + publish_counts
    //   transport = the channel kernel: TX, RX, receive prefixes, fused expand, and - in TX
    //               wavefronts that have run out of tickets - copy_local_tokens + zero_padding;
    //               its last wavefront does reduce_statistics
    // and the separate expand when receive/expand fusion is off.
    const bool timed = rt->timing;
    rt->timing_valid = false;
    if (timed) HIP_TRY(hipEventRecord(rt->marks[0], stream));
    if (!state.fused) HIP_TRY(launch_prologue(state, stream));
    // One launch per dispatch: the prologue rides in the transport launch and has no span of its own.
    if (timed && !state.fused) HIP_TRY(hipEventRecord(rt->marks[1], stream));
    HIP_TRY(launch_transport(state, stream));
    if (timed) HIP_TRY(hipEventRecord(rt->marks[2], stream));
    const bool separate_expand = state.expand && !state.fuse_expand;
    if (separate_expand) HIP_TRY(launch_expand(state, stream));
    if (timed) {
        HIP_TRY(hipEventRecord(rt->marks[3], stream));
        rt->timing_expand = separate_expand;
        rt->timing_split = !state.fused;
        rt->timing_valid = true;
    }
    return 0;
}

int pcie_ep_dispatch_static_scratch(pcie_ep_runtime* rt, const pcie_ep_dispatch_args* args, void* stream_handle) {
    if (!rt) return set_error(PCIE_EP_E_INVALID, "runtime is NULL");
    DeviceState state;
    if (int status = build_state(rt, args, state)) return status;
    const ScratchCarve carve = carve_scratch(rt->z);
    if (carve.bytes > kStaticScratchBytes)
        return set_error(PCIE_EP_E_INVALID,
                         "this configuration needs %zu bytes of transport scratch, more than the %zu bytes of the static scratch; use pcie_ep_dispatch",
                         carve.bytes, kStaticScratchBytes);
    // The kernels take the scratch as pointers, exactly as in pcie_ep_dispatch;
    // here they point into this GPU's static array instead of the runtime's own
    // allocations.  Only the epoch counter, which is state of the host rings and
    // not scratch, stays where pcie_ep_runtime_create put it.
    hipStream_t stream = static_cast<hipStream_t>(stream_handle);
    // Every runtime on this GPU shares the one array.  A dispatch of ANOTHER runtime
    // that has not finished yet would have its ticket queues cleared under it: refuse
    // instead.  (Calls of one runtime are ordered by its caller anyway.)  Under stream
    // capture nothing executes now and an event cannot be queried: the check is
    // skipped there, and replays of such a graph are the caller's to order.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    HIP_TRY(hipStreamIsCapturing(stream, &capture));
    const bool capturing = capture != hipStreamCaptureStatusNone;
    std::lock_guard<std::mutex> scratch_lock(g_scratch_guard);
    if (!capturing) {
        pcie_ep_runtime* last = g_scratch_user[rt->config.device];
        if (last && last != rt && hipEventQuery(last->scratch_done) == hipErrorNotReady)
            return set_error(PCIE_EP_E_STATE, "the static scratch of device %d is in use by a dispatch of another runtime that has not finished",
                             rt->config.device);
    }
    // Per-kernel timing is not recorded here; stamps of an earlier ordinary dispatch must not pass for this one's.
    rt->timing_valid = false;
    unsigned char* base = rt->static_scratch;
    state.queues = reinterpret_cast<TransportQueues*>(base + carve.queues);
    state.layout_flags = reinterpret_cast<uint64_t*>(base + carve.layout);
    state.layout_records = reinterpret_cast<int32_t*>(base + carve.layout + prologue_flag_bytes(rt->z));
    state.chan_remote_tokens = reinterpret_cast<int32_t*>(base + carve.history);
    // The array keeps what its last user left, possibly another runtime whose
    // epoch numbers coincide with this one's: the epoch-tagged words (ticket ring
    // tags, queue counters, prologue chunk flags) start from zero.  A fill kernel,
    // not a memset, so the call may be captured into a graph.
    HIP_TRY(launch_zero(base, carve.clear_bytes, stream));
    if (!state.fused) HIP_TRY(launch_prologue(state, stream));
    HIP_TRY(launch_transport(state, stream));
    if (state.expand && !state.fuse_expand) HIP_TRY(launch_expand(state, stream));
    if (!capturing) {
        HIP_TRY(hipEventRecord(rt->scratch_done, stream));
        g_scratch_user[rt->config.device] = rt;
    }
    return 0;
}

int pcie_ep_transport_residency(pcie_ep_runtime* rt, int32_t compute_units, int32_t* needed, int32_t* resident) {
    if (!rt || rt->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    if (!needed || !resident || compute_units < 0) return set_error(PCIE_EP_E_INVALID, "bad residency arguments");
    HIP_TRY(hipSetDevice(rt->config.device));
    int units = compute_units;
    if (!units) HIP_TRY(hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, rt->config.device));
    DeviceState probe{};
    probe.z = rt->z;
    probe.tx_waves = rt->tx_waves;
    probe.rx_waves = rt->rx_waves;
    probe.worker_groups = rt->worker_groups;
    probe.fused = rt->fused ? 1 : 0;
    int per_unit = 0;
    HIP_TRY(transport_workgroups_per_unit(probe, &per_unit));
    // The control and payload workgroups wait for each other through device memory
    // and must run together; the local-bypass workgroups behind them may start late.
    *needed = control_groups(probe) + (rt->worker_groups > 0 ? rt->worker_groups : 0) +
              (rt->fused ? 1 + std::max(1, prologue_chunks(rt->z, rt->z.dims.max_tokens, rt->tx_waves + rt->rx_waves)) : 0);
    *resident = per_unit * units;
    return 0;
}

int pcie_ep_profile_shape(pcie_ep_runtime* rt, int32_t* rows, int32_t* fields, int32_t* channels, int32_t* payload_wavefronts) {
    if (!rt || rt->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    if (!rows || !fields || !channels || !payload_wavefronts) return set_error(PCIE_EP_E_INVALID, "bad profile arguments");
    *rows = rt->profile_row_count;  // 0: the library was built without PCIE_EP_ENABLE_PROFILING
    *fields = kProfileFields;
    *channels = rt->z.dims.channels;
    *payload_wavefronts = (rt->worker_groups > 0 ? rt->worker_groups : rt->z.dims.channels) * (rt->tx_waves + rt->rx_waves);
    return 0;
}

int pcie_ep_profile_read(pcie_ep_runtime* rt, int64_t* records) {
    if (!rt || rt->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    if (!rt->profiling) return set_error(PCIE_EP_E_STATE, "this library was built without PCIE_EP_ENABLE_PROFILING");
    if (!records) return set_error(PCIE_EP_E_INVALID, "bad profile arguments");
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(records, rt->profiling, size_t(rt->profile_row_count) * kProfileFields * sizeof(int64_t), hipMemcpyDeviceToHost));
    return 0;
}

int pcie_ep_graph_launch(void* graph_exec, void* stream) {
    if (!graph_exec) return set_error(PCIE_EP_E_INVALID, "graph_exec is NULL");
    HIP_TRY(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), static_cast<hipStream_t>(stream)));
    return 0;
}

int pcie_ep_set_kernel_timing(pcie_ep_runtime* rt, int32_t enable) {
    if (!rt || rt->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    if (enable && !rt->marks[0])
        for (hipEvent_t& mark : rt->marks) HIP_TRY(hipEventCreate(&mark));
    rt->timing = enable != 0;
    rt->timing_valid = false;
    return 0;
}

int pcie_ep_get_kernel_times(pcie_ep_runtime* rt, float* milliseconds) {
    if (!rt || rt->closed || !milliseconds) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    if (!rt->timing_valid) return set_error(PCIE_EP_E_STATE, "no timed dispatch has been recorded");
    HIP_TRY(hipEventSynchronize(rt->marks[3]));
    milliseconds[0] = milliseconds[1] = milliseconds[2] = 0.0f;
    if (rt->timing_split) HIP_TRY(hipEventElapsedTime(milliseconds + 0, rt->marks[0], rt->marks[1]));
    HIP_TRY(hipEventElapsedTime(milliseconds + 1, rt->marks[rt->timing_split ? 1 : 0], rt->marks[2]));
    if (rt->timing_expand) HIP_TRY(hipEventElapsedTime(milliseconds + 2, rt->marks[2], rt->marks[3]));
    return 0;
}

int pcie_ep_expand_unique(pcie_ep_runtime* rt, const pcie_ep_dispatch_args* args, void* stream_handle) {
    if (!rt) return set_error(PCIE_EP_E_INVALID, "runtime is NULL");
    DeviceState state;
    if (int status = build_state(rt, args, state)) return status;
    state.expand = 1;
    HIP_TRY(launch_expand(state, static_cast<hipStream_t>(stream_handle)));
    return 0;
}

int pcie_ep_set_test_delays(pcie_ep_runtime* rt, uint64_t metadata_ns, uint64_t tx_ns, uint64_t rx_ns, uint64_t scatter_ns) {
    if (!rt) return set_error(PCIE_EP_E_INVALID, "runtime is NULL");
    rt->metadata_delay = rt->ticks_of_ns(metadata_ns);
    rt->tx_delay = rt->ticks_of_ns(tx_ns);
    rt->rx_delay = rt->ticks_of_ns(rx_ns);
    rt->scatter_delay = rt->ticks_of_ns(scatter_ns);
    return 0;
}
int pcie_ep_set_test_prefix_delay_ns(pcie_ep_runtime* rt, uint64_t delay_ns) {
    if (!rt) return set_error(PCIE_EP_E_INVALID, "runtime is NULL");
    rt->prefix_delay = rt->ticks_of_ns(delay_ns);
    return 0;
}
int pcie_ep_set_test_control_abort_after_ns(pcie_ep_runtime* rt, uint64_t delay_ns) {
    if (!rt) return set_error(PCIE_EP_E_INVALID, "runtime is NULL");
    rt->control_abort_after = rt->ticks_of_ns(delay_ns);
    return 0;
}
int pcie_ep_set_test_skip_counts_ack_source(pcie_ep_runtime* rt, int32_t source) {
    if (!rt) return set_error(PCIE_EP_E_INVALID, "runtime is NULL");
    if (source < -1 || source >= rt->z.dims.num_ranks) return set_error(PCIE_EP_E_INVALID, "invalid test counts source");
    rt->counts_ack_skip_source = source;
    return 0;
}

int pcie_ep_set_test_epoch(pcie_ep_runtime* rt, uint64_t epoch) {
    if (!rt || rt->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(rt->epoch, &epoch, sizeof epoch, hipMemcpyHostToDevice));
    return 0;
}

static int page_node(const void* address) {
    int node = -1;
    if (syscall(SYS_get_mempolicy, &node, nullptr, 0ul, address, MPOL_F_NODE | MPOL_F_ADDR) != 0) return -errno;
    return node;
}

int pcie_ep_relay_diagnostics(pcie_ep_runtime* rt, pcie_ep_relay_summary* summary, pcie_ep_relay_flow* flows, int32_t capacity) {
    if (!rt || rt->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    if (!summary || capacity < 0 || (capacity && !flows)) return set_error(PCIE_EP_E_INVALID, "bad relay diagnostics arguments");
    static_assert(sizeof(pcie_ep_relay_flow) == sizeof(RelayFlowRecord), "relay flow record layout");
    std::memset(summary, 0, sizeof *summary);
    const Dimensions& d = rt->z.dims;
    summary->enabled = d.domains ? 1 : 0;
    summary->rank = rt->config.local_rank;
    summary->num_domains = d.domains;
    summary->slot_stride = int64_t(rt->z.slot_stride);
    summary->segment_bytes = int64_t(rt->z.size_bytes);
    summary->replica_region_bytes = d.domains ? int64_t(rt->z.replica_region_bytes) : 0;
    for (int rank = 0; rank < kMaxRanks; ++rank) summary->rank_numa_nodes[rank] = rank < d.num_ranks ? rt->config.rank_numa_nodes[rank] : -1;
    if (!rt->relay) return 0;
    char* own = rt->segments[rt->config.local_rank];
    summary->source_page_node = page_node(own + rt->z.slots_offset);
    for (int domain = 0; domain < d.domains; ++domain) {
        summary->domain_numa_nodes[domain] = rt->domain_node[domain];
        summary->domain_bound[domain] = rt->domain_bound[domain] ? 1 : 0;
        summary->replica_page_node[domain] = page_node(rt->replica[rt->config.local_rank * kMaxDomains + domain]);
    }
    summary->workers = rt->relay->workers();
    summary->flows = rt->relay->flows();
    summary->epoch = rt->relay->ready_epoch();
    std::vector<RelayFlowRecord> records(size_t(summary->flows));
    rt->relay->diagnostics(records.data(), summary->flows);
    for (int index = 0; index < summary->flows; ++index) {
        const RelayFlowRecord& r = records[size_t(index)];
        if (r.epoch == summary->epoch) {
            summary->copies += r.copied_tokens;
            summary->payload_bytes += r.copied_payload_bytes;
        }
        summary->copies_total += r.copies_total;
        summary->payload_bytes_total += r.payload_bytes_total;
        if (index < capacity) std::memcpy(flows + index, &r, sizeof r);
    }
    const std::string errors = rt->relay->worker_errors();
    if (!errors.empty()) return set_error(PCIE_EP_E_PROTOCOL, "relay worker failed: %s", errors.c_str());
    return 0;
}

int pcie_ep_set_relay_delay_ns(pcie_ep_runtime* rt, uint64_t delay_ns) {
    if (!rt || rt->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");
    if (!rt->relay) return set_error(PCIE_EP_E_STATE, "NUMA relay is not enabled");
    rt->relay->set_delay(delay_ns);
    return 0;
}

int pcie_ep_device_numa_node(int32_t device) {
    char bus_id[64] = {};
    if (hipDeviceGetPCIBusId(bus_id, sizeof bus_id, device) != hipSuccess) return -1;
    std::string bus = bus_id;
    for (auto& character : bus) character = char(std::tolower(character));
    std::ifstream file("/sys/bus/pci/devices/" + bus + "/numa_node");
    int node = -1;
    file >> node;
    return node;
}

static uint64_t* host_signal(pcie_ep_runtime* rt, int32_t segment_rank, int32_t which, int32_t index) {
    if (!rt || rt->closed || segment_rank < 0 || segment_rank >= rt->z.dims.num_ranks) return nullptr;
    char* segment = rt->segments[segment_rank];
    switch (which) {
        case 0: return signal_at(segment, rt->z.abort_offset);
        case 1: return index >= 0 && index < rt->z.dims.channels ? signal_at(segment, rt->z.channel_abort_offset, index) : nullptr;
        case 2: return signal_at(segment, rt->z.counts_ready_offset);
        case 3: return index >= 0 && index < rt->z.dims.num_ranks ? signal_at(segment, rt->z.counts_consumed_offset, index) : nullptr;
        case 4: return index >= 0 && index < rt->z.dims.channels * rt->z.dims.domains ? signal_at(segment, rt->z.relay_failed_offset, index) : nullptr;
        case 5: return index >= 0 && index < rt->z.dims.channels * rt->z.dims.domains ? signal_at(segment, rt->z.relay_drained_offset, index) : nullptr;
        default: return nullptr;
    }
}

int pcie_ep_host_signal_store(pcie_ep_runtime* rt, int32_t segment_rank, int32_t which, int32_t index, uint64_t value) {
    uint64_t* signal = host_signal(rt, segment_rank, which, index);
    if (!signal) return set_error(PCIE_EP_E_INVALID, "no such host signal");
    std::atomic_ref<uint64_t>(*signal).store(value, std::memory_order_release);
    return 0;
}
int pcie_ep_host_signal_load(pcie_ep_runtime* rt, int32_t segment_rank, int32_t which, int32_t index, uint64_t* value) {
    uint64_t* signal = host_signal(rt, segment_rank, which, index);
    if (!signal || !value) return set_error(PCIE_EP_E_INVALID, "no such host signal");
    *value = std::atomic_ref<uint64_t>(*signal).load(std::memory_order_acquire);
    return 0;
}

int pcie_ep_quantize_fp8(const void* x, uint8_t* codes, float* scales, int32_t tokens, int32_t hidden, void* stream) {
    if (tokens < 0 || hidden <= 0 || (tokens && (!x || !codes || !scales))) return set_error(PCIE_EP_E_INVALID, "bad quantize arguments");
    HIP_TRY(launch_quantize(static_cast<const uint16_t*>(x), codes, scales, tokens, hidden, static_cast<hipStream_t>(stream)));
    return 0;
}
int pcie_ep_dequantize_fp8(const uint8_t* codes, const float* scales, void* out, int32_t tokens, int32_t hidden, void* stream) {
    if (tokens < 0 || hidden <= 0 || (tokens && (!out || !codes || !scales))) return set_error(PCIE_EP_E_INVALID, "bad dequantize arguments");
    HIP_TRY(launch_dequantize(codes, scales, static_cast<uint16_t*>(out), tokens, hidden, static_cast<hipStream_t>(stream)));
    return 0;
}

int pcie_ep_measure_pinned_copy(int32_t device, int64_t bytes, int32_t repeats, double* h2d_gbps, double* d2h_gbps) {
    if (bytes <= 0 || repeats < 1 || !h2d_gbps || !d2h_gbps) return set_error(PCIE_EP_E_INVALID, "bad measurement arguments");
    HIP_TRY(hipSetDevice(device));
    void *host = nullptr, *dev = nullptr;
    HIP_TRY(hipHostMalloc(&host, size_t(bytes), hipHostMallocCoherent | hipHostMallocMapped | hipHostMallocPortable));
    std::memset(host, 1, size_t(bytes));
    hipStream_t stream = nullptr;
    hipEvent_t begin = nullptr, end = nullptr;
    hipError_t status = hipMalloc(&dev, size_t(bytes));
    if (status == hipSuccess) status = hipStreamCreate(&stream);
    if (status == hipSuccess) status = hipEventCreate(&begin);
    if (status == hipSuccess) status = hipEventCreate(&end);
    double best[2] = {0.0, 0.0};
    for (int direction = 0; direction < 2 && status == hipSuccess; ++direction) {
        for (int i = 0; i <= repeats && status == hipSuccess; ++i) {  // first iteration warms up
            status = hipEventRecord(begin, stream);
            if (status == hipSuccess)
                status = direction == 0 ? hipMemcpyAsync(dev, host, size_t(bytes), hipMemcpyHostToDevice, stream)
                                        : hipMemcpyAsync(host, dev, size_t(bytes), hipMemcpyDeviceToHost, stream);
            if (status == hipSuccess) status = hipEventRecord(end, stream);
            if (status == hipSuccess) status = hipEventSynchronize(end);
            float ms = 0.0f;
            if (status == hipSuccess) status = hipEventElapsedTime(&ms, begin, end);
            if (status == hipSuccess && i > 0 && ms > 0.0f) {
                const double rate = double(bytes) / (ms * 1e6);
                if (rate > best[direction]) best[direction] = rate;
            }
        }
    }
    if (begin) (void)hipEventDestroy(begin);
    if (end) (void)hipEventDestroy(end);
    if (stream) (void)hipStreamDestroy(stream);
    if (dev) (void)hipFree(dev);
    (void)hipHostFree(host);
    if (status != hipSuccess) return set_error(PCIE_EP_E_HIP, "pinned copy measurement failed: %s", hipGetErrorString(status));
    *h2d_gbps = best[0];
    *d2h_gbps = best[1];
    return 0;
}

int pcie_ep_measure_kernel_host_copy(int32_t device, int64_t bytes, int32_t repeats, int32_t wavefronts, double* read_gbps, double* write_gbps) {
    if (bytes < 16 || bytes % 16 || repeats < 1 || wavefronts < 1 || wavefronts > 65536 || !read_gbps || !write_gbps)
        return set_error(PCIE_EP_E_INVALID, "bad measurement arguments");
    HIP_TRY(hipSetDevice(device));
    void *host = nullptr, *dev = nullptr;
    HIP_TRY(hipHostMalloc(&host, size_t(bytes), hipHostMallocCoherent | hipHostMallocMapped | hipHostMallocPortable));
    std::memset(host, 1, size_t(bytes));
    hipStream_t stream = nullptr;
    hipEvent_t begin = nullptr, end = nullptr;
    hipError_t status = hipMalloc(&dev, size_t(bytes));
    if (status == hipSuccess) status = hipStreamCreate(&stream);
    if (status == hipSuccess) status = hipEventCreate(&begin);
    if (status == hipSuccess) status = hipEventCreate(&end);
    double best[2] = {0.0, 0.0};
    for (int direction = 0; direction < 2 && status == hipSuccess; ++direction) {
        for (int i = 0; i <= repeats && status == hipSuccess; ++i) {  // first iteration warms up
            status = hipEventRecord(begin, stream);
            if (status == hipSuccess) status = launch_host_copy(host, dev, bytes, direction == 0, wavefronts, stream);
            if (status == hipSuccess) status = hipEventRecord(end, stream);
            if (status == hipSuccess) status = hipEventSynchronize(end);
            float ms = 0.0f;
            if (status == hipSuccess) status = hipEventElapsedTime(&ms, begin, end);
            if (status == hipSuccess && i > 0 && ms > 0.0f) {
                const double rate = double(bytes) / (ms * 1e6);
                if (rate > best[direction]) best[direction] = rate;
            }
        }
    }
    if (begin) (void)hipEventDestroy(begin);
    if (end) (void)hipEventDestroy(end);
    if (stream) (void)hipStreamDestroy(stream);
    if (dev) (void)hipFree(dev);
    (void)hipHostFree(host);
    if (status != hipSuccess) return set_error(PCIE_EP_E_HIP, "kernel host copy measurement failed: %s", hipGetErrorString(status));
    *read_gbps = best[0];
    *write_gbps = best[1];
    return 0;
}

int pcie_ep_measure_device_copy(int32_t device, int64_t bytes, int32_t repeats, double* gbps) {
    if (bytes < 16 || bytes % 16 || repeats < 1 || !gbps) return set_error(PCIE_EP_E_INVALID, "bad measurement arguments");
    HIP_TRY(hipSetDevice(device));
    void *source = nullptr, *destination = nullptr;
    hipStream_t stream = nullptr;
    hipEvent_t begin = nullptr, end = nullptr;
    hipError_t status = hipMalloc(&source, size_t(bytes));
    if (status == hipSuccess) status = hipMalloc(&destination, size_t(bytes));
    if (status == hipSuccess) status = hipMemset(source, 1, size_t(bytes));
    if (status == hipSuccess) status = hipStreamCreate(&stream);
    if (status == hipSuccess) status = hipEventCreate(&begin);
    if (status == hipSuccess) status = hipEventCreate(&end);
    // One untimed launch, then three batches of `repeats` back-to-back launches
    // between one pair of events each (no event or launch-gap overhead per launch).
    double best = 0.0;
    if (status == hipSuccess) status = launch_copy(source, destination, bytes, stream);
    for (int batch = 0; batch < 3 && status == hipSuccess; ++batch) {
        status = hipEventRecord(begin, stream);
        for (int i = 0; i < repeats && status == hipSuccess; ++i) status = launch_copy(source, destination, bytes, stream);
        if (status == hipSuccess) status = hipEventRecord(end, stream);
        if (status == hipSuccess) status = hipEventSynchronize(end);
        float ms = 0.0f;
        if (status == hipSuccess) status = hipEventElapsedTime(&ms, begin, end);
        if (status == hipSuccess && ms > 0.0f) {
            const double rate = 2.0 * double(bytes) * repeats / (ms * 1e6);  // bytes read + bytes written
            if (rate > best) best = rate;
        }
    }
    if (begin) (void)hipEventDestroy(begin);
    if (end) (void)hipEventDestroy(end);
    if (stream) (void)hipStreamDestroy(stream);
    if (source) (void)hipFree(source);
    if (destination) (void)hipFree(destination);
    if (status != hipSuccess) return set_error(PCIE_EP_E_HIP, "device copy measurement failed: %s", hipGetErrorString(status));
    *gbps = best;
    return 0;
}

int pcie_ep_measure_row_scatter(int32_t device, int32_t rows, int32_t row_bytes, int32_t extra_per_1024, int32_t pattern, int32_t streams,
                                int32_t repeats, double* gbps) {
    if (rows < 1 || row_bytes < 16 || row_bytes % 16 || extra_per_1024 < 0 || extra_per_1024 > 1024 || pattern < 0 || pattern > 4 || streams < 1 ||
        repeats < 1 || !gbps)
        return set_error(PCIE_EP_E_INVALID, "bad measurement arguments");
    HIP_TRY(hipSetDevice(device));
    const size_t bytes = size_t(rows) * size_t(row_bytes);
    void *source = nullptr, *destination = nullptr;
    hipStream_t stream = nullptr;
    hipEvent_t begin = nullptr, end = nullptr;
    hipError_t status = hipMalloc(&source, bytes);
    if (status == hipSuccess) status = hipMalloc(&destination, 2 * bytes);
    if (status == hipSuccess) status = hipMemset(source, 1, bytes);
    if (status == hipSuccess) status = hipStreamCreate(&stream);
    if (status == hipSuccess) status = hipEventCreate(&begin);
    if (status == hipSuccess) status = hipEventCreate(&end);
    // Rows written twice, counted exactly as the kernel selects them.
    int64_t twice = 0;
    for (int row = 0; row < rows; ++row) twice += (row & 1023) * extra_per_1024 / 1024 != ((row & 1023) + 1) * extra_per_1024 / 1024;
    // One untimed launch, then three batches of `repeats` back-to-back launches
    // between one pair of events each: the per-launch mean of a batch carries no
    // event or launch-gap overhead (a tenth of a 100 us kernel otherwise).
    double best = 0.0;
    if (status == hipSuccess) status = launch_row_scatter(source, destination, rows, row_bytes, extra_per_1024, pattern, streams, stream);
    for (int batch = 0; batch < 3 && status == hipSuccess; ++batch) {
        status = hipEventRecord(begin, stream);
        for (int i = 0; i < repeats && status == hipSuccess; ++i)
            status = launch_row_scatter(source, destination, rows, row_bytes, extra_per_1024, pattern, streams, stream);
        if (status == hipSuccess) status = hipEventRecord(end, stream);
        if (status == hipSuccess) status = hipEventSynchronize(end);
        float ms = 0.0f;
        if (status == hipSuccess) status = hipEventElapsedTime(&ms, begin, end);
        if (status == hipSuccess && ms > 0.0f) {
            // bytes read + bytes written; the read-only and write-only patterns move every row once
            const double moved = pattern >= 3 ? double(rows) : double(2 * int64_t(rows) + twice);
            const double rate = moved * double(row_bytes) * repeats / (ms * 1e6);
            if (rate > best) best = rate;
        }
    }
    if (begin) (void)hipEventDestroy(begin);
    if (end) (void)hipEventDestroy(end);
    if (stream) (void)hipStreamDestroy(stream);
    if (source) (void)hipFree(source);
    if (destination) (void)hipFree(destination);
    if (status != hipSuccess) return set_error(PCIE_EP_E_HIP, "row scatter measurement failed: %s", hipGetErrorString(status));
    *gbps = best;
    return 0;
}

int pcie_ep_litmus(int32_t device, int32_t mode, int64_t iterations, int32_t payload_bytes, int32_t writer_delay_ns, int32_t reader_delay_ns,
                   int32_t timeout_ms, pcie_ep_litmus_result* result) {
    std::string error;
    const int status = run_litmus(device, mode, iterations, payload_bytes, writer_delay_ns, reader_delay_ns, timeout_ms, result, error);
    return status ? set_error(status, "%s", error.c_str()) : 0;
}

// ---- peer emulator -----------------------------------------------------------------

#define NEED_PEERS(rt)                                                                                        \
    if (!(rt) || (rt)->closed) return set_error(PCIE_EP_E_STATE, "advanced runtime is closed or closing");    \
    if (!(rt)->peers) return set_error(PCIE_EP_E_STATE, "this runtime was created without a host peer emulator")

int pcie_ep_peer_set_source(pcie_ep_runtime* rt, int32_t rank, const void* x, const int64_t* topk_idx, const float* weights, int32_t tokens) {
    NEED_PEERS(rt);
    if (tokens > 0 && (!x || !topk_idx)) return set_error(PCIE_EP_E_INVALID, "peer inputs are NULL");
    std::string error;
    const int status = rt->peers->set_source(rank, static_cast<const uint16_t*>(x), topk_idx, weights, tokens, error);
    return status ? set_error(status, "%s", error.c_str()) : 0;
}
int pcie_ep_peers_start(pcie_ep_runtime* rt, int32_t epochs, uint32_t flags) {
    NEED_PEERS(rt);
    std::string error;
    const int status = rt->peers->start(epochs, flags, error);
    return status ? set_error(status, "%s", error.c_str()) : 0;
}
int pcie_ep_peers_wait_staged(pcie_ep_runtime* rt, int32_t timeout_ms) {
    NEED_PEERS(rt);
    std::string error;
    const int status = rt->peers->wait_staged(timeout_ms, error);
    return status ? set_error(status, "%s", error.c_str()) : 0;
}
int pcie_ep_peers_wait(pcie_ep_runtime* rt, int32_t timeout_ms) {
    NEED_PEERS(rt);
    std::string error;
    const int status = rt->peers->wait(timeout_ms, error);
    return status ? set_error(status, "%s", error.c_str()) : 0;
}
int pcie_ep_peers_cancel(pcie_ep_runtime* rt) {
    NEED_PEERS(rt);
    rt->peers->cancel();
    return 0;
}
int pcie_ep_peer_captured_count(pcie_ep_runtime* rt, int32_t rank, int64_t* count) {
    NEED_PEERS(rt);
    const int64_t value = rt->peers->captured_count(rank);
    if (value < 0 || !count) return set_error(PCIE_EP_E_INVALID, "no such peer rank");
    *count = value;
    return 0;
}
int pcie_ep_peer_captured_copy(pcie_ep_runtime* rt, int32_t rank, int32_t* tokens, int32_t* rank_ordinals, uint8_t* payload, float* scales,
                               int32_t* expert_idx, int32_t* expert_ordinals, float* weights, uint32_t* destination_masks) {
    NEED_PEERS(rt);
    if (rt->peers->captured_copy(rank, tokens, rank_ordinals, payload, scales, expert_idx, expert_ordinals, weights, destination_masks))
        return set_error(PCIE_EP_E_INVALID, "no such peer rank");
    return 0;
}
int pcie_ep_peers_inject_fault(pcie_ep_runtime* rt, int32_t rank, int32_t fault) {
    NEED_PEERS(rt);
    if (rt->peers->inject_fault(rank, fault)) return set_error(PCIE_EP_E_INVALID, "no such peer rank or fault");
    return 0;
}

// ---- host implementations shared with the emulator -----------------------------------

int pcie_ep_host_quantize_fp8(const void* x, uint8_t* codes, float* scales, int32_t tokens, int32_t hidden) {
    if (tokens < 0 || hidden < 0 || (tokens && hidden && (!x || !codes)) || (tokens && !scales)) return set_error(PCIE_EP_E_INVALID, "bad quantize arguments");
    host_quantize_fp8(static_cast<const uint16_t*>(x), codes, scales, tokens, hidden);
    return 0;
}
int pcie_ep_host_dequantize_fp8(const uint8_t* codes, const float* scales, void* out, int32_t tokens, int32_t hidden) {
    if (tokens < 0 || hidden < 0 || (tokens && hidden && (!out || !codes)) || (tokens && !scales)) return set_error(PCIE_EP_E_INVALID, "bad dequantize arguments");
    host_dequantize_fp8(codes, scales, static_cast<uint16_t*>(out), tokens, hidden);
    return 0;
}
int pcie_ep_host_source_layout(const int64_t* topk_idx, int32_t tokens, int32_t topk, int32_t num_ranks, int32_t num_experts, uint32_t* mask,
                               int32_t* rank_ordinals, int32_t* expert_indices, int32_t* expert_ordinals, int32_t* counts) {
    if (tokens < 0 || topk < 1 || topk > kMaxTopk || num_ranks < 1 || num_ranks > kMaxRanks || num_experts < num_ranks ||
        num_experts % num_ranks || !counts || (tokens && (!topk_idx || !mask || !rank_ordinals || !expert_indices || !expert_ordinals)))
        return set_error(PCIE_EP_E_INVALID, "bad layout arguments");
    return host_source_layout(topk_idx, tokens, topk, num_ranks, num_experts, mask, rank_ordinals, expert_indices, expert_ordinals, counts);
}

}  // extern "C"

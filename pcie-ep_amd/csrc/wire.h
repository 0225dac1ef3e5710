// Host-ring wire format shared by the gfx950 kernels and the host-side peer
// emulator.  Plain C++ (no HIP types) so both sides compile it unchanged.
//
// One *segment* of pinned, fine-grained host memory exists per source rank.
// Only the source writes payload slots, slot metadata, descriptor bodies,
// READY words, the count mailbox, counts_ready, abort and channel_abort; a
// receiver d writes only its ack[channel][d][..] array, the credit word of its own (s -> d)
// descriptor queue and counts_consumed[d].  Every 64-bit signal therefore has
// exactly one writer and nothing ever performs a read-modify-write on host
// memory (the discipline of the reference: csrc/kernels/host_staged/common.cuh:59-64).
//
// The byte layout is private to this build; it keeps the reference's protocol
// objects (Signal / Descriptor / per-slot token metadata / count mailbox:
// common.cuh:61-88, advanced_common.cuh:42-84) but
//  * sizes the per-slot metadata by the runtime top-k instead of 32 branches,
//  * stores it in the tail of the payload slot so one contiguous region is read,
//  * groups the count mailbox by destination so a receiver reads one block.
//
// Relay mode (csrc/comm/numa_relay.hpp; advanced_common.cuh:207-260).  Ranks
// are grouped into NUMA domains.  A source reaches a destination of its own
// domain directly; destinations of another domain n are reached through
// endpoint P + n: the source publishes ONE descriptor per token to that
// endpoint, a CPU relay worker of the source copies the slot into the replica
// ring of domain n (memory bound to that domain's node), publishes replica
// descriptors to every targeted rank of the domain, and ACKs the source slot.
// Receivers of domain n read replica slots and answer with replica ACKs and
// replica credits.  Replica slots, replica descriptors, relay_drained and
// relay_failed are written only by the source's relay; replica ACKs and replica
// credits only by the receiver they belong to.  In direct mode there are no
// domains and none of these regions exist.
#pragma once

#include <cstddef>
#include <cstdint>

#if defined(__HIPCC__)
#define PCIE_EP_HD __host__ __device__ inline
#else
#define PCIE_EP_HD inline
#endif

namespace pcie_ep {

constexpr int kMaxRanks = 16;      // common.cuh:12
constexpr int kMaxTopk = 32;       // common.cuh:13
constexpr int kMaxExperts = 4096;  // common.cuh:14
constexpr int kMaxChannels = 32;   // pcie_ep/config.py:71
constexpr int kMaxDomains = 8;     // NUMA domains of a relay configuration (advanced_common.cuh:8)
constexpr int kMaxEndpoints = kMaxRanks + kMaxDomains;
constexpr int kErrorFields = 8;
constexpr int kStatFields = 8;
constexpr size_t kSignalBytes = 128;  // one writer per 128-byte line
constexpr size_t kPageBytes = 4096;

// Device error codes: values are part of the Python result contract
// (csrc/kernels/host_staged/common.cuh:26-38).
enum ErrorCode : int {
    kOk = 0,
    kErrInvalidRouting = 2,
    kErrCountsMailboxWait = 11,
    kErrCountsReadyWait = 12,
    kErrBatchReadyWait = 13,
    kErrBatchAckWait = 14,
    kErrRingProgressWait = 15,
    kErrExpandedCapacity = 16,
    kErrPayloadSequence = 18,
    kErrAlreadyAborted = 19,
    kErrEpochExhausted = 20,
};

// stats[] fields (API.md:148 of the reference).
enum StatField : int {
    kStatHostWrites = 0,     // own tokens published to the host ring
    kStatHostReads = 1,      // remote unique rows read from host rings
    kStatDeliveries = 2,     // sum over published tokens of remote destination ranks
    // 3..6 are event counts (not stall times) that depend on timing and are not compared.
    kStatPreparedAhead = 3,  // TX tickets prepared while an earlier payload of the channel was still in flight
    kStatRxNotReady = 4,     // descriptor polling passes of RX control that found no new descriptor
    kStatTxCreditMiss = 5,   // TX waits for a payload slot ACK or descriptor credit
    kStatRingFull = 6,       // control waits for a free entry of a ticket ring (the hand-off stage being busy)
    kStatDescriptors = 7,    // endpoint descriptors published
};

struct alignas(128) Signal {
    uint64_t value;
    char pad[120];
};

// One entry of a (source -> destination, channel) notification queue: 16 bytes,
// written only by the source — with ONE 16-byte store (the GPU) or as fields
// followed by a release store of `ready` (a CPU) — and read by the destination
// with ONE 16-byte load (the GPU) or an acquire load of `ready` followed by the
// fields (a CPU).  A naturally aligned 16-byte access inside one cache line is a
// single PCIe transaction and a single coherent snapshot, so `payload_slot` and
// `token_index` are valid whenever `ready` matches.  Entries are packed eight to
// a 128-byte line, which is what one look-ahead poll of the GPU fetches.
// The payload sequence of the reference's descriptor is sequence(epoch,
// token_index) by construction and is not stored; the destination's unique-row
// ordinal travels in the slot metadata.
//
// Credits flow the other way through ONE word per queue, written only by the
// destination: sequence(epoch, last consumed ordinal).  Entries of a queue are
// consumed in order, so the word says how many entries of this epoch are free
// again (the reference keeps a consumed_sequence in every descriptor, which
// puts two writers on one line).
struct alignas(16) Descriptor {
    uint64_t ready;  // sequence(epoch, ordinal) once the entry is complete
    int32_t payload_slot;
    int32_t token_index;
};
static_assert(sizeof(Signal) == 128 && sizeof(Descriptor) == 16, "wire ABI");

// Per-slot token metadata, stored after the payload bytes of the slot.
//   header (32 B) | rank_ordinals[kMaxRanks] (64 B) | expert_indices[K] |
//   expert_ordinals[K] | weights[K]
struct SlotMetaHeader {
    int32_t token_index;
    uint32_t destination_mask;
    float scale;  // FP8 per-token scale, 1.0 on a BF16 wire
    int32_t reserved[5];
};
static_assert(sizeof(SlotMetaHeader) == 32, "wire ABI");
constexpr int kMetaRankOrdinalsOffset = 32;
constexpr int kMetaBranchOffset = 32 + 4 * kMaxRanks;  // 96

PCIE_EP_HD size_t align_up(size_t value, size_t alignment) { return (value + alignment - 1) / alignment * alignment; }

// `(epoch << 32) | (index + 1)`; zero means never written
// (csrc/kernels/host_staged/advanced_common.cuh:203-205).
PCIE_EP_HD uint64_t sequence(uint64_t epoch, int index) { return (epoch << 32) | uint64_t(uint32_t(index + 1)); }

struct Dimensions {
    int num_ranks;
    int max_tokens;
    int hidden;
    int topk;
    int num_experts;
    int channels;
    int payload_slots;     // Q, per channel
    int descriptor_slots;  // L, per (channel, destination)
    int wire_fp8;          // 0: BF16 payload, 1: E4M3FN payload + FP32 scale
    int domains;           // N NUMA domains in relay mode, 0 in direct mode
    int replica_slots;     // R per (channel, domain)
    int rank_domain[kMaxRanks];  // domain of every rank (relay mode)
};

struct SegmentLayout {
    Dimensions dims;
    int local_experts;
    int payload_bytes;   // bytes of one row on the wire
    int meta_offset;     // offset of the metadata inside a slot
    int meta_bytes;      // 96 + 12*K rounded to 16
    int mailbox_dwords;  // dwords of one per-destination mailbox block
    size_t slot_stride;
    size_t mailbox_stride;
    size_t counts_ready_offset;
    size_t counts_consumed_offset;  // [P] signals
    size_t abort_offset;
    size_t channel_abort_offset;    // [C] signals
    size_t mailbox_offset;          // [P] blocks
    size_t slots_offset;            // [C*Q] slots, page aligned
    size_t ack_offset;              // [C][P+N] arrays of Q words, one array (one writer) per 128-byte aligned block
    size_t ack_stride;              // bytes of one such array
    size_t descriptors_offset;      // [C][P] queues of L packed entries, each queue 128-byte aligned
    size_t descriptor_queue_stride;
    size_t credits_offset;          // [C][P+N] signals: sequence(epoch, last ordinal the destination consumed)
    // Relay mode only.
    int endpoints;                  // P + N
    size_t relay_mailbox_offset;    // [N] blocks of C dwords: tokens of each channel bound for the domain through the relay
    size_t relay_mailbox_stride;
    size_t replica_ack_offset;      // [C][N][P] arrays of R words
    size_t replica_ack_stride;
    size_t replica_descriptors_offset;  // [C][N][P] queues of L packed entries
    size_t replica_credits_offset;  // [C][N][P] signals
    size_t relay_drained_offset;    // [C][N] signals: epoch whose flow has been copied and released
    size_t relay_failed_offset;     // [C][N] signals: non-zero relay failure code
    size_t size_bytes;
    // Replica payload slots live in one separate region per domain, [C][R] slots
    // of slot_stride bytes, so that each can be bound to its domain's memory.
    size_t replica_region_bytes;
};

// Mailbox block written by source s for destination d:
//   dword 0: unique tokens s -> d;  dwords 1..EL: branches per local expert of d;
//   dwords 1+EL .. 1+EL+C-1: unique tokens of each channel destined to d.
PCIE_EP_HD SegmentLayout make_segment_layout(const Dimensions& dims) {
    SegmentLayout z{};
    z.dims = dims;
    z.local_experts = dims.num_experts / dims.num_ranks;
    z.payload_bytes = dims.hidden * (dims.wire_fp8 ? 1 : 2);
    z.meta_offset = int(align_up(size_t(z.payload_bytes), 16));
    z.meta_bytes = int(align_up(size_t(kMetaBranchOffset + 12 * dims.topk), 16));
    z.slot_stride = align_up(size_t(z.meta_offset + z.meta_bytes), kPageBytes);
    z.mailbox_dwords = 1 + z.local_experts + dims.channels;
    z.mailbox_stride = align_up(size_t(z.mailbox_dwords) * 4, kSignalBytes);
    size_t cursor = 0;
    auto reserve = [&](size_t bytes) {
        const size_t offset = cursor;
        cursor += align_up(bytes, kSignalBytes);
        return offset;
    };
    z.counts_ready_offset = reserve(sizeof(Signal));
    z.counts_consumed_offset = reserve(size_t(dims.num_ranks) * sizeof(Signal));
    z.abort_offset = reserve(sizeof(Signal));
    z.channel_abort_offset = reserve(size_t(dims.channels) * sizeof(Signal));
    z.mailbox_offset = reserve(size_t(dims.num_ranks) * z.mailbox_stride);
    z.endpoints = dims.num_ranks + dims.domains;
    z.relay_mailbox_stride = align_up(size_t(dims.channels) * 4, kSignalBytes);
    z.relay_mailbox_offset = reserve(size_t(dims.domains) * z.relay_mailbox_stride);
    cursor = align_up(cursor, kPageBytes);
    const size_t slots = size_t(dims.channels) * dims.payload_slots;
    z.slots_offset = reserve(slots * z.slot_stride);
    // Payload ACKs: receiver d owns the array [channel][d] and stores sequence(epoch, token) into word
    // `slot` once it has read that slot.  Grouped by writer, a line still has one writer, and the source's
    // drain reads eight consecutive slots of one receiver with a single 64-byte read.
    z.ack_stride = align_up(size_t(dims.payload_slots) * 8, kSignalBytes);
    z.ack_offset = reserve(size_t(dims.channels) * z.endpoints * z.ack_stride);
    z.descriptor_queue_stride = align_up(size_t(dims.descriptor_slots) * sizeof(Descriptor), kSignalBytes);
    z.descriptors_offset = reserve(size_t(dims.channels) * z.endpoints * z.descriptor_queue_stride);
    z.credits_offset = reserve(size_t(dims.channels) * z.endpoints * sizeof(Signal));
    const size_t flows = size_t(dims.channels) * dims.domains;
    z.replica_ack_stride = align_up(size_t(dims.replica_slots) * 8, kSignalBytes);
    z.replica_ack_offset = reserve(flows * dims.num_ranks * z.replica_ack_stride);
    z.replica_descriptors_offset = reserve(flows * dims.num_ranks * z.descriptor_queue_stride);
    z.replica_credits_offset = reserve(flows * dims.num_ranks * sizeof(Signal));
    z.relay_drained_offset = reserve(flows * sizeof(Signal));
    z.relay_failed_offset = reserve(flows * sizeof(Signal));
    z.size_bytes = align_up(cursor, kPageBytes);
    z.replica_region_bytes = align_up(size_t(dims.channels) * dims.replica_slots * z.slot_stride, kPageBytes);
    return z;
}

// Endpoint through which `source` reaches `destination`: the destination itself
// inside one domain (or in direct mode), the relay endpoint P + domain otherwise
// (advanced_common.cuh:207-212).
PCIE_EP_HD int endpoint_of(const Dimensions& d, int source, int destination) {
    if (!d.domains || d.rank_domain[source] == d.rank_domain[destination]) return destination;
    return d.num_ranks + d.rank_domain[destination];
}
// Endpoints a token with destination ranks `rank_mask` is published to by `source`.
PCIE_EP_HD uint32_t endpoint_mask_of(const Dimensions& d, int source, uint32_t rank_mask) {
    rank_mask &= ~(1u << source);
    if (!d.domains) return rank_mask;
    uint32_t endpoints = 0;
    for (int rank = 0; rank < d.num_ranks; ++rank)
        if ((rank_mask >> rank) & 1u) endpoints |= 1u << endpoint_of(d, source, rank);
    return endpoints;
}
// Whether `receiver` reads the rows of `source` from a replica ring (advanced_common.cuh:233-235).
PCIE_EP_HD bool reads_replica(const Dimensions& d, int source, int receiver) {
    return d.domains && d.rank_domain[source] != d.rank_domain[receiver];
}

PCIE_EP_HD uint64_t* signal_at(char* segment, size_t offset, size_t index = 0) {
    return &reinterpret_cast<Signal*>(segment + offset)[index].value;
}
PCIE_EP_HD char* slot_at(const SegmentLayout& z, char* segment, int channel, int slot) {
    return segment + z.slots_offset + (size_t(channel) * z.dims.payload_slots + slot) * z.slot_stride;
}
// `endpoint` is a destination rank or, in relay mode, P + domain.
PCIE_EP_HD uint64_t* ack_at(const SegmentLayout& z, char* segment, int channel, int slot, int endpoint) {
    return reinterpret_cast<uint64_t*>(segment + z.ack_offset + (size_t(channel) * z.endpoints + endpoint) * z.ack_stride) + slot;
}
PCIE_EP_HD Descriptor* descriptor_at(const SegmentLayout& z, char* segment, int channel, int endpoint, int ordinal) {
    char* queue = segment + z.descriptors_offset + (size_t(channel) * z.endpoints + endpoint) * z.descriptor_queue_stride;
    return reinterpret_cast<Descriptor*>(queue) + ordinal % z.dims.descriptor_slots;
}
PCIE_EP_HD uint64_t* credit_at(const SegmentLayout& z, char* segment, int channel, int endpoint) {
    return signal_at(segment, z.credits_offset, size_t(channel) * z.endpoints + endpoint);
}
// Relay mode: replica ring of (channel, domain) inside the segment of the source
// whose relay fills it; `region` is that source's replica payload region of the domain.
PCIE_EP_HD size_t flow_index(const SegmentLayout& z, int channel, int domain) { return size_t(channel) * z.dims.domains + domain; }
PCIE_EP_HD char* replica_slot_at(const SegmentLayout& z, char* region, int channel, int slot) {
    return region + (size_t(channel) * z.dims.replica_slots + slot) * z.slot_stride;
}
PCIE_EP_HD uint64_t* replica_ack_at(const SegmentLayout& z, char* segment, int channel, int domain, int slot, int destination) {
    return reinterpret_cast<uint64_t*>(segment + z.replica_ack_offset + (flow_index(z, channel, domain) * z.dims.num_ranks + destination) * z.replica_ack_stride) + slot;
}
PCIE_EP_HD Descriptor* replica_descriptor_at(const SegmentLayout& z, char* segment, int channel, int domain, int destination, int ordinal) {
    char* queue = segment + z.replica_descriptors_offset + (flow_index(z, channel, domain) * z.dims.num_ranks + destination) * z.descriptor_queue_stride;
    return reinterpret_cast<Descriptor*>(queue) + ordinal % z.dims.descriptor_slots;
}
PCIE_EP_HD uint64_t* replica_credit_at(const SegmentLayout& z, char* segment, int channel, int domain, int destination) {
    return signal_at(segment, z.replica_credits_offset, flow_index(z, channel, domain) * z.dims.num_ranks + destination);
}
PCIE_EP_HD int32_t* relay_mailbox_at(const SegmentLayout& z, char* segment, int domain) {
    return reinterpret_cast<int32_t*>(segment + z.relay_mailbox_offset + size_t(domain) * z.relay_mailbox_stride);
}
// The source may write entry `ordinal` of a queue of L entries once entry
// `ordinal - L` has been consumed, i.e. once the credit word of this epoch
// names an ordinal >= ordinal - L.
PCIE_EP_HD bool credit_covers(uint64_t credit, uint64_t epoch, int ordinal, int descriptor_slots) {
    if (ordinal < descriptor_slots) return true;
    return (credit >> 32) == epoch && int64_t(credit & 0xFFFFFFFFull) - 1 >= int64_t(ordinal) - descriptor_slots;
}
PCIE_EP_HD int32_t* mailbox_at(const SegmentLayout& z, char* segment, int destination) {
    return reinterpret_cast<int32_t*>(segment + z.mailbox_offset + size_t(destination) * z.mailbox_stride);
}

// Preallocated output capacities (csrc/buffers/advanced.hpp:296-298).
PCIE_EP_HD int64_t unique_capacity(const Dimensions& d) { return int64_t(d.num_ranks) * d.max_tokens; }
PCIE_EP_HD int64_t expanded_capacity(const Dimensions& d) {
    const int local = d.num_experts / d.num_ranks;
    return unique_capacity(d) * (d.topk < local ? d.topk : local) + int64_t(local) * 255;
}

}  // namespace pcie_ep

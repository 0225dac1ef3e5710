// Channel transport kernel: TX control (+ guardian), RX control (+ receive
// prefixes), TX payload workers and RX/scatter workers, all as single
// wavefronts with their own role.
//
// Replaces advanced_transport_pipelined and its roles
// (csrc/kernels/host_staged/fused_receive.cuh:333-360;
// advanced_dispatch.cuh:287-477 tx_control, :479-625 rx_control, :627-689
// tx_worker; fused_receive.cuh:199-305 producer/consumer) and, for the unique
// layout, advanced_transport (advanced_dispatch.cuh:919-958).
//
// Design for MI355X (64-lane wavefronts, 8 XCDs):
//  * A payload worker is ONE wavefront that owns a whole row: 14 x 16-byte
//    loads per lane are issued back to back (896 vectors of a 14 336-byte BF16
//    row), the row lives in registers, and the same wavefront stores it to
//    every destination expert row.  The staged row is read once; there is no
//    LDS tile and no producer/consumer hand-off (the reference stages through
//    shared memory with 3+3 warps per ticket).
//  * Control wavefronts work on 64 candidates at a time with ballots: TX control
//    derives ring slots and per-destination descriptor ordinals for 64 tokens
//    from popcounts of ballots; RX control probes up to 64/P descriptors per
//    source per iteration instead of one source per iteration.
//  * Work is handed out through two global ticket rings in device memory (one
//    for TX, one for RX).  Control wavefronts only reserve and hand out tickets;
//    the payload workgroups hold payload wavefronts, which claim tickets of ANY
//    channel, so every channel's rows are moved by all payload XCDs.  This matters
//    because the XCDs get unequal shares of the host link: with workers bound to
//    their channel's workgroup, equal work finished in 8.8 ms on the best XCD and
//    12.8 ms on the worst.  It also decouples the bytes in flight (worker
//    wavefronts x row size), which set the latency of every control-path read,
//    from the number of channels.
//  * Which workgroup runs on which XCD is chosen (workgroup id = row * 8 + XCD):
//    two XCDs hold the control class - the epoch begin and the layout chunks of the
//    prologue when it rides in this launch, and per pair of channels one workgroup
//    of transmit controls and one of receive controls, on different XCDs - and six
//    hold the payload class (payload and local-bypass workgroups).  A host read
//    stays in its XCD's memory queues for as long as the link needs for the bytes
//    requested before it, and every other memory operation through that XCD waits
//    behind it: controls that shared an XCD with payload wavefronts saw their
//    tickets and flags arrive tens of microseconds late.
//  * With the prologue in the same launch (one launch per dispatch), the roles
//    here start with the queues not yet reset: one thread per workgroup waits for
//    the epoch begin's word before its role touches them, the transmit side and
//    the local bypass wait for the plan's word, the receive side for neither.
//  * Workers publish their own descriptors and payload ACKs as soon as their own
//    stores / loads have completed; control wavefronts only reserve and hand out.
//  * A payload wavefront has no fixed direction: before every row it takes the
//    direction that needs it, in proportion to the rows left to send and to
//    receive, so that the writes are spread thinly over the whole dispatch (row
//    writes compete with the read REQUESTS for the upstream half of the link) and
//    both directions end together whatever the routing's send/receive ratio is.
//  * Vector memory operations complete in order: wherever several host words are
//    wanted at once (count mailboxes, ACK arrays), their addresses are computed
//    first and the loads issued in one run, with no other load in between.
//  * Every read from host memory is a whole 16-byte vector per lane (payload, slot
//    metadata, descriptor entries) or a packed word array (ACKs): small scattered
//    reads cost the host link far more than their bytes.
//  * The workgroups after the payload workgroups do the local bypass (own tokens
//    routed to own experts: advanced_copy_local_tokens, advanced_layout.cuh:217-248)
//    and the zeroing of the alignment gaps (:250-265) as soon as the receive
//    prefixes are known, token by token from a shared counter.  That work only
//    touches HBM and runs on compute units the transport leaves idle, so it hides
//    completely behind the host link.  The last role wavefront to end reduces the
//    per-channel statistics (:267-283).  The dispatch needs no kernel after this one.
#include "device_common.h"
#include "launch.h"
#include "prologue_body.h"
#include "row_codec.h"

namespace pcie_ep {

namespace {

constexpr int kScratchDwords = 128;  // per wavefront: one slot metadata record or one ticket
constexpr int kMaxWaves = 12;

struct WaveScratch {
    uint32_t words[kMaxWaves][kScratchDwords];
};

// Local time only: payload workers never scan the host abort flags themselves
// (hundreds of wavefronts doing so would be PCIe traffic of their own); the
// channel's guardian does and raises the channel's abort word.
struct Deadline {
    uint64_t start;
    __device__ explicit Deadline(uint64_t begin) : start(begin) {}
    __device__ __forceinline__ bool expired(const DeviceState& state) const { return now_ticks() - start > progress_timeout_ticks(state); }
};

__device__ __forceinline__ bool aborted(TransportQueues& q) { return device_load(&q.abort.value) != 0; }
__device__ __forceinline__ void raise_abort(TransportQueues& q) { device_store(&q.abort.value, 1u); }

// Prologue inside this launch: a role may touch the queues and the diagnostics once
// the epoch begin has cleared them.  One thread per workgroup polls (hundreds of
// wavefronts polling one word would slow down the very stores they wait for).
// Bounded: an epoch begin that never runs ends the role.
__device__ __forceinline__ bool wait_for_begin(const DeviceState& state, TransportQueues& q) {
    const uint32_t tag = epoch_flag(dispatch_epoch(state));
    const uint64_t start = now_ticks();
    // The word cannot be there in the first microsecond: stay off the memory the clearing goes to.
    __builtin_amdgcn_s_sleep(48);
    while (device_load(&q.begun.value) != tag) {
        if (now_ticks() - start > state.timeout_ticks) return false;
        __builtin_amdgcn_s_sleep(16);
    }
    return true;
}
// ... and read the route plan once the leader has published the counts and every
// chunk's part of the plan is in memory.  False when the prologue failed (abort) or
// never finished (timeout, recorded as a ring-progress error).
__device__ __forceinline__ bool wait_for_plan(const DeviceState& state, TransportQueues& q, int lane) {
    if (!state.fused) return true;
    const uint32_t tag = epoch_flag(dispatch_epoch(state));
    const uint64_t start = now_ticks();
    while (true) {
        int verdict = 0;
        if (lane == 0) {
            if (device_load(&q.plan_ready.value) == tag) verdict = 1;
            else if (aborted(q)) verdict = -1;
            else if (now_ticks() - start > progress_timeout_ticks(state)) {
                record_error(state, kErrRingProgressWait);
                raise_abort(q);
                verdict = -1;
            }
        }
        verdict = broadcast_first(verdict);
        if (verdict) return verdict > 0;
        backoff();
    }
}

// Producer side: reserve `count` consecutive tickets (one fetch-add per wavefront).
__device__ __forceinline__ int reserve_tickets(QueueCounter& tail, int count, int lane) {
    uint32_t base = 0;
    if (lane == 0) base = device_add(&tail.value, uint32_t(count));
    return broadcast_first(int(base));
}
__device__ __forceinline__ bool ring_entry_free(const uint64_t* taken, uint64_t epoch, int ticket) {
    const int previous = ticket - kRing;
    return previous < 0 || device_load(taken + previous % kRing) == sequence(epoch, previous);
}

// Consumer side: claim the next ticket, then wait until its entry is complete.
// Returns 1 when available, -1 when there is no such ticket or on abort.
__device__ __forceinline__ int claim_ticket(QueueCounter& head, int lane) {
    uint32_t ticket = 0;
    if (lane == 0) ticket = device_add(&head.value, 1u);
    return broadcast_first(int(ticket));
}
__device__ __forceinline__ int wait_ticket(const DeviceState& state, TransportQueues& q, const uint64_t* ready, QueueCounter& head, int ticket,
                                  uint64_t epoch, int lane, const Deadline& deadline) {
    while (true) {
        int action = 0;
        if (lane == 0) {
            if (aborted(q)) action = -1;
            else if (device_load(ready + ticket % kRing) == sequence(epoch, ticket)) action = 1;
            else {
                const int limit = device_load(&head.total);
                if (limit >= 0 && ticket >= limit) action = -1;
                else if (deadline.expired(state)) {
                    record_error(state, kErrRingProgressWait);
                    raise_abort(q);
                    action = -1;
                }
            }
        }
        action = broadcast_first(action);
        if (action) return action;
        backoff();
    }
}

// ---------------------------------------------------------------------------------------
// Receive prefixes (advanced_layout.cuh:94-195).  One wavefront of the grid is
// elected by a device-scope CAS; it waits for every source's counts_ready,
// folds the mailboxes in rank order and publishes a generation-valued READY.
// ---------------------------------------------------------------------------------------
// The producer's first look at every source's counts_ready (lane r: rank r), issued by the
// kernel's entry code before the role is let in; see RxFirstPoll.
struct PrefixFirstLook {
    uint64_t word;
    bool issued;
};
__device__ __forceinline__ PrefixFirstLook prefix_first_look(const DeviceState& state, int lane) {
    const SegmentLayout& z = state.z;
    const int ranks = z.dims.num_ranks;
    PrefixFirstLook look{0, true};
    if (lane < ranks && !(state.fused != 0 && lane == state.local_rank))
        look.word = host_load_global(signal_at(state.seg[lane], z.counts_ready_offset));
    return look;
}

__device__ __forceinline__ bool compute_receive_prefixes(const DeviceState& state, int lane, PrefixFirstLook entry_look PCIE_EP_PROFILE(, RoleProfile& profile)) {
    const SegmentLayout& z = state.z;
    const int ranks = z.dims.num_ranks, local = z.local_experts, channels = z.dims.channels;
    const int me = state.local_rank;
    const uint64_t epoch = dispatch_epoch(state);
    const uint64_t start = now_ticks();
    HealthCheck health(state, start);
    PCIE_EP_PROFILE(profile.first(kProfilePrefixEnterNs);)
    if (lane == 0) {
        state.prefix_tx_timestamps_ns[0] = ticks_to_ns(state, start);
        test_delay(state.prefix_delay);
    }
    // This runs while the payload wavefronts already stream rows, so it keeps to
    // the discipline of the hot path: host words are read with the system-scope
    // policy (never from a GPU cache, so no invalidate is needed), results are
    // written through to device memory (so no cache write-back is needed), and
    // ordering is by waiting for this wavefront's own operations.  A cache
    // write-back here would have to flush the rows the scatter is writing.
    // Once every source's counts are ready, every mailbox word this wavefront needs
    // is requested before the first one is used: one round trip over the host link
    // instead of one per group.  Vector memory operations complete in order, so
    // nothing else may be loaded in between - not even a segment's base address out of the kernel arguments:
    // waiting for that load would wait for every host word requested before it.
    // The addresses are therefore computed first (lane r holds the base of rank
    // r's segment and hands it out by lane shuffle) - before the wait for the
    // sources, where it costs nothing - and the loads follow in one run.
    const char* const lane_segment = state.seg[lane < ranks ? lane : 0];
    // Prologue in the same launch: the own counts are taken from the route plan in
    // device memory once the leader has announced it, not from the own mailbox in
    // host memory; the other sources' words are requested before that wait.
    const bool own_from_plan = state.fused != 0;
    // The first look at every source's counts_ready is requested now; its value is
    // used after the address arithmetic below, which so runs inside its round trip.
    uint64_t first_look = entry_look.word;
    if (!entry_look.issued && lane < ranks && !(own_from_plan && lane == me))
        first_look = host_load_global(signal_at(const_cast<char*>(lane_segment), z.counts_ready_offset));
    const auto segment_of = [&](int rank) {
        const uint64_t bits = reinterpret_cast<uint64_t>(lane_segment);
        return reinterpret_cast<char*>(uint64_t(uint32_t(__shfl(int(uint32_t(bits)), rank))) | uint64_t(uint32_t(__shfl(int(uint32_t(bits >> 32)), rank))) << 32);
    };
    constexpr int kExpectedPerLane = kMaxChannels * kMaxRanks / kWave;
    const int32_t* expected_address[kExpectedPerLane];
#pragma unroll
    for (int i = 0; i < kExpectedPerLane; ++i) {
        const int index = lane + i * kWave;
        const bool valid = index < channels * ranks;
        char* segment = segment_of(valid ? index % ranks : 0);
        expected_address[i] = valid ? mailbox_at(z, segment, me) + 1 + local + index / ranks : nullptr;
        if (own_from_plan && valid && index % ranks == me) expected_address[i] = state.plan_chan_counts + (index / ranks) * ranks + me;
    }
    const int32_t* first_address[kMaxRanks];
#pragma unroll
    for (int source = 0; source < kMaxRanks; ++source) {
        char* segment = segment_of(source < ranks ? source : 0);
        first_address[source] = (source < ranks && lane < local) ? mailbox_at(z, segment, me) + 1 + lane : nullptr;
        if (own_from_plan && source == me && lane < local) first_address[source] = state.plan_counts + ranks + me * local + lane;
    }
    const int32_t* unique_address = lane < ranks ? mailbox_at(z, const_cast<char*>(lane_segment), me) : nullptr;
    if (own_from_plan && lane == me) unique_address = state.plan_counts + me;
    // All sources are polled in parallel, one lane each.
    bool ready = lane >= ranks || (own_from_plan && lane == me) || first_look == epoch;
    while (true) {
        if (__all(ready)) break;
        if (!ready) ready = host_load_global(signal_at(const_cast<char*>(lane_segment), z.counts_ready_offset)) == epoch;
        if (__all(ready)) break;
        if (health.poll(state, lane)) {
            if (lane == 0) record_error(state, kErrCountsReadyWait);
            return false;
        }
        // Nothing will come of this dispatch when the prologue of the same launch has failed.
        if (state.fused && broadcast_first(aborted(*state.queues) ? 1 : 0)) return false;
        backoff();
    }
    wait_memory_ops();
    compiler_barrier();
    PCIE_EP_PROFILE(profile.first(kProfilePrefixCountsReadyNs);)
    // Host words first (every word of the other sources, in one run) ...
    int unique = 0;
    if (unique_address && !(own_from_plan && lane == me)) unique = host_field_load_global(unique_address);
    int expected_values[kExpectedPerLane];
#pragma unroll
    for (int i = 0; i < kExpectedPerLane; ++i)
        expected_values[i] = (expected_address[i] && !(own_from_plan && (lane + i * kWave) % ranks == me)) ? host_field_load_global(expected_address[i]) : 0;
    int first_counts[kMaxRanks];
#pragma unroll
    for (int source = 0; source < kMaxRanks; ++source)
        first_counts[source] = (first_address[source] && !(own_from_plan && source == me)) ? host_field_load_global(first_address[source]) : 0;
    // The reads are on the link (requests leave in issue order): the receive side
    // may now flood it with row reads without delaying these few words.
    compiler_barrier();
    if (lane == 0) device_store(state.receive_prefix_state, epoch | kPrefixRequested);
    compiler_barrier();
    if (own_from_plan) {
        // ... then the own words, out of device memory, once the plan is there.
        if (!wait_for_plan(state, *state.queues, lane)) return false;
        if (lane == me) unique = device_load_global(unique_address);
#pragma unroll
        for (int i = 0; i < kExpectedPerLane; ++i)
            if (expected_address[i] && (lane + i * kWave) % ranks == me) expected_values[i] = device_load_global(expected_address[i]);
#pragma unroll
        for (int source = 0; source < kMaxRanks; ++source)
            if (source == me && first_address[source]) first_counts[source] = device_load_global(first_address[source]);
    }
    // Per-source unique counts -> source_offsets (lane = source).
    int inclusive = unique;
    PCIE_EP_PROFILE(if (__builtin_amdgcn_readfirstlane(inclusive) >= 0) profile.first(kProfilePrefixMailboxNs);)  // the first use of a mailbox word: the reads have returned
    for (int offset = 1; offset < kMaxRanks; offset <<= 1) {
        const int other = __shfl_up(inclusive, offset);
        if (lane >= offset) inclusive += other;
    }
    if (lane < ranks) device_store(state.source_offsets + lane + 1, inclusive);
    if (lane == 0) device_store(state.source_offsets, 0);
    const int total_unique = __shfl(inclusive, ranks - 1);
    // Expert branches: lane = local expert; all sources' loads are issued first.
    int carry_offset = 0;
    int64_t expanded_total = 0;
    for (int begin = 0; begin < local; begin += kWave) {
        const int expert = begin + lane;
        int counts[kMaxRanks];
#pragma unroll
        for (int source = 0; source < kMaxRanks; ++source) {
            if (begin == 0) counts[source] = first_counts[source];
            else if (own_from_plan && source == me) counts[source] = expert < local ? device_load(state.plan_counts + ranks + me * local + expert) : 0;
            else counts[source] = (source < ranks && expert < local) ? host_field_load(mailbox_at(z, state.seg[source], me) + 1 + expert) : 0;
        }
        int running = 0;
#pragma unroll
        for (int source = 0; source < kMaxRanks; ++source) {
            if (source < ranks && expert < local) device_store(state.source_expert_prefix + source * local + expert, running);
            running += counts[source];
        }
        const int padded = (running + state.alignment - 1) / state.alignment * state.alignment;
        int scan = padded;
        for (int offset = 1; offset < kWave; offset <<= 1) {
            const int other = __shfl_up(scan, offset);
            if (lane >= offset) scan += other;
        }
        const int exclusive = carry_offset + scan - padded;
        if (expert < local) {
            device_store(state.expert_counts + expert, running);
            device_store(state.expert_offsets + expert, exclusive);
            device_store(state.expert_prefix + expert, exclusive + running);
            if (expert == local - 1) device_store(state.expert_offsets + local, exclusive + padded);
        }
        carry_offset += __shfl(scan, kWave - 1);
        int sum = running;
        for (int offset = 32; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset);
        expanded_total += sum;
    }
    // Expected tokens per (channel, source) for this receiver.
#pragma unroll
    for (int i = 0; i < kExpectedPerLane; ++i) {
        const int index = lane + i * kWave;
        if (index < channels * ranks) device_store(state.expected_receive_counts + index, expected_values[i]);
    }
    const int own_unique = __shfl(unique, me);
    if (lane == 0) {
        device_store(state.unique_count, int64_t(total_unique));
        device_store(state.expanded_count, expanded_total);
        // Receive tickets of this dispatch: every unique row of a remote source.
        device_store(&state.queues->rx_head.total, total_unique - own_unique);
    }
    return true;
}

// A source may overwrite its count mailbox for the next epoch once this rank has
// said so.  Every lane has its counts in registers by now (the loads above were
// waited for, wave-wide), so the ACK needs no fence (advanced_layout.cuh:91-93).
__device__ __forceinline__ void acknowledge_counts(const DeviceState& state, int lane) {
    const SegmentLayout& z = state.z;
    wait_memory_ops();
    if (lane < z.dims.num_ranks && lane != state.local_rank && lane != state.counts_ack_skip_source)
        host_field_store(signal_at(state.seg[lane], z.counts_consumed_offset, state.local_rank), dispatch_epoch(state));
}

__device__ __forceinline__ void produce_receive_prefixes(const DeviceState& state, int lane, PrefixFirstLook entry_look PCIE_EP_PROFILE(, RoleProfile& profile));

// One wavefront of the grid (the first RX control to get there) computes the
// receive prefixes; nobody waits here.
__device__ __forceinline__ void elect_receive_prefixes(const DeviceState& state, int lane PCIE_EP_PROFILE(, RoleProfile& profile)) {
    const uint64_t epoch = dispatch_epoch(state);
    int claimed = 0;
    if (lane == 0) {
        unsigned long long expected = 0;
        claimed = atomicCAS(reinterpret_cast<unsigned long long*>(state.receive_prefix_state), expected, epoch) == 0ull;
    }
    if (!broadcast_first(claimed)) return;
    produce_receive_prefixes(state, lane, PrefixFirstLook{0, false} PCIE_EP_PROFILE(, profile));
}

// With payload workgroups of their own, the control workgroups have wavefronts to
// spare (a third one exists with three or more payload wavefronts per workgroup):
// the receive prefixes are then produced by that one (wavefront 2 of
// channel 0's workgroup) and no RX control is held up by them - the channel of an
// elected RX control starts to receive a prefix computation late.
__device__ __forceinline__ bool dedicated_prefix_producer(const DeviceState& state) { return state.worker_groups > 0 && state.tx_waves + state.rx_waves >= 3; }

__device__ __forceinline__ void receive_prefix_role(const DeviceState& state, int lane, PrefixFirstLook entry_look) {
    PCIE_EP_PROFILE(RoleProfile profile(state.clock_khz);)
    if (lane == 0) device_store(state.receive_prefix_state, dispatch_epoch(state));
    produce_receive_prefixes(state, lane, entry_look PCIE_EP_PROFILE(, profile));
    PCIE_EP_PROFILE(profile.save(state.profiling, profile_rows(state.z.dims.channels, state.worker_groups * (state.tx_waves + state.rx_waves)) - 1, lane);)
}

__device__ __forceinline__ void produce_receive_prefixes(const DeviceState& state, int lane, PrefixFirstLook entry_look PCIE_EP_PROFILE(, RoleProfile& profile)) {
    const uint64_t epoch = dispatch_epoch(state);
    const bool success = compute_receive_prefixes(state, lane, entry_look PCIE_EP_PROFILE(, profile));
    // The results were written through; they are complete once this wavefront's
    // stores have been acknowledged.  Local consumers come first, the ACK to the
    // sources (which nobody on this GPU waits for) second.
    wait_memory_ops();
    if (lane == 0) {
        state.prefix_tx_timestamps_ns[1] = ticks_to_ns(state, now_ticks());
        device_store(state.receive_prefix_state + 1, success ? epoch : kPrefixFailed);
    }
    PCIE_EP_PROFILE(profile.first(kProfilePrefixPublishedNs);)
    if (success) acknowledge_counts(state, lane);
}

// 1 once the receive prefixes of this epoch are published, -1 when they never
// will be (their producer failed or the dispatch has an error), 0 otherwise.
// The elected producer owns the timeout; everybody else only reads device flags.
__device__ __forceinline__ int receive_prefix_verdict(const DeviceState& state, uint64_t epoch, int lane) {
    int verdict = 0;
    if (lane == 0) {
        // Relaxed: what the flag guards is read with device-scope loads.
        const uint64_t value = device_load(state.receive_prefix_state + 1);
        if (value == epoch) verdict = 1;
        else if (value == kPrefixFailed || load_error_code(state)) verdict = -1;
    }
    return broadcast_first(verdict);
}

// ---------------------------------------------------------------------------------------
// TX control + guardian
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ void tx_control(const DeviceState& state, TransportQueues& q, int channel, int lane) {
    const SegmentLayout& z = state.z;
    const int channels = z.dims.channels, me = state.local_rank;
    const int endpoints = z.endpoints;  // destination ranks, then (relay mode) one relay endpoint per domain
    const int slots = z.dims.payload_slots;
    const int stride = (z.dims.max_tokens + channels - 1) / channels;
    char* own = state.seg[me];
    const uint64_t epoch = dispatch_epoch(state);
    const uint64_t start = now_ticks();
    HealthCheck health(state, start, true, channel, channels);
    PCIE_EP_PROFILE(RoleProfile profile(state.clock_khz);)
    if (lane == 0) device_store(state.channel_timestamps_ns + channel * 2, ticks_to_ns(state, start));
    const int tokens = state.num_tokens;
    const int candidates = tokens > channel ? (tokens - channel + channels - 1) / channels : 0;
    const uint64_t below = lanes_below(lane);
    const __amdgpu_buffer_rsrc_t ring = device_resource(q.tx, sizeof(q.tx));
    int produced = 0;
    int reserved[kMaxEndpoints];
#pragma unroll
    for (int endpoint = 0; endpoint < kMaxEndpoints; ++endpoint) reserved[endpoint] = 0;
    bool failed = !wait_for_plan(state, q, lane);
    int64_t stage_busy = 0, prepared_ahead = 0;

    for (int base = 0; base < candidates && !failed; base += kWave) {
        const int candidate = base + lane;
        const int token = channel + candidate * channels;
        // Where the token is published: its destination ranks, with those of other
        // domains folded into one relay endpoint per domain (advanced_common.cuh:207-225).
        const uint32_t remote = candidate < candidates ? endpoint_mask_of(z.dims, me, state.plan_mask[token]) : 0u;
        const uint64_t batch = __ballot(remote != 0);
        if (!batch) continue;
        const int ordinal = produced + __popcll(batch & below);
        int my_descriptor[kMaxEndpoints];
#pragma unroll
        for (int endpoint = 0; endpoint < kMaxEndpoints; ++endpoint) {
            my_descriptor[endpoint] = 0;
            if (endpoint < endpoints) {
                const uint64_t hits = __ballot((remote >> endpoint) & 1u);
                my_descriptor[endpoint] = reserved[endpoint] + __popcll(hits & below);
                reserved[endpoint] += __popcll(hits);
            }
        }
        // Ring history: which token occupied ordinal i (needed when a slot is reused).
        if (remote) device_store(state.chan_remote_tokens + size_t(channel) * stride + ordinal, token);
        const int ticket_index = reserve_tickets(q.tx_tail, __popcll(batch), lane) + __popcll(batch & below);
        // Tickets prepared while an earlier payload of this channel is still in
        // flight: the control path runs ahead of the payload path (the event the
        // reference counts in stats[3]: advanced_dispatch.cuh:384-387).
        if (produced > 0 && broadcast_first(int(device_load(&q.tx_retired[channel].value))) < produced) prepared_ahead += __popcll(batch);
        bool pending = remote != 0;
        while (true) {
            if (pending && ring_entry_free(q.tx_taken, epoch, ticket_index)) {
                const uint32_t at = uint32_t(ticket_index % kRing) * uint32_t(sizeof(TxEntry));
                device_store_b32(ring, at + 0, uint32_t(token));
                device_store_b32(ring, at + 4, uint32_t(ordinal));
                device_store_b32(ring, at + 8, remote);
                device_store_b32(ring, at + 12, uint32_t(channel));
#pragma unroll
                for (int endpoint = 0; endpoint < kMaxEndpoints; ++endpoint)
                    if (endpoint < endpoints) device_store_b32(ring, at + 16 + 4 * endpoint, uint32_t(my_descriptor[endpoint]));
                // Ring history and the ticket body are complete before the tag.
                wait_memory_ops();
                device_store(q.tx_ready + ticket_index % kRing, sequence(epoch, ticket_index));
                pending = false;
            }
            if (!__any(pending)) break;
            ++stage_busy;
            const bool unhealthy = health.poll(state, lane);
            if (unhealthy || broadcast_first(aborted(q) ? 1 : 0)) {
                // A peer's abort flag or the timeout: raise the kernel-wide abort at
                // once, the workers are spinning on tickets that will never be marked ready.
                if (unhealthy && lane == 0) {
                    record_error(state, kErrRingProgressWait);
                    raise_abort(q);
                }
                failed = true;
                break;
            }
            backoff();
        }
        produced += __popcll(batch);
        PCIE_EP_PROFILE(profile.first(kProfileFirstTicketNs); profile.last(kProfileLastTicketNs);)
    }
    PCIE_EP_PROFILE(profile.values[kProfileItems] = uint64_t(produced);)

    // Wait for the workers, then drain the ACKs of the last ring window: earlier
    // slots were checked when they were reused (advanced_dispatch.cuh:229-285).
    // Lanes poll different (ordinal, destination) pairs in parallel.
    bool drained = failed;
    // Relay mode: every relay flow of the channel, also one without work, must
    // have consumed this epoch's counts and released its replica slots before a
    // later dispatch may overwrite the mailbox (advanced_dispatch.cuh:213-225).
    bool relays_drained = z.dims.domains == 0;
    int drain_ordinal = produced > slots ? produced - slots : 0;
    uint64_t next_drain_poll = 0;
    bool workers_finished = false;
    while (true) {
        if (broadcast_first(aborted(q) ? 1 : 0)) break;
        if (!workers_finished) {
            workers_finished = broadcast_first(int(device_load(&q.tx_retired[channel].value))) >= produced;
            PCIE_EP_PROFILE(if (workers_finished) profile.first(kProfileWorkersDoneNs);)
        }
        if (workers_finished && !drained) {
            // Each pass checks up to kDrainBatch * (64 / endpoints) ordinals of every
            // endpoint; lanes of one endpoint read consecutive ACK words (one 64-byte read
            // per eight slots) and all reads of a pass are on the link before the first
            // is used, so a ring window costs a few round trips, not one per handful of slots.
            // While the channel's receive side is still busy the drain is not what the
            // kernel waits for: it then polls sparingly, so that the small reads do not
            // compete with the row reads for the link.
            const bool receive_busy = broadcast_first(int(device_load(&q.rx_finished[channel].value))) == 0;
            if (!receive_busy || broadcast_first(now_ticks() >= next_drain_poll ? 1 : 0)) {
                PCIE_EP_PROFILE(const uint64_t poll_begin = profile.now(); profile.add(kProfilePolls);)
                constexpr int kDrainBatch = 8;
                const int group = kWave / endpoints;
                const int per_pass = group * kDrainBatch;
                const int endpoint = lane / group;
                // Vector memory operations complete in order: what the ACK addresses depend
                // on (tokens, route masks) is loaded first, the host reads follow in one run.
                uint64_t seen[kDrainBatch], wanted[kDrainBatch];
                const uint64_t* address[kDrainBatch];
#pragma unroll
                for (int batch = 0; batch < kDrainBatch; ++batch) {
                    const int my_ordinal = drain_ordinal + batch * group + lane % group;
                    seen[batch] = wanted[batch] = 0;
                    address[batch] = nullptr;
                    if (endpoint < endpoints && my_ordinal < produced) {
                        const int token = device_load(state.chan_remote_tokens + size_t(channel) * stride + my_ordinal);
                        const uint32_t remote = endpoint_mask_of(z.dims, me, state.plan_mask[token]);
                        if ((remote >> endpoint) & 1u) {
                            wanted[batch] = sequence(epoch, token);
                            address[batch] = ack_at(z, own, channel, my_ordinal % slots, endpoint);
                        }
                    }
                }
                wait_memory_ops();
                compiler_barrier();
#pragma unroll
                for (int batch = 0; batch < kDrainBatch; ++batch)
                    if (address[batch]) seen[batch] = host_load_global(address[batch]);
                int missing_ordinal = 0x7FFFFFFF;
#pragma unroll
                for (int batch = kDrainBatch - 1; batch >= 0; --batch)
                    if (seen[batch] != wanted[batch]) missing_ordinal = drain_ordinal + batch * group + lane % group;
                for (int offset = 32; offset > 0; offset >>= 1) {
                    const int other = __shfl_xor(missing_ordinal, offset);
                    missing_ordinal = other < missing_ordinal ? other : missing_ordinal;
                }
                // Everything before the first miss is done.
                drain_ordinal = missing_ordinal < drain_ordinal + per_pass ? missing_ordinal : drain_ordinal + per_pass;
                if (drain_ordinal >= produced) drained = true;
                else if (missing_ordinal != 0x7FFFFFFF) next_drain_poll = now_ticks() + 20 * state.clock_khz / 1000;
                PCIE_EP_PROFILE(profile.add(kProfilePollSum, profile.now() - poll_begin); if (drained) profile.first(kProfileDrainedNs); else profile.add(kProfilePollMisses);)
            }
        }
        if (workers_finished && drained && !relays_drained) {
            bool done = true;
            if (lane < z.dims.domains) done = host_load(signal_at(own, z.relay_drained_offset, flow_index(z, channel, lane))) == epoch;
            relays_drained = __all(done);
        }
        if (workers_finished && drained && (relays_drained || failed) && broadcast_first(int(device_load(&q.rx_finished[channel].value)))) break;
        // Guardian: this wavefront outlives TX so that a stalled RX still times out.
        PCIE_EP_PROFILE(const uint64_t health_begin = profile.now();)
        const bool unhealthy = health.poll(state, lane);
        PCIE_EP_PROFILE(profile.add(kProfileHealthSum, profile.now() - health_begin);)
        const bool forced = channel == 0 && state.control_abort_after && now_ticks() - start >= state.control_abort_after;
        if (unhealthy || broadcast_first(forced ? 1 : 0)) {
            if (lane == 0) {
                record_error(state, kErrRingProgressWait);
                raise_abort(q);
            }
            break;
        }
        backoff();
    }
    if (lane == 0) {
        atomicAdd(reinterpret_cast<unsigned long long*>(state.channel_stats + channel * kStatFields + kStatRingFull),
                  static_cast<unsigned long long>(stage_busy));
        atomicAdd(reinterpret_cast<unsigned long long*>(state.channel_stats + channel * kStatFields + kStatPreparedAhead),
                  static_cast<unsigned long long>(prepared_ahead));
        // Only this wavefront writes the channel's mapped abort word.
        if (aborted(q)) store_release_system(signal_at(own, z.channel_abort_offset, channel), epoch);
        // Both directions are complete (or aborted): the channel's end time.
        device_store(state.channel_timestamps_ns + channel * 2 + 1, ticks_to_ns(state, now_ticks()));
    }
    PCIE_EP_PROFILE(profile.values[kProfileHealthScans] = uint64_t(health.scans); if (produced == 0) profile.first(kProfileDrainedNs);
                    profile.last(kProfileFinishedNs); profile.save(state.profiling, channel, lane);)
}

// ---------------------------------------------------------------------------------------
// RX control
// ---------------------------------------------------------------------------------------
// The first look of a receive control at its descriptor queues (entry `ahead` of every
// source's queue): the same load as in the first pass of rx_control's loop, issued by
// the kernel's entry code while the role still waits to be let in (the queues it hands
// tickets out through are being reset), so that the round trip over the host link and
// that wait overlap.
struct RxFirstPoll {
    u32x4 published;
    bool issued;
};
// Which descriptor queue a lane of a receive control looks at: up to 64 / P entries ahead in every source's queue.
struct RxLane {
    int lookahead, source, ahead, my_domain;
    bool member, replica;
    __device__ __forceinline__ RxLane(const DeviceState& state, int lane) {
        const SegmentLayout& z = state.z;
        const int ranks = z.dims.num_ranks, me = state.local_rank;
        lookahead = kWave / ranks > 32 ? 32 : kWave / ranks;
        source = lane / lookahead;
        ahead = lane % lookahead;
        member = source < ranks && source != me;
        // A source of another domain is read from the replica ring its relay fills
        // for this rank's domain (advanced_common.cuh:237-247).
        replica = member && reads_replica(z.dims, source, me);
        my_domain = z.dims.domains ? z.dims.rank_domain[me] : 0;
    }
    // Entry `ordinal` of the lane's queue (entry 0 of the own queue for a lane without one: never loaded).
    __device__ __forceinline__ Descriptor* entry(const DeviceState& state, int channel, int ordinal) const {
        const SegmentLayout& z = state.z;
        const int me = state.local_rank;
        char* segment = state.seg[member ? source : me];
        return replica ? replica_descriptor_at(z, segment, channel, my_domain, me, ordinal) : descriptor_at(z, segment, channel, me, ordinal);
    }
};
__device__ __forceinline__ RxFirstPoll rx_first_poll(const DeviceState& state, int channel, int lane) {
    const RxLane at(state, lane);
    RxFirstPoll poll{{0u, 0u, 0u, 0u}, true};
    if (at.member) poll.published = host_load_b128_at(at.entry(state, channel, at.ahead));
    return poll;
}

__device__ __forceinline__ void rx_control(const DeviceState& state, TransportQueues& q, int channel, int lane, RxFirstPoll first_poll) {
    const SegmentLayout& z = state.z;
    const int ranks = z.dims.num_ranks, me = state.local_rank;
    const uint64_t begin = now_ticks();
    const uint64_t epoch = dispatch_epoch(state);
    PCIE_EP_PROFILE(RoleProfile profile(state.clock_khz);)
    if (!dedicated_prefix_producer(state)) elect_receive_prefixes(state, lane PCIE_EP_PROFILE(, profile));
    // Polling does not wait for the prefixes: a descriptor entry is valid as soon as
    // its tag carries this epoch and the next ordinal, whatever the counts say, so
    // rows are requested from the first microseconds of the kernel on.  The counts
    // (how many rows each source sends on this channel) are only needed to know
    // when to stop; the payload wavefronts wait for the prefixes after they have
    // requested a row, before they compute where it goes.
    const RxLane at(state, lane);
    const int lookahead = at.lookahead, source = at.source, ahead = at.ahead, my_domain = at.my_domain;
    const bool member = at.member, replica = at.replica;
    int expected = member ? 0x7FFFFFFF : 0, total = 0x7FFFFFFF;
    bool counts_known = false, prefix_failed = false;
    const uint64_t below = lanes_below(lane);
    const uint64_t group_mask = (1ull << lookahead) - 1ull;
    const __amdgpu_buffer_rsrc_t ring = device_resource(q.rx, sizeof(q.rx));
    Deadline deadline(begin);
    int consumed = 0, issued = 0;
    int64_t not_ready = 0, ring_waits = 0;
    bool failed = false;
    while (!failed && !prefix_failed) {
        // The pass that consumes the look taken at entry goes straight to it: the abort word and the
        // prefixes' state (two trips to device memory) cannot have anything to say a few microseconds
        // into the launch, and are looked at from the second pass on.
        const bool entry_pass = first_poll.issued && consumed == 0 && issued == 0 && !counts_known;
        if (!entry_pass && broadcast_first(aborted(q) ? 1 : 0)) break;
        if (!counts_known && !entry_pass) {
            const int verdict = receive_prefix_verdict(state, epoch, lane);
            if (verdict < 0) {
                prefix_failed = true;
                break;
            }
            if (verdict > 0) {
                expected = member ? device_load(state.expected_receive_counts + channel * ranks + source) : 0;
                total = ahead == 0 ? expected : 0;
                for (int offset = 32; offset > 0; offset >>= 1) total += __shfl_xor(total, offset);
                counts_known = true;
                PCIE_EP_PROFILE(profile.first(kProfileCountsKnownNs);)
            }
        }
        if (counts_known && issued >= total) break;
        const int ordinal = consumed + ahead;
        const bool want = member && ordinal < expected;
        Descriptor* descriptor = at.entry(state, channel, want ? ordinal : 0);
        // One 16-byte load brings READY together with the slot and token it guards.
        u32x4 published = {0u, 0u, 0u, 0u};
        PCIE_EP_PROFILE(const uint64_t poll_begin = profile.now(); profile.add(kProfilePolls);)
        if (entry_pass) {
            // Nothing has been consumed and the counts are not known: this pass would load exactly what was loaded at entry.
            published = first_poll.published;
            first_poll.issued = false;
        } else if (want) {
            published = host_load_b128_at(descriptor);
        }
        PCIE_EP_PROFILE(profile.add(kProfilePollSum, profile.now() - poll_begin);)
        const bool ready = want && (uint64_t(published[0]) | uint64_t(published[1]) << 32) == sequence(epoch, ordinal);
        const uint64_t ready_lanes = __ballot(ready);
        // Descriptors of one source are consumed in order: accept the leading run.
        const uint64_t group = (ready_lanes >> (source < ranks ? source * lookahead : 0)) & group_mask;
        const int run = __builtin_ctzll(~group | (1ull << lookahead));
        const bool accept = ready && ahead < run;
        const uint64_t accepted = __ballot(accept);
        if (!accepted) {
            PCIE_EP_PROFILE(profile.add(kProfilePollMisses);)
            ++not_ready;
            backoff();
            continue;
        }
        // Slot and token come from the peer (or its relay) and become the base of a
        // host read: a value outside the ring would make the payload wavefront read
        // beyond the pinned segment, which is a memory fault, not a protocol error.
        // Same verdict as a wrong identity: terminal, nothing is ACKed.
        {
            const int named_slot = int(published[2]), named_token = int(published[3]);
            const int ring_slots = replica ? z.dims.replica_slots : z.dims.payload_slots;
            const bool outside = accept && (named_slot < 0 || named_slot >= ring_slots || named_token < 0 || named_token >= z.dims.max_tokens);
            if (__any(outside)) {
                if (lane == 0) {
                    record_error(state, kErrPayloadSequence);
                    raise_abort(q);
                }
                failed = true;
                break;
            }
        }
        const int ticket_index = reserve_tickets(q.rx_tail, __popcll(accepted), lane) + __popcll(accepted & below);
        const int slot = int(published[2]), token = int(published[3]);
        const uint64_t payload_sequence = sequence(epoch, token);
        bool pending = accept;
        while (true) {
            if (pending && ring_entry_free(q.rx_taken, epoch, ticket_index)) {
                const uint32_t at = uint32_t(ticket_index % kRing) * uint32_t(sizeof(RxEntry));
                device_store_b32(ring, at + 0, uint32_t(source));
                device_store_b32(ring, at + 4, uint32_t(slot));
                device_store_b32(ring, at + 8, uint32_t(token));
                device_store_b32(ring, at + 12, uint32_t(channel));
                device_store_b32(ring, at + 16, uint32_t(payload_sequence));
                device_store_b32(ring, at + 20, uint32_t(payload_sequence >> 32));
                device_store_b32(ring, at + 24, uint32_t(issued + __popcll(accepted & below)));
                device_store_b32(ring, at + 28, replica ? 1u : 0u);
                // The ticket body is complete before its tag.
                wait_memory_ops();
                device_store(q.rx_ready + ticket_index % kRing, sequence(epoch, ticket_index));
                pending = false;
            }
            if (!__any(pending)) break;
            ++ring_waits;
            if (broadcast_first((aborted(q) || deadline.expired(state)) ? 1 : 0)) {
                failed = true;
                break;
            }
            backoff();
        }
        issued += __popcll(accepted);
        PCIE_EP_PROFILE(profile.first(kProfileFirstTicketNs); profile.last(kProfileLastTicketNs);)
        // Every accepted entry is captured in a ticket: return the credits, one
        // store per source for the whole run (entries are consumed in order).  The
        // payload ACK and the ticket ring entry are separate resources.
        if (member && ahead == 0 && run > 0 && !failed)
            host_field_store(replica ? replica_credit_at(z, state.seg[source], channel, my_domain, me) : credit_at(z, state.seg[source], channel, me),
                             sequence(epoch, consumed + run - 1));
        if (member) consumed += run;
    }
    if (prefix_failed) {
        if (lane == 0) {
            raise_abort(q);
            device_store(&q.rx_finished[channel].value, 1u);
        }
        PCIE_EP_PROFILE(profile.save(state.profiling, state.z.dims.channels + channel, lane);)
        return;
    }
    // RX is finished when every ticket has been retired by a worker.
    while (true) {
        if (broadcast_first(aborted(q) ? 1 : 0)) break;
        if (broadcast_first(int(device_load(&q.rx_retired[channel].value))) >= issued && issued >= total) break;
        backoff();
    }
    PCIE_EP_PROFILE(profile.first(kProfileWorkersDoneNs); profile.values[kProfileItems] = uint64_t(issued);)
    if (lane == 0) {
        atomicAdd(reinterpret_cast<unsigned long long*>(state.channel_stats + channel * kStatFields + kStatRxNotReady),
                  static_cast<unsigned long long>(not_ready));
        // Column 1 of the receive/expand diagnostic: how many receive tickets of
        // this channel have completed their scatter (fused_receive.cuh:290-294).
        if (state.overlap_diagnostic) state.receive_expand_overlap[channel * 2 + 1] = int64_t(device_load(&q.rx_retired[channel].value));
        atomicAdd(reinterpret_cast<unsigned long long*>(state.channel_stats + channel * kStatFields + kStatRingFull),
                  static_cast<unsigned long long>(ring_waits));
        device_store(&q.rx_finished[channel].value, 1u);
    }
    PCIE_EP_PROFILE(profile.last(kProfileFinishedNs); profile.save(state.profiling, state.z.dims.channels + channel, lane);)
}

// ---------------------------------------------------------------------------------------
// Local bypass, padding and the final reduction
// ---------------------------------------------------------------------------------------
// Work items: own tokens 0 .. T-1, then (with zero padding on an expanded
// layout) the local experts' alignment gaps.  Every wavefront of the local
// workgroups claims items one at a time until none is left.
template <bool kVector>
__device__ __forceinline__ void local_rows(const DeviceState& state, TransportQueues& q, int lane) {
    const uint64_t epoch = dispatch_epoch(state);
    // Destination rows depend on the receive prefixes of this epoch.
    int ready = 0;
    if (lane == 0) {
        while (true) {
            const uint64_t value = device_load(state.receive_prefix_state + 1);  // what it guards is read with device-scope loads
            if (value == epoch) { ready = 1; break; }
            // The wavefront that computes the prefixes owns the timeout.
            if (value == kPrefixFailed || aborted(q) || load_error_code(state)) break;
            __builtin_amdgcn_s_sleep(48);
        }
    }
    if (!broadcast_first(ready)) return;
    if (!wait_for_plan(state, q, lane)) return;
    const bool padding = state.expand && state.fuse_expand && state.zero_padding;
    const int items = state.num_tokens + (padding ? state.z.local_experts : 0);
    while (true) {
        uint32_t claimed = 0;
        if (lane == 0) claimed = aborted(q) ? 0xFFFFFFFFu : device_add(&q.local_head.value, 1u);
        const int item = broadcast_first(int(claimed));
        if (item < 0 || item >= items) return;
        if (item >= state.num_tokens) {
            zero_padding_of_expert<kVector>(state, item - state.num_tokens, lane);
        } else if (!local_token_rows<kVector>(state, item, lane)) {
            if (lane == 0) {
                record_error(state, kErrExpandedCapacity);
                raise_abort(q);
            }
            return;
        }
    }
}

// Called by every role wavefront as its last act.  Everything the reduction
// reads was written with device-scope stores or atomics, so waiting for this
// wavefront's own operations is all the ordering the count needs.
__device__ __forceinline__ void finish_role(const DeviceState& state, TransportQueues& q, int lane, uint32_t roles) {
    wait_memory_ops();
    uint32_t earlier = 0;
    if (lane == 0) earlier = device_add(&q.finished.value, 1u);
    if (uint32_t(broadcast_first(int(earlier))) + 1u != roles) return;
    // Last one out: column sums of the per-channel statistics and the span of
    // the channel timestamps.  Done after failures too (the reference launches
    // advanced_reduce_statistics unconditionally).
    // The whole kernel waits for this wavefront: every word is requested before the
    // first is used (lane l reads words l, l + 64, ...), and the sums and the span
    // come out of lane shuffles - two round trips to memory, not one per channel.
    const int channels = state.z.dims.channels;
    constexpr int kStatWordsPerLane = kMaxChannels * kStatFields / kWave;
    int64_t words[kStatWordsPerLane];
#pragma unroll
    for (int i = 0; i < kStatWordsPerLane; ++i) {
        const int word = lane + i * kWave;
        words[i] = word < channels * kStatFields ? device_load(state.channel_stats + word) : 0;
    }
    // Channel c's start and end stamps are words 2c and 2c + 1: lane l takes word l.
    const int64_t stamp = lane < channels * 2 ? device_load(state.channel_timestamps_ns + lane) : 0;
    // kStatFields divides 64: word w belongs to field w % kStatFields whatever i is.
    int64_t sum = 0;
#pragma unroll
    for (int i = 0; i < kStatWordsPerLane; ++i) sum += words[i];
    for (int offset = kStatFields; offset < kWave; offset <<= 1) sum += __shfl_xor(sum, offset);
    if (lane < kStatFields) state.stats[lane] = sum;
    // Even lanes hold start stamps (earliest non-zero wins), odd lanes end stamps (latest wins).
    int64_t span = lane % 2 == 0 && stamp == 0 ? INT64_MAX : stamp;
    for (int offset = 2; offset < kWave; offset <<= 1) {
        const int64_t other = __shfl_xor(span, offset);
        span = lane % 2 == 0 ? (other < span ? other : span) : (other > span ? other : span);
    }
    if (lane == 0) state.transport_timestamps_ns[0] = span == INT64_MAX ? 0 : span;
    if (lane == 1) state.transport_timestamps_ns[1] = span;
    // Prologue inside this launch: every workgroup has read the epoch word by now.
    if (lane == 0 && state.fused) *state.epoch = dispatch_epoch(state);
}

// ---------------------------------------------------------------------------------------
// TX payload worker
// ---------------------------------------------------------------------------------------
template <bool kFp8, bool kVector>
__device__ __forceinline__ float tx_copy_row(const DeviceState& state, const uint16_t* input, __amdgpu_buffer_rsrc_t slot, int lane) {
    const int hidden = state.z.dims.hidden;
    if constexpr (kFp8) return quantize_row<kVector>(input, HostCodes{slot}, hidden, lane);
    copy_row_to_host<kVector>(input, slot, hidden, lane);
    return 1.0f;
}

// Counters a payload wavefront accumulates over the rows it moves, flushed once when it ends.
struct WorkerCounters {
    int64_t writes = 0, deliveries = 0, published = 0, credit_miss = 0, reads = 0;
};

// Moves the own token of transmit ticket `ticket_index` (already marked ready)
// into its host slot and publishes it.  Returns false when the wavefront must stop.
template <bool kFp8, bool kVector>
__device__ __forceinline__ bool tx_row(const DeviceState& state, TransportQueues& q, uint32_t* scratch, int lane, int ticket_index, const Deadline& deadline,
                       WorkerCounters& counters PCIE_EP_PROFILE(, RoleProfile& profile, bool sampled)) {
    const SegmentLayout& z = state.z;
    const int ranks = z.dims.num_ranks, topk = z.dims.topk, me = state.local_rank;
    const int endpoint_count = z.endpoints;
    const int slots = z.dims.payload_slots, descriptors = z.dims.descriptor_slots;
    const int stride = (z.dims.max_tokens + z.dims.channels - 1) / z.dims.channels;
    char* own = state.seg[me];
    const uint64_t epoch = dispatch_epoch(state);
    const int meta_dwords = z.meta_bytes / 4;
    const __amdgpu_buffer_rsrc_t ring = device_resource(q.tx, sizeof(q.tx));
    {
        // Copy the ticket out of the ring (one dword per lane), then free its entry.
        const uint32_t entry_base = uint32_t(ticket_index % kRing) * uint32_t(sizeof(TxEntry));
        const uint32_t word = device_load_b32(ring, entry_base + uint32_t(lane < int(sizeof(TxEntry) / 4) ? lane : 0) * 4u);
        const int token = __shfl(int(word), 0), ordinal = __shfl(int(word), 1);
        const uint32_t endpoints = uint32_t(__shfl(int(word), 2));
        const int channel = __shfl(int(word), 3);
        const int my_descriptor = __shfl(int(word), 4 + (lane < endpoint_count ? lane : 0));
        wait_memory_ops();
        if (lane == 0) device_store(q.tx_taken + ticket_index % kRing, sequence(epoch, ticket_index));
        const int slot = ordinal % slots;
        const bool targeted = lane < endpoint_count && ((endpoints >> lane) & 1u);
        if (ordinal == 0 && lane == 0) state.prefix_tx_timestamps_ns[(channel + 1) * 2] = ticks_to_ns(state, now_ticks());

        // Flow control: the slot's previous occupant must be ACKed by all its
        // targets and a descriptor entry must have been consumed before reuse
        // (advanced_dispatch.cuh:158-187).  One lane per endpoint.
        bool slot_ok = true, credit_ok = true;
        uint64_t previous_sequence = 0;
        if (ordinal >= slots) {
            const int previous_token = device_load(state.chan_remote_tokens + size_t(channel) * stride + ordinal - slots);
            const uint32_t previous_remote = endpoint_mask_of(z.dims, me, state.plan_mask[previous_token]);
            slot_ok = !(lane < endpoint_count && ((previous_remote >> lane) & 1u));
            previous_sequence = sequence(epoch, previous_token);
        }
        if (targeted && my_descriptor >= descriptors) credit_ok = false;
        bool stop = false;
        PCIE_EP_PROFILE(const uint64_t flow_begin = sampled ? profile.now() : 0;)
        while (true) {
            if (!slot_ok) slot_ok = host_load(ack_at(z, own, channel, slot, lane)) == previous_sequence;
            if (!credit_ok) credit_ok = credit_covers(host_load(credit_at(z, own, channel, lane)), epoch, my_descriptor, descriptors);
            if (__all(slot_ok && credit_ok)) break;
            ++counters.credit_miss;
            if (broadcast_first((aborted(q) || deadline.expired(state)) ? 1 : 0)) {
                stop = true;
                break;
            }
            backoff();
        }
        if (stop) return false;
        compiler_barrier();
        PCIE_EP_PROFILE(const uint64_t copy_begin = sampled ? profile.now() : 0; if (sampled) profile.add(kProfileTxFlowWaitSum, copy_begin - flow_begin);)

        // Slot metadata: composed in this wavefront's LDS scratch, then copied out
        // as consecutive dwords.  Weights are the live ones of this dispatch.
        char* slot_base = slot_at(z, own, channel, slot);
        for (int index = lane; index < meta_dwords; index += kWave) scratch[index] = 0;
        fence_lds();
        if (lane == 0) {
            scratch[0] = uint32_t(token);
            scratch[1] = state.plan_mask[token];
        }
        if (lane < ranks) scratch[kMetaRankOrdinalsOffset / 4 + lane] = uint32_t(state.plan_rank_ord[size_t(token) * ranks + lane]);
        if (lane < topk) {
            scratch[kMetaBranchOffset / 4 + lane] = uint32_t(state.plan_exp_idx[size_t(token) * topk + lane]);
            scratch[kMetaBranchOffset / 4 + topk + lane] = uint32_t(state.plan_exp_ord[size_t(token) * topk + lane]);
            scratch[kMetaBranchOffset / 4 + 2 * topk + lane] =
                float_bits(state.topk_weights ? state.topk_weights[size_t(token) * topk + lane] : 1.0f);
        }
        if (lane == kWave - 1) test_delay(state.tx_delay);
        const __amdgpu_buffer_rsrc_t slot_resource = host_resource(slot_base, uint32_t(z.meta_offset + z.meta_bytes));
        const float scale = tx_copy_row<kFp8, kVector>(state, state.x + size_t(token) * z.dims.hidden,
                                                       host_resource(slot_base, uint32_t(z.payload_bytes)), lane);
        if (lane == 0) scratch[2] = float_bits(scale);
        fence_lds();
        if (lane == meta_dwords - 1 || (lane == kWave - 1 && meta_dwords > kWave)) test_delay(state.metadata_delay);
        for (int index = lane; index < meta_dwords; index += kWave)
            host_store_b32(slot_resource, uint32_t(z.meta_offset + index * 4), scratch[index]);
        // Every lane's payload and metadata stores have been acknowledged before
        // any lane publishes a descriptor (the counters are wave-wide).
        wait_memory_ops();
        PCIE_EP_PROFILE(if (sampled) profile.add(kProfileTxCopySum, profile.now() - copy_begin);)
        if (targeted) {
            // READY, slot and token in one 16-byte store: nothing to order inside the entry.
            const uint64_t ready = sequence(epoch, my_descriptor);
            const u32x4 entry = {uint32_t(ready), uint32_t(ready >> 32), uint32_t(slot), uint32_t(token)};
            host_store_b128(host_resource(descriptor_at(z, own, channel, lane, my_descriptor), 16), 0, entry);
        }
        if (ordinal == 0 && lane == 0) state.prefix_tx_timestamps_ns[(channel + 1) * 2 + 1] = ticks_to_ns(state, now_ticks());
        ++counters.writes;
        // Logical deliveries count destination ranks; a relay endpoint stands for
        // all targeted ranks of its domain with one descriptor.
        counters.deliveries += __popc(state.plan_mask[token] & ~(1u << me));
        counters.published += __popc(endpoints);
        fence_lds();  // scratch is reused by the next ticket
        if (lane == 0) device_add(&q.tx_retired[channel].value, 1u);
    }
    return true;
}

// ---------------------------------------------------------------------------------------
// RX + scatter worker
// ---------------------------------------------------------------------------------------
// Reads the row of receive ticket `ticket_index` (already marked ready) from its
// host slot and stores it to its destination rows.  Returns false when the
// wavefront must stop.
template <bool kFp8, bool kVector>
__device__ __forceinline__ bool rx_row(const DeviceState& state, TransportQueues& q, uint32_t* scratch, int lane, int ticket_index, WorkerCounters& counters,
                       const Deadline& deadline, bool& gate_open, bool& prefixes_known PCIE_EP_PROFILE(, RoleProfile& profile, bool sampled)) {
    const SegmentLayout& z = state.z;
    const int topk = z.dims.topk, me = state.local_rank, local = z.local_experts;
    const int hidden = z.dims.hidden;
    const uint64_t epoch = dispatch_epoch(state);
    const bool scatter = state.expand && state.fuse_expand;
    const __amdgpu_buffer_rsrc_t ring = device_resource(q.rx, sizeof(q.rx));
    {
        const uint32_t entry_base = uint32_t(ticket_index % kRing) * uint32_t(sizeof(RxEntry));
        const uint32_t word = device_load_b32(ring, entry_base + uint32_t(lane < 8 ? lane : 0) * 4u);
        const int source = __shfl(int(word), 0), slot = __shfl(int(word), 1), ticket_token = __shfl(int(word), 2);
        const int channel = __shfl(int(word), 3);
        const uint64_t payload_sequence = uint64_t(uint32_t(__shfl(int(word), 4))) | uint64_t(uint32_t(__shfl(int(word), 5))) << 32;
        const int channel_ordinal = __shfl(int(word), 6);
        const bool replica = __shfl(int(word), 7) != 0;
        PCIE_EP_PROFILE(profile.first(kProfileFirstEntryNs);)
        // The ticket now lives in registers: its ring entry may be reused while
        // this wavefront is still moving the row.
        wait_memory_ops();
        if (lane == 0) device_store(q.rx_taken + ticket_index % kRing, sequence(epoch, ticket_index));
        const char* slot_base = replica ? replica_slot_at(z, state.replica_in[source], channel, slot) : slot_at(z, state.seg[source], channel, slot);
        uint64_t* slot_ack = replica ? replica_ack_at(z, state.seg[source], channel, z.dims.rank_domain[me], slot, me)
                                     : ack_at(z, state.seg[source], channel, slot, me);
        const __amdgpu_buffer_rsrc_t payload = host_resource(slot_base, uint32_t(z.payload_bytes));
        const __amdgpu_buffer_rsrc_t slot_meta = host_resource(slot_base + z.meta_offset, uint32_t(z.meta_bytes));
        if (lane == kWave - 1) test_delay(state.rx_delay);
        // Tickets are handed out from the first descriptor on, but no row is requested
        // before the producer of the prefixes has put its reads of the count mailboxes
        // on the link (a few hundred bytes that everything waits for must not queue
        // behind megabytes of row reads).  That producer has seen every source's counts by
        // then.  The prologue of the same launch may still be laying out thousands of own
        // tokens: count stores that leave with rows already in flight are acknowledged some
        // 12 us later than on an idle link (measured), so a peer whose counts came early
        // learns this rank's that much later.  It holds its first rows in registers for as
        // long, with their requests on the link - no link time is lost - and among ranks
        // that start together every gate opens after the last counts have arrived anyway.
        // The wavefront waits here with its ticket read and its addresses computed:
        // the requests leave the moment the gate opens.
        while (!gate_open) {
            int gate = 0;
            if (lane == 0) {
                if (device_load(state.receive_prefix_state) & kPrefixRequested) gate = 1;
                else if (aborted(q) || device_load(state.receive_prefix_state + 1) == kPrefixFailed) gate = -1;
                else if (deadline.expired(state)) {
                    record_error(state, kErrRingProgressWait);
                    raise_abort(q);
                    gate = -1;
                }
            }
            gate = broadcast_first(gate);
            if (gate < 0) return false;
            if (gate > 0) gate_open = true;
            else __builtin_amdgcn_s_sleep(24);
        }
        PCIE_EP_PROFILE(profile.first(kProfileGateOpenNs);)
        // Column 0 of the receive/expand diagnostic: this row's host read starts
        // while an earlier row of the channel has not finished its scatter (the
        // conservative proof point of fused_receive.cuh:216-225; a count, not a time).
        if (state.overlap_diagnostic && lane == 0 && channel_ordinal > 0 &&
            int(device_load(&q.rx_retired[channel].value)) < channel_ordinal)
            atomicAdd(reinterpret_cast<unsigned long long*>(state.receive_expand_overlap + channel * 2), 1ull);

        PCIE_EP_PROFILE(const uint64_t request_begin = sampled ? profile.now() : 0;)
        // Metadata first (it arrives first), payload right behind it.
        const u32x4 meta_vector = host_load_b128(slot_meta, uint32_t(lane) * 16u);  // 16 bytes per lane; out of range reads as 0

        RowVectors row;
        const int wire_vectors = kFp8 ? hidden / 16 : hidden / 8;
        const int wire_per_pass = kFp8 ? (kPassItems / 2) * kWave : kPassItems * kWave;
        if constexpr (kVector) {
            // First (usually only) pass of the row.
            if constexpr (kFp8) {
#pragma unroll
                for (int j = 0; j < kPassItems / 2; ++j) row.v[j] = host_load_b128(payload, uint32_t(j * kWave + lane) * 16u);
            } else {
#pragma unroll
                for (int j = 0; j < kPassItems; ++j) row.v[j] = host_load_b128(payload, uint32_t(j * kWave + lane) * 16u);
            }
        }
        PCIE_EP_PROFILE(profile.first(kProfileFirstRequestNs);)
        if (lane < kScratchDwords / 4) {
            scratch[lane * 4] = meta_vector[0];
            scratch[lane * 4 + 1] = meta_vector[1];
            scratch[lane * 4 + 2] = meta_vector[2];
            scratch[lane * 4 + 3] = meta_vector[3];
        }
        fence_lds();
        PCIE_EP_PROFILE(profile.first(kProfileFirstDataNs);)
        const int token = int(scratch[0]);
        const float scale = bits_float(scratch[2]);
        if (token != ticket_token || payload_sequence != sequence(epoch, token)) {
            // Terminal: never forge an ACK for a slot whose identity is unknown
            // (advanced_dispatch.cuh:607-610).
            if (lane == 0) {
                record_error(state, kErrPayloadSequence);
                raise_abort(q);
            }
            return false;
        }

        // The row has been requested; where it goes depends on the receive prefixes,
        // which may still be on their way in the first microseconds of the kernel.
        PCIE_EP_PROFILE(const uint64_t prefix_begin = sampled ? profile.now() : 0;)
        while (!prefixes_known) {
            const int verdict = receive_prefix_verdict(state, epoch, lane);
            if (verdict < 0 || broadcast_first(aborted(q) ? 1 : 0)) return false;
            if (verdict > 0) prefixes_known = true;
            // The row itself is microseconds away: a slow poll costs nothing, and a couple of hundred
            // wavefronts polling fast would slow down the very stores of the prefixes they wait for.
            else __builtin_amdgcn_s_sleep(48);
        }

        PCIE_EP_PROFILE(if (sampled) profile.add(kProfileRxPrefixWaitSum, profile.now() - prefix_begin);)
        // Destination rows, one lane per branch.  Everything the row numbers are
        // made of comes from the peer: the token must be addressed to this rank and
        // its ordinals must lie inside the counts that peer announced, or a store
        // would land in another expert's rows or before the pool.  Same verdict as a
        // wrong identity: terminal, and the slot is not ACKed.
        int64_t my_row = -1;
        int my_expert = -1;
        bool out_of_range = lane == 0 && !((scratch[1] >> me) & 1u);
        if (lane < topk) {
            const int global_expert = int(scratch[kMetaBranchOffset / 4 + lane]);
            const int expert = global_expert - me * local;
            if (global_expert >= 0 && expert >= 0 && expert < local) {
                const int ordinal = int(scratch[kMetaBranchOffset / 4 + topk + lane]);
                const int before = device_load(state.source_expert_prefix + source * local + expert);
                const int through = source + 1 < z.dims.num_ranks ? device_load(state.source_expert_prefix + (source + 1) * local + expert)
                                                                  : device_load(state.expert_counts + expert);
                out_of_range |= ordinal < 0 || ordinal >= through - before;
                if (scatter) {
                    my_expert = expert;
                    my_row = int64_t(device_load(state.expert_offsets + expert)) + before + ordinal;
                }
            }
        }
        if (lane == 0) {
            const int ordinal = int(scratch[kMetaRankOrdinalsOffset / 4 + me]);
            const int first = device_load(state.source_offsets + source);
            out_of_range |= ordinal < 0 || ordinal >= device_load(state.source_offsets + source + 1) - first;
            if (!scatter) my_row = int64_t(first) + ordinal;
        }
        if (__any(out_of_range)) {
            if (lane == 0) {
                record_error(state, kErrPayloadSequence);
                raise_abort(q);
            }
            return false;
        }
        const int64_t capacity = scatter ? state.expanded_capacity : unique_capacity(z.dims);
        if (__any(my_row >= capacity)) {
            if (lane == 0) {
                record_error(state, kErrExpandedCapacity);
                raise_abort(q);
            }
            return false;
        }
        const uint64_t destinations = __ballot(my_row >= 0);
        uint16_t* output_base = scatter ? state.expanded_payload : state.unique_payload;
        if (lane == kWave - 1) test_delay(state.scatter_delay);

        if constexpr (kVector) {
            const int out_vectors = hidden / 8;
            for (int first_wire = 0; first_wire < wire_vectors; first_wire += wire_per_pass) {
                if (first_wire > 0) {
                    if constexpr (kFp8) {
#pragma unroll
                        for (int j = 0; j < kPassItems / 2; ++j) row.v[j] = host_load_b128(payload, uint32_t(first_wire + j * kWave + lane) * 16u);
                    } else {
#pragma unroll
                        for (int j = 0; j < kPassItems; ++j) row.v[j] = host_load_b128(payload, uint32_t(first_wire + j * kWave + lane) * 16u);
                    }
                }
                const bool last_pass = first_wire + wire_per_pass >= wire_vectors;
                if (last_pass) {
                    // All loads of the staged row have returned: release the host slot.
                    if (lane == 0) host_store_release(slot_ack, payload_sequence);
                    PCIE_EP_PROFILE(if (sampled) { wait_memory_ops(); profile.add(kProfileRxRequestSum, profile.now() - request_begin); })
                }
                if constexpr (kFp8) {
                    // 16 codes -> 16 BF16 (two 16-byte vectors); expanded in place from the top.
#pragma unroll
                    for (int j = kPassItems / 2 - 1; j >= 0; --j) {
                        u32x4 lo, hi;
                        dequantize_vector(row.v[j], scale, lo, hi);
                        row.v[2 * j] = lo;
                        row.v[2 * j + 1] = hi;
                    }
                }
                uint64_t remaining = destinations;
                while (remaining) {
                    const int branch = __builtin_ctzll(remaining);
                    remaining &= remaining - 1;
                    const int64_t out_row = __shfl(my_row, branch);
                    u32x4* output = reinterpret_cast<u32x4*>(output_base + size_t(out_row) * hidden);
                    if constexpr (kFp8) {
                        // Wire vector i holds elements [16 i, 16 i + 16) -> output vectors 2 i and 2 i + 1.
#pragma unroll
                        for (int j = 0; j < kPassItems / 2; ++j) {
                            const int index = first_wire + j * kWave + lane;
                            if (index < wire_vectors) {
                                __builtin_nontemporal_store(row.v[2 * j], output + 2 * index);
                                __builtin_nontemporal_store(row.v[2 * j + 1], output + 2 * index + 1);
                            }
                        }
                    } else {
                        row_store_vectors<true>(row, output, first_wire, out_vectors, lane);
                    }
                }
            }
        } else {
            // Scalar fall-back (row length not a multiple of 16 bytes): 2-byte items.
            for (int first = 0; first < hidden; first += kPassScalars * kWave) {
                RowScalars items;
#pragma unroll
                for (int j = 0; j < kPassScalars; ++j) {
                    const int index = first + j * kWave + lane;
                    if (index < hidden) {
                        if constexpr (kFp8) items.v[j] = fp8_dequantize_element(host_load_b8(payload, uint32_t(index)), scale);
                        else items.v[j] = host_load_b16(payload, uint32_t(index) * 2u);
                    }
                }
                if (first + kPassScalars * kWave >= hidden) {
                    if (lane == 0) host_store_release(slot_ack, payload_sequence);
                }
                uint64_t remaining = destinations;
                while (remaining) {
                    const int branch = __builtin_ctzll(remaining);
                    remaining &= remaining - 1;
                    const int64_t out_row = __shfl(my_row, branch);
                    uint16_t* output = output_base + size_t(out_row) * hidden;
#pragma unroll
                    for (int j = 0; j < kPassScalars; ++j) {
                        const int index = first + j * kWave + lane;
                        if (index < hidden) output[index] = items.v[j];
                    }
                }
            }
        }

        // Row metadata (advanced_layout.cuh:207-215; layout.cuh:31-48).
        if (scatter) {
            if (my_row >= 0) {
                state.expanded_expert_idx[my_row] = my_expert;
                state.expanded_weights[my_row] = bits_float(scratch[kMetaBranchOffset / 4 + 2 * topk + lane]);
                state.expanded_source_meta[my_row * 3] = source;
                state.expanded_source_meta[my_row * 3 + 1] = token;
                state.expanded_source_meta[my_row * 3 + 2] = lane;
            }
        } else {
            const int64_t out_row = __shfl(my_row, 0);
            if (lane < topk) {
                const int expert = int(scratch[kMetaBranchOffset / 4 + lane]);
                const bool is_local = expert >= me * local && expert < (me + 1) * local;
                state.unique_topk_idx[out_row * topk + lane] = is_local ? expert - me * local : -1;
                state.unique_topk_weights[out_row * topk + lane] = is_local ? bits_float(scratch[kMetaBranchOffset / 4 + 2 * topk + lane]) : 0.0f;
                state.unique_expert_ordinals[out_row * topk + lane] = int(scratch[kMetaBranchOffset / 4 + topk + lane]);
            }
            if (lane == 0) {
                state.unique_source_meta[out_row * 3] = source;
                state.unique_source_meta[out_row * 3 + 1] = token;
                state.unique_source_meta[out_row * 3 + 2] = -1;
            }
        }
        ++counters.reads;
        PCIE_EP_PROFILE(if (sampled) profile.add(kProfileRxScatterSum, profile.now() - request_begin);)
        fence_lds();  // scratch is reused by the next ticket
        if (lane == 0) device_add(&q.rx_retired[channel].value, 1u);
    }
    return true;
}

// ---------------------------------------------------------------------------------------
// Payload wavefront: moves rows of either direction
// ---------------------------------------------------------------------------------------
// A payload wavefront serves whichever direction needs it.  The two directions
// share the host link: row reads return on the downstream half, but their
// requests travel upstream beside the row writes, so a transmit side that runs
// flat out (about 24 GB/s next to saturated reads) takes request slots from the
// receive side (55 instead of 57 GB/s) and is then idle for the rest of the
// dispatch.  The wavefronts therefore split in proportion to the work that is
// LEFT in each direction: with rem_tx and rem_rx rows still unclaimed,
//     transmitting wavefronts : receiving wavefronts = kTxWeight * rem_tx : kRxWeight * (rem_rx - lead)
// (one wavefront's share of the link's write rate is about 4/9 of its share of
// the read rate), re-evaluated before every row, so the writes are spread
// thinly over the whole dispatch whatever the routing's send/receive ratio is.
// `lead` makes the transmit side end a little earlier than the receive side (by
// the time the link needs for kTxLeadBytes, at most a quarter of the rows to
// receive): a transmitted row is only finished
// when its receivers have acknowledged it, and that round trip then hides
// behind the last received rows instead of following them.  The rule corrects
// itself: a direction that falls behind has more left and gets more wavefronts;
// at most half of the wavefronts transmit and, while anything is left to send, at
// least kMinTxWaves.  Until both totals are known (the receive total comes with
// the receive prefixes) those kMinTxWaves transmit and everybody else waits for
// the first descriptors.  A wavefront whose direction has nothing to
// claim takes a ticket of the other direction instead - at once when its own
// direction is finished, after kIdleCrossoverUs otherwise (at the start of a
// dispatch the first descriptors are a few microseconds away and a receive
// wavefront must not bind itself to a transmit row for them) - but only a
// ticket its producer has already reserved (head < tail), so it never commits
// itself to a row that does not exist yet.
constexpr int64_t kTxWeight = 9, kRxWeight = 4;
constexpr int64_t kTxLeadBytes = 24 << 20;
constexpr int kMinTxWaves = 16;
constexpr uint64_t kIdleCrossoverUs = 30;
constexpr int kPreGateRows = 32;

template <bool kFp8, bool kVector>
__device__ __forceinline__ void payload_worker(const DeviceState& state, TransportQueues& q, uint32_t* scratch, int lane, int order, int waves) {
    const uint64_t epoch = dispatch_epoch(state);
    Deadline deadline(now_ticks());
    WorkerCounters counters;
    PCIE_EP_PROFILE(RoleProfile profile(state.clock_khz); uint64_t idle_begin = 0; int rows_moved = 0;)
    bool prefixes_known = false, gate_open = false;
    const int lead = int(kTxLeadBytes / int64_t(state.z.meta_offset + state.z.meta_bytes));
    uint64_t idle_since = 0;  // 0: the last look found work
    while (true) {
        // 0: nothing to do now, 1: transmit, 2: receive, -1: both directions are finished or the kernel aborts.
        int choice = 0;
        PCIE_EP_PROFILE(const uint64_t look_begin = profile.now();)
        int gate_seen = gate_open ? 1 : 0;
        if (lane == 0) {
            if (aborted(q)) choice = -1;
            else {
                const int tx_head = int(device_load(&q.tx_head.value)), rx_head = int(device_load(&q.rx_head.value));
                const bool tx_backlog = tx_head < int(device_load(&q.tx_tail.value));
                bool rx_backlog = rx_head < int(device_load(&q.rx_tail.value));
                // Receive tickets are there long before the first row may be requested (rx_row
                // holds the gate).  Only the first kPreGateRows of them are claimed ahead of
                // it, by wavefronts that then wait with their addresses ready: if every
                // wavefront did, they would all fire at once and each would have its first
                // row after the time the link needs for all of them, with nobody left to transmit.
                if (rx_backlog && !gate_seen && rx_head >= kPreGateRows) {
                    gate_seen = (device_load(state.receive_prefix_state) & kPrefixRequested) != 0;
                    rx_backlog = gate_seen != 0;
                }
                const int tx_total = device_load(&q.tx_head.total), rx_total = device_load(&q.rx_head.total);
                const bool tx_done = tx_total >= 0 && tx_head >= tx_total, rx_done = rx_total >= 0 && rx_head >= rx_total;
                // Totals unknown: a handful of wavefronts start to transmit, the others
                // wait for the first descriptors.
                bool prefer_tx = order < kMinTxWaves && 2 * order < waves;
                if (tx_total >= 0 && rx_total >= 0) {
                    const int rx_rows = rx_total - rx_head - (lead < rx_total / 4 ? lead : rx_total / 4);
                    const int64_t tx_left = tx_done ? 0 : kTxWeight * (tx_total - tx_head), rx_left = rx_rows > 0 ? kRxWeight * rx_rows : 0;
                    prefer_tx = rx_done || (tx_left > 0 && 2 * order < waves &&
                                            (order < kMinTxWaves || int64_t(order) * (tx_left + rx_left) < int64_t(waves) * tx_left));
                }
                const bool own_backlog = prefer_tx ? tx_backlog : rx_backlog, other_backlog = prefer_tx ? rx_backlog : tx_backlog;
                const bool own_done = prefer_tx ? tx_done : rx_done;
                if (own_backlog) choice = prefer_tx ? 1 : 2;
                else if (other_backlog) {
                    const uint64_t now = now_ticks();
                    if (!idle_since) idle_since = now;
                    // Towards the receive side after a while; towards the transmit side only once
                    // everything has been received.  A transmit row waits for its receivers (slot ACK,
                    // descriptor credit); if every wavefront of a rank could end up in such a wait, two
                    // ranks whose receivers are each other's kernels could wait for each other for ever.
                    // The wavefronts that do not transmit by the rule above (at least half of them)
                    // therefore never do while a row may still come in.
                    if (own_done || (prefer_tx && now - idle_since > kIdleCrossoverUs * state.clock_khz / 1000)) choice = prefer_tx ? 2 : 1;
                }
                if (choice) idle_since = 0;
                else {
                    if (tx_done && rx_done) choice = -1;
                    else if (deadline.expired(state)) {
                        record_error(state, kErrRingProgressWait);
                        raise_abort(q);
                        choice = -1;
                    }
                }
            }
        }
        choice = broadcast_first(choice);
        gate_open = broadcast_first(gate_seen) != 0;
        if (choice < 0) break;
        if (choice == 0) {
            PCIE_EP_PROFILE(if (!idle_begin) idle_begin = profile.now();)
            // Every look is seven loads of the queue counters; a couple of hundred idle wavefronts
            // looking four times a microsecond would keep the producers' own updates of those
            // counters waiting.  About a microsecond between looks.
            __builtin_amdgcn_s_sleep(32);
            continue;
        }
        PCIE_EP_PROFILE(if (idle_begin) { profile.add(kProfileIdleSum, profile.now() - idle_begin); idle_begin = 0; })
        const bool transmit = choice == 1;
        QueueCounter& head = transmit ? q.tx_head : q.rx_head;
        PCIE_EP_PROFILE(profile.first(kProfileFirstClaimNs); const uint64_t claim_begin = profile.now(); if (!profile.values[kProfileFirstLookNs]) profile.values[kProfileFirstLookNs] = look_begin;)
        const int ticket_index = claim_ticket(head, lane);
        // Several wavefronts may have seen the same backlog: a claim beyond the last
        // ticket of the dispatch is simply dropped, an earlier one waits for its tag.
        if (wait_ticket(state, q, transmit ? q.tx_ready : q.rx_ready, head, ticket_index, epoch, lane, deadline) < 0) {
            if (broadcast_first(aborted(q) ? 1 : 0)) break;
            continue;
        }
        PCIE_EP_PROFILE(profile.first(kProfileFirstTaggedNs); profile.add(kProfileTicketWaitSum, profile.now() - claim_begin); const bool sampled = rows_moved++ % kProfileSampleStride == 0;
                        if (sampled) profile.add(transmit ? kProfileSampledTxRows : kProfileSampledRxRows); profile.add(transmit ? kProfileTxRows : kProfileRxRows);)
        const bool go_on = transmit ? tx_row<kFp8, kVector>(state, q, scratch, lane, ticket_index, deadline, counters PCIE_EP_PROFILE(, profile, sampled))
                                    : rx_row<kFp8, kVector>(state, q, scratch, lane, ticket_index, counters, deadline, gate_open, prefixes_known PCIE_EP_PROFILE(, profile, sampled));
        PCIE_EP_PROFILE(profile.last(kProfileLastRowNs);)
        if (!go_on) break;
    }
    // Workers serve every channel; their counts go to channel 0's row of the
    // per-channel statistics, whose column sums are what callers read.
    if (lane == 0) {
        auto* stats = reinterpret_cast<unsigned long long*>(state.channel_stats);
        if (counters.writes || counters.credit_miss) {
            atomicAdd(stats + kStatHostWrites, static_cast<unsigned long long>(counters.writes));
            atomicAdd(stats + kStatDeliveries, static_cast<unsigned long long>(counters.deliveries));
            atomicAdd(stats + kStatDescriptors, static_cast<unsigned long long>(counters.published));
            atomicAdd(stats + kStatTxCreditMiss, static_cast<unsigned long long>(counters.credit_miss));
        }
        if (counters.reads) atomicAdd(stats + kStatHostReads, static_cast<unsigned long long>(counters.reads));
    }
    PCIE_EP_PROFILE(profile.values[kProfileItems] = uint64_t(rows_moved); profile.save(state.profiling, 2 * state.z.dims.channels + order, lane);)
}

// Workgroup b < C is the control workgroup of channel b (wavefront 0 TX control,
// wavefront 1 RX control); workgroups b >= C hold payload wavefronts only.  With
// no payload workgroups configured the control workgroups carry the payload
// wavefronts themselves.
template <bool kFp8, bool kVector>
__global__ void __launch_bounds__(kTransportMaxThreads) transport_kernel(DeviceState launch_state) {
    // The launch argument is read where it lies, in the kernel-argument segment:
    // every field is then a scalar load from constant memory and every pointer in
    // it a global pointer.  A by-value copy would be a private object of 1 KB that
    // each role reads back through scratch loads, with generic pointers in it.
#if defined(__HIP_DEVICE_COMPILE__)
    const DeviceState& state = *reinterpret_cast<const DeviceState*>(__builtin_amdgcn_kernarg_segment_ptr());
#else
    const DeviceState& state = launch_state;  // the host pass only parses the kernel
#endif
    __shared__ WaveScratch lds;
    extern __shared__ __align__(16) unsigned char prologue_lds[];  // sized by the launcher when the prologue rides in this launch
    const int channels = state.z.dims.channels;
    int block = transport_block(transport_grid(state), int(blockIdx.x));
    if (block < 0) return;  // a filler id
    int wave = threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    uint32_t* scratch = lds.words[wave];
    TransportQueues& q = *state.queues;
    const int payload_waves = state.tx_waves + state.rx_waves;
    const int payload_groups = state.worker_groups > 0 ? state.worker_groups : 0;
    const int waves_per_group = int(blockDim.x) / kWave;
    const int prologue_groups = fused_prologue_groups(state);
    // Role wavefronts of the launch: controls, payload and local-bypass wavefronts, the producer of the receive
    // prefixes where it is a wavefront of its own, one per prologue workgroup and a second one for the epoch begin.
    const uint32_t roles = uint32_t(2 * channels + (payload_groups ? payload_groups : channels) * payload_waves + state.local_groups * waves_per_group +
                                    (dedicated_prefix_producer(state) ? 1 : 0) + prologue_groups + (prologue_groups ? 1 : 0));
    bool begun = true;
    if (state.fused) {
        // The prologue's workgroups carry the lowest indices: they are started first.
        // Workgroup 0 begins the epoch, the ones after it lay out one chunk of tokens each.
        if (block < prologue_groups) {
            if (block == 0) {
                // The helpers' findings: zeroed before any wavefront of the workgroup goes its own way.
                __shared__ int findings[kTransportMaxThreads / kWave];
                if (threadIdx.x < kTransportMaxThreads / kWave) findings[threadIdx.x] = 0;
                __syncthreads();
                epoch_begin_role(state, wave, lane, waves_per_group, findings);
                if (wave >= 2) return;
                return finish_role(state, q, lane, roles);
            }
            prologue_chunk<8, true>(state, prologue_lds, waves_per_group, state.prologue_chunks, block - 1);
            if (wave == 0) finish_role(state, q, lane, roles);
            return;
        }
        block -= prologue_groups;
    }
    const int channel_groups = control_groups(state);
    // Which control this wavefront is, if any - known before the role may start.  The two roles whose first
    // action is a read over the host link issue it now: a receive control its first look at the descriptor
    // queues, the producer of the prefixes its first look at the sources' counts_ready.  The wait for the epoch
    // begin (the queues are being reset; 3 us into the launch) then runs inside that round trip (4.4 us).
    const bool control_of_pair = payload_groups && block < channel_groups;
    const bool transmit_group = control_of_pair && (block + prologue_groups) % kControlXcds == 0;
    const bool prefix_producer = transmit_group && block / 2 == 0 && wave == 2 && dedicated_prefix_producer(state);
    int receive_channel = -1;
    if (control_of_pair && !transmit_group && wave < 2 && 2 * (block / 2) + wave < channels) receive_channel = 2 * (block / 2) + wave;
    if (!payload_groups && block < channel_groups && wave == 1) receive_channel = block;
    RxFirstPoll first_poll{{0u, 0u, 0u, 0u}, false};
    if (receive_channel >= 0) first_poll = rx_first_poll(state, receive_channel, lane);
    PrefixFirstLook first_look{0, false};
    if (prefix_producer) first_look = prefix_first_look(state, lane);
    if (state.fused) {
        begun = __syncthreads_or(threadIdx.x == 0 ? int(wait_for_begin(state, q)) : 0) != 0;
    } else if (__syncthreads_or(threadIdx.x == 0 ? int(load_error_code(state) != 0) : 0)) {
        return;  // the prologue kernel in front of this one failed
    }
    if (block >= channel_groups + payload_groups) {
        if (begun) local_rows<kVector>(state, q, lane);
        return finish_role(state, q, lane, roles);
    }
    if (block < channel_groups) {
        if (payload_groups) {
            // Control workgroups of their own: the two control XCDs alternate over their
            // ids, and a workgroup holds the controls of ONE direction for a pair of
            // channels (wavefront w: channel 2 * pair + w), transmit on one XCD, receive
            // on the other.  A receive control polls descriptors in host memory all the
            // time, and each of those reads stays in its XCD's memory queues for as long
            // as the row reads in front of it on the link take; the transmit controls,
            // the producer of the prefixes and the prologue only touch device memory
            // while rows flow and must not wait behind them.
            const bool transmit = (block + prologue_groups) % kControlXcds == 0;
            const int pair = block / 2, channel = 2 * pair + wave;
            if (wave < 2) {
                if (channel >= channels) return;
                if (begun) {
                    if (transmit) tx_control(state, q, channel, lane);
                    else rx_control(state, q, channel, lane, first_poll);
                }
                return finish_role(state, q, lane, roles);
            }
            // The producer of the receive prefixes: third wavefront of the first transmit control workgroup.
            if (!prefix_producer) return;
            if (begun) receive_prefix_role(state, lane, first_look);
            return finish_role(state, q, lane, roles);
        }
        if (wave < 2) {
            if (begun) {
                if (wave == 0) tx_control(state, q, block, lane);
                else rx_control(state, q, block, lane, first_poll);
            }
            return finish_role(state, q, lane, roles);
        }
        wave -= 2;
    }
    if (wave >= payload_waves) return;
    // Position of this wavefront among all payload wavefronts, wavefront-major: a
    // direction's share is spread over the workgroups before it doubles up in one.
    const int groups = payload_groups ? payload_groups : channels;
    const int group = payload_groups ? block - channel_groups : block;
    if (begun) payload_worker<kFp8, kVector>(state, q, scratch, lane, wave * groups + group, groups * payload_waves);
    finish_role(state, q, lane, roles);
    // Every role loop has an explicit completion, abort or timeout exit and no
    // workgroup barrier follows the entry verdict.
}

}  // namespace

int transport_threads(const DeviceState& state) {
    const int payload = state.tx_waves + state.rx_waves;
    const int control = state.worker_groups > 0 ? 2 : 2 + payload;
    return (control > payload ? control : payload) * kWave;
}

// How many transport workgroups one compute unit holds at once (registers, LDS and
// wavefront slots of the instantiation that `state` selects).
hipError_t transport_workgroups_per_unit(const DeviceState& state, int* per_unit) {
    const int threads = transport_threads(state);
    if (threads > kTransportMaxThreads) return hipErrorInvalidValue;
    const bool fp8 = state.z.dims.wire_fp8 != 0;
    const bool vector = fp8 ? state.z.dims.hidden % 16 == 0 : state.z.dims.hidden % 8 == 0;
    const size_t lds = state.fused ? prologue_lds_bytes(state.z, threads / kWave) : 0;
    if (fp8 && vector) return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_unit, transport_kernel<true, true>, threads, lds);
    if (fp8) return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_unit, transport_kernel<true, false>, threads, lds);
    if (vector) return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_unit, transport_kernel<false, true>, threads, lds);
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_unit, transport_kernel<false, false>, threads, lds);
}

hipError_t launch_transport(const DeviceState& state, hipStream_t stream) {
    const dim3 grid(transport_grid(state).blocks), block(transport_threads(state));
    if (int(block.x) > kTransportMaxThreads) return hipErrorInvalidValue;
    size_t dynamic_lds = 0;
    if (state.fused) {
        // The prologue's chunks are the workgroup's own wavefronts; the conditions are those of fused_prologue_fits().
        if (!fused_prologue_fits(state.z, int(block.x), state.z.dims.max_tokens)) return hipErrorInvalidValue;
        dynamic_lds = prologue_lds_bytes(state.z, int(block.x) / kWave);
    }
    const bool fp8 = state.z.dims.wire_fp8 != 0;
    // BF16 rows need 16-byte granularity on both sides; FP8 additionally needs
    // whole 16-code vectors on the wire.
    const bool vector = fp8 ? state.z.dims.hidden % 16 == 0 : state.z.dims.hidden % 8 == 0;
    if (fp8 && vector) hipLaunchKernelGGL((transport_kernel<true, true>), grid, block, dynamic_lds, stream, state);
    else if (fp8) hipLaunchKernelGGL((transport_kernel<true, false>), grid, block, dynamic_lds, stream, state);
    else if (vector) hipLaunchKernelGGL((transport_kernel<false, true>), grid, block, dynamic_lds, stream, state);
    else hipLaunchKernelGGL((transport_kernel<false, false>), grid, block, dynamic_lds, stream, state);
    return hipGetLastError();
}

}  // namespace pcie_ep

// The dispatch prologue as device code: epoch begin, route validation, stable
// layout and count publication of one chunk of tokens per workgroup.
//
// Replaces five launches of the reference's eager dispatch
// (csrc/buffers/advanced.hpp:472-486): advanced_begin_epoch
// (advanced_layout.cuh:9-89), advanced_route_flags (:287-309),
// advanced_stable_ordinals (:311-356), advanced_prepare_channels_parallel
// (:358-425) and publish_counts (layout.cuh:7-29).
//
// Layout method (wave64): the tokens are cut into chunks of W wavefronts, one
// workgroup per chunk.  For every bin (P destination ranks, then E experts)
// and every wavefront of the chunk a 64-bit hit mask is built in LDS (rank
// bins from ballots, expert bins with one LDS OR per branch).  A thread per
// bin turns the W popcounts into exclusive prefixes and publishes the chunk's
// bin totals; the chunk's base is the sum of the totals of all earlier chunks
// (each chunk waits for the flags of its predecessors: every workgroup of the
// small grid is resident, and lower chunks never wait for higher ones).  Every
// token then reads back `base[bin] + prefix[wave][bin] + popcount(mask[wave][bin]
// & lanes_below)` - its stable ordinal.  Work is O(T*K), not O((P+E)*T*K), and
// bit-identical to a serial scan because an ordinal only depends on which
// earlier tokens hit the bin.  A token's expert ids stay in registers between
// the passes.  Chunk 0 (the leader) additionally begins the epoch, sums the chunk
// totals and publishes the counts.
//
// The same code runs in two places (kFused):
//  * as a kernel of its own in front of the transport kernel (chunks of up to 16
//    wavefronts); the kernel boundary hands its results to the transport kernel;
//  * as the first workgroups of the transport kernel's own launch (chunks of the
//    transport workgroup's four wavefronts).  The transport roles then start
//    with it: the receive side polls descriptors and the other sources' counts
//    while the layout is computed.  The epoch begin (clearing, abort words, the
//    wait for the previous count mailbox: everything that needs a round trip over
//    the host link before the counts may be stored) is then a workgroup of its
//    own, epoch_begin_role(), so that the layout never waits for it.  What
//    crosses workgroups inside the one launch goes through device-scope flags:
//    `begun` (diagnostics cleared, queues reset), `verdict` (no abort word set,
//    previous mailbox consumed), `plan_chunks` / `plan_ready` (route plan written
//    through to memory, transmit total known, counts published) and the abort
//    word (the prologue failed).  The epoch word is then advanced by the last
//    role of the launch to end, so that every workgroup of the launch reads the
//    same value at its start.
#pragma once

#include "device_common.h"
#include "launch.h"

namespace pcie_ep {

// Workgroup barrier that orders LDS only: a wavefront with host or device
// memory operations in flight does not drain them just to share an LDS table.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Per-chunk record in the layout scratch (int32 units).  The first error_key()
// fields are also the order of the plan's totals in the leader's LDS.
struct ChunkRecord {
    int bins, channels, ranks, domains;
    __host__ __device__ int stride() const { return error_key() + 4; }
    __host__ __device__ int counts() const { return 0; }
    __host__ __device__ int chan_counts() const { return bins; }
    __host__ __device__ int chan_remote() const { return bins + channels * ranks; }
    __host__ __device__ int chan_relay() const { return chan_remote() + channels; }
    __host__ __device__ int error_key() const { return chan_relay() + channels * domains; }
};

// Field-wise sums over `count` chunk records (record r begins at first + r * stride,
// `fields` consecutive words of each are summed) into sums[fields] in LDS, by the
// whole workgroup.  A read of another workgroup's record is a trip to memory of half
// a microsecond: the (record, field) pairs are dealt round the threads and read
// kBatch at a time, each batch issued back to back and waited for once, so the
// trips overlap instead of following each other.
template <int kBatch>
__device__ __forceinline__ void sum_chunk_records(const int32_t* first, int stride, int fields, int count, int* sums) {
    for (int field = threadIdx.x; field < fields; field += blockDim.x) sums[field] = 0;
    lds_barrier();
    const int total = fields * count, step = int(blockDim.x);
    int record = int(threadIdx.x) / fields, field = int(threadIdx.x) % fields;
    for (int n = threadIdx.x; n < total; n += step * kBatch) {
        int value[kBatch], where[kBatch];
#pragma unroll
        for (int slot = 0; slot < kBatch; ++slot) {
            const bool valid = n + slot * step < total;
            where[slot] = valid ? field : -1;
            // Past the end: a harmless read of the first word instead of a branch between the loads.
            value[slot] = device_load_global(first + (valid ? size_t(record) * stride + field : size_t(0)));
            field += step;
            while (field >= fields) {
                field -= fields;
                ++record;
            }
        }
#pragma unroll
        for (int slot = 0; slot < kBatch; ++slot)
            if (where[slot] >= 0 && value[slot] != 0) atomicAdd(sums + where[slot], value[slot]);
    }
    lds_barrier();
}

// The count mailboxes of every destination (layout.cuh:7-20) from the plan's
// totals in LDS: host stores issued, not waited for.  A mailbox block starts on a
// 128-byte line and is stored as whole 16-byte vectors (the words behind its last
// field are padding of the block): 17 transactions per destination instead of 65.
__device__ __forceinline__ void store_counts(const DeviceState& state, const ChunkRecord& record, const int* totals) {
    const SegmentLayout& z = state.z;
    char* own = state.seg[state.local_rank];
    const int ranks = z.dims.num_ranks, local = z.local_experts;
    const int vectors = (z.mailbox_dwords + 3) / 4;
    const __amdgpu_buffer_rsrc_t mailboxes = host_resource(own + z.mailbox_offset, uint32_t(size_t(ranks) * z.mailbox_stride));
    for (int index = threadIdx.x; index < ranks * vectors; index += blockDim.x) {
        const int destination = index / vectors, vector = index % vectors;
        u32x4 value;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int field = vector * 4 + k;
            int word = 0;
            if (field == 0) word = totals[record.counts() + destination];
            else if (field <= local) word = totals[record.counts() + ranks + destination * local + field - 1];
            else if (field < z.mailbox_dwords) word = totals[record.chan_counts() + (field - 1 - local) * ranks + destination];
            value[k] = uint32_t(word);
        }
        host_store_b128(mailboxes, uint32_t(size_t(destination) * z.mailbox_stride) + uint32_t(vector) * 16u, value);
    }
    // Relay mode: what each (channel, domain) relay flow of this source will carry.
    const int domains = z.dims.domains, channels = z.dims.channels;
    for (int index = threadIdx.x; index < domains * channels; index += blockDim.x) {
        const int domain = index / channels, channel = index % channels;
        host_field_store(relay_mailbox_at(z, own, domain) + channel, totals[record.chan_relay() + channel * domains + domain]);
    }
}

// counts_ready after the mailboxes.  Every writer waits for its own stores; the
// leader publishes after the join (a leader-only wait would not cover the other
// writers: layout.cuh:21-28).
__device__ __forceinline__ void publish_counts(const DeviceState& state, uint64_t epoch PCIE_EP_PROFILE(, RoleProfile& profile)) {
    const SegmentLayout& z = state.z;
    wait_memory_ops();
    __syncthreads();
    PCIE_EP_PROFILE(profile.first(kPrologueMailboxAckedNs);)
    if (threadIdx.x == 0) host_store_release(signal_at(state.seg[state.local_rank], z.counts_ready_offset), epoch);
    PCIE_EP_PROFILE(profile.first(kPrologueCountsReadyNs);)
}

// ---- begin of the epoch (advanced_layout.cuh:9-89) ---------------------------------------
// The per-dispatch diagnostics and the ticket queues are cleared, every rank's
// abort words are looked at (any one set is terminal: code 19), the epoch number
// is checked (code 20) and the previous count mailbox must have been consumed by
// every peer (code 11).

// Clearing, by `count` threads of which this one is number `index`.  kThrough:
// written through to memory, for readers on other compute units of the same launch.
template <bool kThrough>
__device__ __forceinline__ void clear_epoch_state(const DeviceState& state, int index, int count) {
    const int channels = state.z.dims.channels;
    TransportQueues& q = *state.queues;
    const auto clear = [](auto* address, auto value) {
        if constexpr (kThrough) device_store(address, value);
        else *address = value;
    };
    for (int i = index; i < kErrorFields; i += count) clear(state.errors + i, int64_t(0));
    for (int i = index; i < kStatFields; i += count) clear(state.stats + i, int64_t(0));
    for (int i = index; i < channels * kStatFields; i += count) clear(state.channel_stats + i, int64_t(0));
    for (int i = index; i < channels * 2; i += count) {
        clear(state.channel_timestamps_ns + i, int64_t(0));
        clear(state.receive_expand_overlap + i, int64_t(0));
    }
    for (int i = index; i < 2; i += count) {
        clear(state.transport_timestamps_ns + i, int64_t(0));
        clear(state.receive_prefix_state + i, uint64_t(0));
    }
    for (int i = index; i < (channels + 1) * 2; i += count) clear(state.prefix_tx_timestamps_ns + i, int64_t(0));
    // Ticket queues of the transport kernel: counters back to zero, totals
    // unknown.  The rings' tags carry the epoch and need no clearing.
    QueueCounter* globals[] = {&q.rx_tail, &q.tx_tail, &q.rx_head, &q.tx_head, &q.abort, &q.local_head, &q.finished, &q.plan_chunks};
    if (index < 8) {
        clear(&globals[index]->value, 0u);
        clear(&globals[index]->total, -1);
    }
    for (int i = index; i < channels; i += count) {
        QueueCounter* counters[] = {&q.rx_retired[i], &q.tx_retired[i], &q.rx_finished[i]};
        for (QueueCounter* counter : counters) {
            clear(&counter->value, 0u);
            clear(&counter->total, -1);
        }
    }
}

// All abort words of all ranks, read by `count` threads of which this one is
// number `index` (whole wavefronts, all lanes active): true when one of this
// thread's words is set.  Memory operations of a wavefront complete in order, so
// nothing may be loaded between the host words - not even a segment's base
// address: lane r holds the base of rank r's segment and hands it out by lane
// shuffle, and all of a thread's words are requested before the first is looked at.
__device__ __forceinline__ bool read_abort_words(const DeviceState& state, int index, int count) {
    const SegmentLayout& z = state.z;
    const int per_rank = abort_flags_per_rank(z), flags = z.dims.num_ranks * per_rank;
    const int lane = lane_id();
    const uint64_t lane_segment = reinterpret_cast<uint64_t>(state.seg[lane < z.dims.num_ranks ? lane : 0]);
    wait_memory_ops();
    const auto segment_of = [&](int rank) {
        return reinterpret_cast<char*>(uint64_t(uint32_t(__shfl(int(uint32_t(lane_segment)), rank))) |
                                       uint64_t(uint32_t(__shfl(int(uint32_t(lane_segment >> 32)), rank))) << 32);
    };
    // Direct mode has at most kMaxRanks * (1 + kMaxChannels) = 528 abort words: nine per lane of one wavefront.
    constexpr int kLoadsPerThread = 9;
    const uint64_t* address[kLoadsPerThread];
#pragma unroll
    for (int i = 0; i < kLoadsPerThread; ++i) {
        const int flag = index + i * count;
        char* segment = segment_of(flag < flags ? flag / per_rank : 0);
        address[i] = flag < flags ? abort_flag_at(z, segment, flag % per_rank) : nullptr;
    }
    uint64_t words[kLoadsPerThread];
#pragma unroll
    for (int i = 0; i < kLoadsPerThread; ++i) words[i] = address[i] ? host_load_global(address[i]) : 0;
    bool set = false;
    // (Relay mode with many domains has more flags than that: the rest is read the plain way.)
    for (int flag = index + kLoadsPerThread * count; flag < flags; flag += count)
        set |= host_load(abort_flag_at(z, state.seg[flag / per_rank], flag % per_rank)) != 0;
#pragma unroll
    for (int i = 0; i < kLoadsPerThread; ++i) set |= words[i] != 0;
    return set;
}

// Wavefront-wide wait until every peer has consumed the previous count mailbox
// (advanced_layout.cuh:60-88): only then may the counts be overwritten.  `consumed_word`
// is lane r's first look at rank r's word.  False after the timeout or a peer's abort.
__device__ __forceinline__ bool wait_mailbox_consumed(const DeviceState& state, uint64_t tag, uint64_t consumed_word, int lane) {
    const SegmentLayout& z = state.z;
    char* own = state.seg[state.local_rank];
    const bool polls = lane < z.dims.num_ranks && lane != state.local_rank;
    bool consumed = !polls || consumed_word == tag - 1;
    HealthCheck health(state, now_ticks());
    while (!__all(consumed)) {
        if (health.poll(state, lane)) return false;
        backoff();
        if (!consumed) consumed = host_load(signal_at(own, z.counts_consumed_offset, lane)) == tag - 1;
    }
    return true;
}

// A launch of its own: the leader workgroup begins the epoch.  Returns false when
// the dispatch must not go on; the error is then recorded and the own channel
// abort word stored.
__device__ __forceinline__ bool begin_epoch(const DeviceState& state, uint64_t tag PCIE_EP_PROFILE(, RoleProfile& profile)) {
    const SegmentLayout& z = state.z;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    char* own = state.seg[state.local_rank];
    clear_epoch_state<false>(state, threadIdx.x, blockDim.x);
    uint64_t consumed_word = tag - 1;
    if (wave == 0 && tag > 1 && lane < z.dims.num_ranks && lane != state.local_rank) consumed_word = host_load(signal_at(own, z.counts_consumed_offset, lane));
    const bool any_abort = __syncthreads_or(read_abort_words(state, threadIdx.x, blockDim.x));
    PCIE_EP_PROFILE(profile.first(kPrologueBegunNs); profile.first(kPrologueVerdictNs);)
    __shared__ int begin_failed;
    if (threadIdx.x == 0) {
        begin_failed = 0;
        if (tag >= 0x100000000ull) record_error(state, kErrEpochExhausted);
        else if (any_abort) record_error(state, kErrAlreadyAborted);
        // Terminal for this buffer.
        if (load_error_code(state)) {
            host_store_release(signal_at(own, z.channel_abort_offset), tag);
            begin_failed = 1;
        }
    }
    __syncthreads();
    if (begin_failed) return false;
    if (wave == 0 && tag > 1 && !wait_mailbox_consumed(state, tag, consumed_word, lane) && lane == 0) {
        record_error(state, kErrCountsMailboxWait);
        host_store_release(signal_at(own, z.channel_abort_offset), tag);
        begin_failed = 1;
    }
    __syncthreads();
    PCIE_EP_PROFILE(profile.first(kPrologueMailboxFreeNs);)
    return !begin_failed;
}

// Inside the transport launch the epoch begins in a workgroup of its own, as
// independent wavefronts (memory operations of a wavefront complete in order, so
// one that has asked for host words cannot learn that its stores have arrived
// before those words are back):
//  * wavefront 0 clears (written through) and announces `begun`, which every
//    other role of the launch waits for before it touches the queues or records
//    anything;
//  * the other wavefronts share the abort words between them (the round trip of a
//    few hundred scattered host words is shorter from several wavefronts); the
//    helpers hand their findings to wavefront 1 through LDS, which also waits for
//    the count mailbox; on success it announces `verdict`, which the layout's
//    leader waits for before it stores the counts, otherwise it records the error
//    (after `begun`) and raises the launch's abort word.
// Wavefronts 0 and 1 are roles of the launch (they call finish_role), the helpers are not.
__device__ __forceinline__ void epoch_begin_role(const DeviceState& state, int wave, int lane, int waves, int* findings) {
    const SegmentLayout& z = state.z;
    TransportQueues& q = *state.queues;
    char* own = state.seg[state.local_rank];
    const uint64_t tag = *state.epoch + 1;
    PCIE_EP_PROFILE(RoleProfile profile(state.clock_khz);
                    const int profile_row = profile_rows(z.dims.channels, (state.worker_groups > 0 ? state.worker_groups : z.dims.channels) * (state.tx_waves + state.rx_waves)) - 2;)
    if (wave == 0) {
        clear_epoch_state<true>(state, lane, kWave);
        wait_memory_ops();
        if (lane == 0) device_store(&q.begun.value, epoch_flag(tag));
        PCIE_EP_PROFILE(profile.first(kPrologueBegunNs);
                        if (lane == 0 && state.profiling) state.profiling[size_t(profile_row) * kProfileFields + kPrologueBegunNs] = int64_t(profile.values[kPrologueBegunNs]);)
        return;
    }
    // findings[w]: 0 until reader w (1 .. waves - 1) has looked at its words, then 1 (none set) or 2.
    const int readers = waves - 1;
    if (wave > 1) {
        const bool set = __any(read_abort_words(state, (wave - 1) * kWave + lane, readers * kWave));
        if (lane == 0) lds_store(findings + wave, set ? 2 : 1);
        return;
    }
    uint64_t consumed_word = tag - 1;
    if (tag > 1 && lane < z.dims.num_ranks && lane != state.local_rank) consumed_word = host_load(signal_at(own, z.counts_consumed_offset, lane));
    bool any_abort = __any(read_abort_words(state, lane, readers * kWave));
    for (int helper = 2; helper < waves; ++helper) {
        int finding = 0;
        // The helpers end by themselves after one round trip over the host link.
        while (!(finding = broadcast_first(lds_load(findings + helper)))) backoff();
        any_abort |= finding == 2;
    }
    PCIE_EP_PROFILE(profile.first(kPrologueVerdictNs);)
    int code = 0;
    if (tag >= 0x100000000ull) code = kErrEpochExhausted;
    else if (any_abort) code = kErrAlreadyAborted;
    else if (tag > 1 && !wait_mailbox_consumed(state, tag, consumed_word, lane)) code = kErrCountsMailboxWait;
    PCIE_EP_PROFILE(profile.first(kPrologueMailboxFreeNs);)
    if (lane == 0) {
        if (!code) device_store(&q.verdict.value, epoch_flag(tag));
        // The error record and the counter of finished roles are cleared by the other
        // wavefront: nothing is recorded, and this role does not end, before it has said so.
        const uint64_t start = now_ticks();
        while (device_load(&q.begun.value) != epoch_flag(tag) && now_ticks() - start < state.timeout_ticks) backoff();
        if (code) {
            record_error(state, code);
            // Terminal for this buffer.
            host_store_release(signal_at(own, z.channel_abort_offset), tag);
            device_store(&q.abort.value, 1u);
        }
    }
    // (Wavefront 0 writes the `begun` stamp of this record itself.)
    PCIE_EP_PROFILE(profile.values[kProfileExitNs] = profile.now();
                    if (lane == 0 && state.profiling)
                        for (int field = 0; field < kProfileFields; ++field)
                            if (field != kPrologueBegunNs) state.profiling[size_t(profile_row) * kProfileFields + field] = int64_t(profile.values[field]);)
}

template <int kTopk, bool kFused>
__device__ __forceinline__ void prologue_chunk(const DeviceState& state, unsigned char* lds, int chunk_waves, int chunks, int chunk) {
    const SegmentLayout& z = state.z;
    const int ranks = z.dims.num_ranks, experts = z.dims.num_experts, topk = z.dims.topk;
    const int channels = z.dims.channels, local = z.local_experts;
    const int bins = ranks + experts;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const bool leader = chunk == 0;
    TransportQueues& q = *state.queues;
    // What other workgroups of the same launch read is written through to memory
    // and ordered by waiting for the stores, never by a cache write-back.
    const auto plan_store = [](auto* address, auto value) {
        if constexpr (kFused) device_store(address, value);
        else *address = value;
    };
    // Four consecutive words of a plan array (16-byte aligned), as one store.
    const auto plan_store4 = [](__amdgpu_buffer_rsrc_t array, size_t word, int a, int b, int c, int d) {
        const u32x4 value = {uint32_t(a), uint32_t(b), uint32_t(c), uint32_t(d)};
        if constexpr (kFused) device_store_b128(array, uint32_t(word * 4), value);
        else plain_store_b128(array, uint32_t(word * 4), value);
    };
    const auto plan_array = [](int32_t* base, size_t words) { return device_resource(base, uint32_t(align_up(words * 4, 16))); };
    char* own = state.seg[state.local_rank];
    const int domains = z.dims.domains;
    const ChunkRecord record{bins, channels, ranks, domains};
    uint64_t* chunk_flags = state.layout_flags;
    int32_t* chunk_records = state.layout_records;
    // The epoch word is advanced only after every chunk's flag carries this tag
    // (by the leader, or - inside the transport launch - by the last role to end),
    // so every workgroup of the launch reads the same (previous) epoch here.
    const uint64_t tag = *state.epoch + 1;
    const uint64_t begin_ticks = now_ticks();
    PCIE_EP_PROFILE(RoleProfile profile(state.clock_khz);
                    const int profile_row = profile_rows(channels, (state.worker_groups > 0 ? state.worker_groups : channels) * (state.tx_waves + state.rx_waves)) - 3;)
    __shared__ int stalled;
    if (threadIdx.x == 0) stalled = 0;

    // ---- route ids of this thread's token: requested before anything else ------------------
    const bool layout = !state.reuse_plan && chunk < chunks;
    const int tokens = state.num_tokens;
    const int token = (chunk * chunk_waves + wave) * kWave + lane;
    const bool participant = layout && wave < chunk_waves;
    const bool live = participant && token < tokens;
    int64_t raw[kTopk];
#pragma unroll
    for (int branch = 0; branch < kTopk; ++branch) raw[branch] = (live && branch < topk) ? state.topk_idx[size_t(token) * topk + branch] : -1;

    bool begun = true;
    if constexpr (!kFused) {
        // A launch of its own: the leader begins the epoch itself.
        if (leader) begun = begin_epoch(state, tag PCIE_EP_PROFILE(, profile));
    }

    // ---- stable layout ---------------------------------------------------------------
    uint64_t* masks = reinterpret_cast<uint64_t*>(lds);                       // [W][bins]
    int* base = reinterpret_cast<int*>(masks + size_t(bins) * chunk_waves);    // [bins]
    int* chan_counts = base + bins;                                            // [C][P]
    int* chan_remote = chan_counts + channels * ranks;                         // [C]
    int* chan_relay = chan_remote + channels;                                  // [C][N]
    int* first_error = chan_relay + channels * domains;                        // lowest token * 64 + branch
    // Exclusive prefixes inside the chunk never exceed its 1024 tokens: 16 bits each.
    uint16_t* prefix = reinterpret_cast<uint16_t*>(first_error + 2);           // [W][bins]
    // The leader is chunk 0, whose base is zero: it keeps the totals of the whole
    // plan (in the order of a chunk record) where the other chunks keep their base.
    int* totals = base;
    int expert[kTopk];
    uint32_t destination_mask = 0;
    int route_error = 0x7FFFFFFF;
    if (layout) {
        for (int i = threadIdx.x; i < bins * chunk_waves; i += blockDim.x) masks[i] = 0;
        for (int i = threadIdx.x; i < channels * ranks; i += blockDim.x) chan_counts[i] = 0;
        for (int i = threadIdx.x; i < channels; i += blockDim.x) chan_remote[i] = 0;
        for (int i = threadIdx.x; i < channels * domains; i += blockDim.x) chan_relay[i] = 0;
        if (threadIdx.x == 0) *first_error = 0x7FFFFFFF;
        lds_barrier();
        const int channel = token % channels;
#pragma unroll
        for (int branch = 0; branch < kTopk; ++branch) {
            // Invalid: < -1, >= E, or equal to an earlier id of the same token
            // (advanced_layout.cuh:296-307).  -1 is a legal skip.
            bool invalid = raw[branch] < -1 || raw[branch] >= experts;
#pragma unroll
            for (int previous = 0; previous < branch; ++previous) invalid |= raw[branch] >= 0 && raw[branch] == raw[previous];
            expert[branch] = invalid ? -1 : int(raw[branch]);
            if (live && branch < topk) {
                if (invalid) atomicMin(first_error, token * 64 + branch);
                if (expert[branch] >= 0) {
                    destination_mask |= 1u << (expert[branch] / local);
                    atomicOr(reinterpret_cast<unsigned long long*>(masks + size_t(wave) * bins + ranks + expert[branch]), 1ull << lane);
                }
            }
        }
        PCIE_EP_PROFILE(profile.first(kPrologueRoutesNs);)
        if (participant) {
            for (int rank = 0; rank < ranks; ++rank) {
                const uint64_t hits = __ballot((destination_mask >> rank) & 1u);
                if (lane == 0) masks[size_t(wave) * bins + rank] = hits;
            }
        }
        if (live) {
            // Channel c owns tokens c, c + C, ...; counts include the own rank
            // (advanced_layout.cuh:385-412).
            for (int rank = 0; rank < ranks; ++rank)
                if ((destination_mask >> rank) & 1u) atomicAdd(chan_counts + channel * ranks + rank, 1);
            if (destination_mask & ~(1u << state.local_rank)) atomicAdd(chan_remote + channel, 1);
            // Relay endpoints of the token: one per other domain it reaches
            // (the endpoint counts of advanced_layout.cuh:405-412).
            const uint32_t relayed = endpoint_mask_of(z.dims, state.local_rank, destination_mask) >> ranks;
            for (int domain = 0; domain < domains; ++domain)
                if ((relayed >> domain) & 1u) atomicAdd(chan_relay + channel * domains + domain, 1);
        }
        lds_barrier();
        PCIE_EP_PROFILE(profile.first(kPrologueMasksNs);)
        if (chunks == 1) {
            // The whole plan is this workgroup's: its totals ARE the plan's totals
            // (they stay where they are in LDS, behind the bin totals) and nothing
            // has to travel through the chunk records and flags.
            for (int bin = threadIdx.x; bin < bins; bin += blockDim.x) {
                int running = 0;
                for (int w = 0; w < chunk_waves; ++w) {
                    prefix[size_t(w) * bins + bin] = uint16_t(running);
                    running += __popcll(masks[size_t(w) * bins + bin]);
                }
                totals[bin] = running;
            }
            route_error = *first_error;
            lds_barrier();
        } else {
            // Publish this chunk's totals, then its flag.
            int32_t* mine = chunk_records + size_t(chunk) * record.stride();
            for (int bin = threadIdx.x; bin < bins; bin += blockDim.x) {
                int running = 0;
                for (int w = 0; w < chunk_waves; ++w) {
                    prefix[size_t(w) * bins + bin] = uint16_t(running);
                    running += __popcll(masks[size_t(w) * bins + bin]);
                }
                device_store(mine + record.counts() + bin, running);
            }
            for (int i = threadIdx.x; i < channels * ranks; i += blockDim.x) device_store(mine + record.chan_counts() + i, chan_counts[i]);
            for (int i = threadIdx.x; i < channels; i += blockDim.x) device_store(mine + record.chan_remote() + i, chan_remote[i]);
            for (int i = threadIdx.x; i < channels * domains; i += blockDim.x) device_store(mine + record.chan_relay() + i, chan_relay[i]);
            if (threadIdx.x == 0) device_store(mine + record.error_key(), *first_error);
            wait_memory_ops();
            __syncthreads();
            if (threadIdx.x == 0) device_store(chunk_flags + chunk, tag);
            // Base of this chunk: totals of every earlier chunk (none for the leader).
            for (int earlier = threadIdx.x; earlier < chunk; earlier += blockDim.x) {
                while (device_load(chunk_flags + earlier) != tag) {
                    if (now_ticks() - begin_ticks > state.timeout_ticks) {
                        stalled = 1;
                        break;
                    }
                    backoff();
                }
            }
            __syncthreads();
            if (!stalled && !leader) sum_chunk_records<16>(chunk_records + record.counts(), record.stride(), bins, chunk, base);
            __syncthreads();
        }
        PCIE_EP_PROFILE(profile.first(kPrologueChunkTotalsNs);)
    }
    // This chunk's part of the route plan: every token's stable ordinals.  Nothing
    // in this workgroup reads them; the leader writes its own after the counts are
    // on their way to the peers.
    const auto write_ordinals = [&]() {
        if (live && !stalled) {
            const uint64_t below = lanes_below(lane);
            plan_store(state.plan_mask + token, destination_mask);
            const auto rank_ordinal = [&](int rank) -> int {
                const size_t at = size_t(wave) * bins + rank;
                return ((destination_mask >> rank) & 1u) ? (leader ? 0 : base[rank]) + int(prefix[at]) + int(__popcll(masks[at] & below)) : -1;
            };
            // A token's ordinals are consecutive words: whole 16-byte vectors wherever
            // the row length allows it.
            if (ranks % 4 == 0) {
                const __amdgpu_buffer_rsrc_t rank_ordinals = plan_array(state.plan_rank_ord, size_t(z.dims.max_tokens) * ranks);
                for (int rank = 0; rank < ranks; rank += 4)
                    plan_store4(rank_ordinals, size_t(token) * ranks + rank, rank_ordinal(rank), rank_ordinal(rank + 1), rank_ordinal(rank + 2),
                                rank_ordinal(rank + 3));
            } else {
                for (int rank = 0; rank < ranks; ++rank) plan_store(state.plan_rank_ord + size_t(token) * ranks + rank, rank_ordinal(rank));
            }
            int ordinal[kTopk];
#pragma unroll
            for (int branch = 0; branch < kTopk; ++branch) {
                ordinal[branch] = -1;
                if (branch < topk && expert[branch] >= 0) {
                    const size_t at = size_t(wave) * bins + ranks + expert[branch];
                    ordinal[branch] = (leader ? 0 : base[ranks + expert[branch]]) + prefix[at] + __popcll(masks[at] & below);
                }
            }
            if (topk % 4 == 0) {
                const __amdgpu_buffer_rsrc_t expert_ids = plan_array(state.plan_exp_idx, size_t(z.dims.max_tokens) * topk);
                const __amdgpu_buffer_rsrc_t expert_ordinals = plan_array(state.plan_exp_ord, size_t(z.dims.max_tokens) * topk);
#pragma unroll
                for (int branch = 0; branch < kTopk; branch += 4) {
                    if (branch < topk) {
                        plan_store4(expert_ids, size_t(token) * topk + branch, expert[branch], expert[branch + 1], expert[branch + 2], expert[branch + 3]);
                        plan_store4(expert_ordinals, size_t(token) * topk + branch, ordinal[branch], ordinal[branch + 1], ordinal[branch + 2], ordinal[branch + 3]);
                    }
                }
            } else {
#pragma unroll
                for (int branch = 0; branch < kTopk; ++branch) {
                    if (branch < topk) {
                        plan_store(state.plan_exp_idx + size_t(token) * topk + branch, expert[branch]);
                        plan_store(state.plan_exp_ord + size_t(token) * topk + branch, ordinal[branch]);
                    }
                }
            }
        }
    };
    // Inside the transport launch: wait for a word of the epoch begin.  False when
    // the epoch failed there (abort) or the word never came.
    const auto wait_for_word = [&](const uint32_t* word) {
        int outcome = 0;
        if (threadIdx.x == 0) {
            while (true) {
                if (device_load(word) == epoch_flag(tag)) { outcome = 1; break; }
                if (device_load(&q.abort.value) != 0) break;
                if (now_ticks() - begin_ticks > state.timeout_ticks + state.timeout_ticks / 8) {
                    stalled = 1;
                    break;
                }
                backoff();
            }
        }
        return __syncthreads_or(outcome) != 0;
    };
    if (!leader) {
        write_ordinals();
        if constexpr (kFused) {
            // This chunk's part of the plan is in memory: count it for the leader
            // (the counter is reset by the epoch begin).
            wait_memory_ops();
            if (wait_for_word(&q.begun.value) && threadIdx.x == 0) device_add(&q.plan_chunks.value, 1u);
        }
        return;
    }

    // ---- leader: totals of the whole plan (in LDS) ----------------------------------------
    const int fields = record.error_key();  // counts, channel counts, channel remote tokens, relay counts
    if (state.reuse_plan) {
        // A cached plan: its totals are in memory.
        for (int field = threadIdx.x; field < fields; field += blockDim.x) {
            if (field < bins) totals[field] = state.plan_counts[field];
            else if (field < record.chan_remote()) totals[field] = state.plan_chan_counts[field - record.chan_counts()];
            else if (field < record.chan_relay()) totals[field] = state.plan_chan_remote[field - record.chan_remote()];
            else totals[field] = state.plan_chan_relay[field - record.chan_relay()];
        }
    } else if (chunks != 1) {
        if (!layout && threadIdx.x == 0) *first_error = 0x7FFFFFFF;  // nothing to lay out: no chunk has run
        for (int other = threadIdx.x; other < chunks; other += blockDim.x) {
            while (device_load(chunk_flags + other) != tag) {
                if (now_ticks() - begin_ticks > state.timeout_ticks) {
                    stalled = 1;
                    break;
                }
                backoff();
            }
        }
        __syncthreads();
        if (!stalled) {
            // The lowest error key of any chunk (the leader's own is in place already).
            for (int other = threadIdx.x; other < chunks; other += blockDim.x)
                atomicMin(first_error, device_load(chunk_records + size_t(other) * record.stride() + record.error_key()));
            sum_chunk_records<32>(chunk_records, record.stride(), fields, chunks, totals);
            route_error = *first_error;
        }
    }
    lds_barrier();
    PCIE_EP_PROFILE(profile.first(kPrologueTotalsNs);)

    // ---- epoch verdict -----------------------------------------------------------------
    if constexpr (kFused) begun = wait_for_word(&q.verdict.value);
    else if (threadIdx.x == 0) *state.epoch = tag;
    // The leader's own findings.  Nothing of the error record is touched unless there
    // is something to record (inside the transport launch it is cleared elsewhere,
    // and `verdict` does not say that this has happened yet).
    const int finding = stalled ? kErrRingProgressWait : (route_error != 0x7FFFFFFF ? kErrInvalidRouting : 0);
    if (__syncthreads_or(threadIdx.x == 0 && (finding != 0 || !begun))) {
        bool cleared = true;
        if constexpr (kFused) cleared = wait_for_word(&q.begun.value);
        if (threadIdx.x == 0) {
            if (begun && cleared) {
                if (finding == kErrInvalidRouting) record_error(state, finding, route_error / 64, route_error % 64);
                else record_error(state, finding);
                // Terminal for this buffer.
                host_store_release(signal_at(own, z.channel_abort_offset), tag);
            } else if (kFused && cleared && stalled) {
                record_error(state, kErrRingProgressWait);
            }
            // The transport roles of the same launch are waiting for the plan: they leave instead.
            if constexpr (kFused) device_store(&q.abort.value, 1u);
        }
        PCIE_EP_PROFILE(profile.save(state.profiling, profile_row, threadIdx.x);)
        return;
    }
    const uint64_t epoch = tag;

    // The counts leave for the peers first; the plan's totals and the leader's own
    // ordinals, which only this GPU reads, are written inside the stores' round trip.
    store_counts(state, record, totals);
    if (!state.reuse_plan) {
        // Four arrays, each with room up to the next multiple of four words.
        int32_t* const bases[] = {state.plan_counts, state.plan_chan_counts, state.plan_chan_remote, state.plan_chan_relay};
        const int first[] = {record.counts(), record.chan_counts(), record.chan_remote(), record.chan_relay(), record.error_key()};
        int before = 0;
#pragma unroll
        for (int array = 0; array < 4; ++array) {
            const int words = first[array + 1] - first[array], vectors = (words + 3) / 4;
            const __amdgpu_buffer_rsrc_t target = plan_array(bases[array], size_t(words));
            for (int index = (int(threadIdx.x) - before + int(blockDim.x)) % int(blockDim.x); index < vectors; index += blockDim.x) {
                int word[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) word[k] = index * 4 + k < words ? totals[first[array] + index * 4 + k] : 0;
                plan_store4(target, size_t(index) * 4, word[0], word[1], word[2], word[3]);
            }
            // The next array starts with the threads behind those that served this one.
            before = (before + vectors) % int(blockDim.x);
        }
    }
    // Transmit tickets of this dispatch: every own token with a remote destination.
    if (threadIdx.x == 0) {
        int remote_tokens = 0;
        for (int channel = 0; channel < channels; ++channel) remote_tokens += totals[record.chan_remote() + channel];
        plan_store(&q.tx_head.total, remote_tokens);
    }
    write_ordinals();
    PCIE_EP_PROFILE(profile.first(kPrologueLayoutNs);)
    publish_counts(state, epoch PCIE_EP_PROFILE(, profile));
    if constexpr (kFused) {
        // The counts are with the peers; now the own rows may follow.  Every chunk's
        // part of the plan must be in memory before the transmit side reads it.
        if (threadIdx.x == 0 && !state.reuse_plan) {
            while (int(device_load(&q.plan_chunks.value)) < chunks - 1) {
                if (now_ticks() - begin_ticks > state.timeout_ticks) {
                    record_error(state, kErrRingProgressWait);
                    device_store(&q.abort.value, 1u);
                    break;
                }
                backoff();
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) device_store(&q.plan_ready.value, epoch_flag(tag));
        PCIE_EP_PROFILE(profile.first(kProloguePlanReadyNs);)
    }
    PCIE_EP_PROFILE(profile.save(state.profiling, profile_row, threadIdx.x);)
}

}  // namespace pcie_ep

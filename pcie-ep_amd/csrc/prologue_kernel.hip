// Prologue kernel: epoch begin, route validation, stable layout and count
// publication, fused into one launch.
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
// & lanes_below)` — its stable ordinal.  Work is O(T*K), not O((P+E)*T*K), and
// bit-identical to a serial scan because an ordinal only depends on which
// earlier tokens hit the bin.  A token's expert ids stay in registers between
// the passes.  Workgroup 0 additionally begins the epoch, sums the chunk totals
// and publishes the counts.
#include "device_common.h"
#include "launch.h"

namespace pcie_ep {

namespace {

__device__ void publish_counts(const DeviceState& state, uint64_t epoch PCIE_EP_PROFILE(, RoleProfile& profile)) {
    const SegmentLayout& z = state.z;
    char* own = state.seg[state.local_rank];
    const int ranks = z.dims.num_ranks, local = z.local_experts;
    const int total = ranks * z.mailbox_dwords;
    for (int index = threadIdx.x; index < total; index += blockDim.x) {
        const int destination = index / z.mailbox_dwords;
        const int field = index % z.mailbox_dwords;
        int value;
        if (field == 0) value = state.plan_counts[destination];
        else if (field <= local) value = state.plan_counts[ranks + destination * local + field - 1];
        else value = state.plan_chan_counts[(field - 1 - local) * ranks + destination];
        host_field_store(mailbox_at(z, own, destination) + field, value);
    }
    // Relay mode: what each (channel, domain) relay flow of this source will carry.
    const int domains = z.dims.domains, channels = z.dims.channels;
    for (int index = threadIdx.x; index < domains * channels; index += blockDim.x) {
        const int domain = index / channels, channel = index % channels;
        host_field_store(relay_mailbox_at(z, own, domain) + channel, state.plan_chan_relay[channel * domains + domain]);
    }
    // Every writer waits for its own stores; the leader publishes after the join
    // (a leader-only wait would not cover the other writers: layout.cuh:21-28).
    wait_memory_ops();
    __syncthreads();
    PCIE_EP_PROFILE(profile.first(kPrologueMailboxAckedNs);)
    if (threadIdx.x == 0) host_store_release(signal_at(own, z.counts_ready_offset), epoch);
    PCIE_EP_PROFILE(profile.first(kPrologueCountsReadyNs);)
}

}  // namespace

// Per-chunk record in the layout scratch (int32 units).
struct ChunkRecord {
    int bins, channels, ranks, domains;
    __host__ __device__ int stride() const { return error_key() + 4; }
    __host__ __device__ int counts() const { return 0; }
    __host__ __device__ int chan_counts() const { return bins; }
    __host__ __device__ int chan_remote() const { return bins + channels * ranks; }
    __host__ __device__ int chan_relay() const { return chan_remote() + channels; }
    __host__ __device__ int error_key() const { return chan_relay() + channels * domains; }
};

template <int kTopk>
__global__ void __launch_bounds__(kPrologueMaxThreads) prologue_kernel(DeviceState state, int chunk_waves, int chunks) {
    extern __shared__ __align__(16) unsigned char lds[];
    const SegmentLayout& z = state.z;
    const int ranks = z.dims.num_ranks, experts = z.dims.num_experts, topk = z.dims.topk;
    const int channels = z.dims.channels, local = z.local_experts;
    const int bins = ranks + experts;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int chunk = blockIdx.x;
    const bool leader = chunk == 0;
    char* own = state.seg[state.local_rank];
    const int domains = z.dims.domains;
    const ChunkRecord record{bins, channels, ranks, domains};
    uint64_t* chunk_flags = state.layout_flags;
    int32_t* chunk_records = state.layout_records;
    // The leader bumps the epoch only after every chunk's flag carries this tag,
    // so every workgroup of the launch reads the same (previous) epoch here.
    const uint64_t tag = *state.epoch + 1;
    const uint64_t begin_ticks = now_ticks();
    PCIE_EP_PROFILE(RoleProfile profile(state.clock_khz);
                    const int profile_row = profile_rows(channels, (state.worker_groups > 0 ? state.worker_groups : channels) * (state.tx_waves + state.rx_waves)) - 1;)
    __shared__ int stalled;
    if (threadIdx.x == 0) stalled = 0;

    // Direct mode has at most kMaxRanks * (1 + kMaxChannels) = 528 abort words, a workgroup at least 256 threads.
    constexpr int kAbortLoadsPerThread = 3;
    uint64_t abort_words[kAbortLoadsPerThread] = {0, 0, 0};
    uint64_t consumed_word = tag - 1;
    if (leader) {
        // ---- begin epoch: clear per-dispatch diagnostics -----------------------------
        for (int i = threadIdx.x; i < kErrorFields; i += blockDim.x) state.errors[i] = 0;
        for (int i = threadIdx.x; i < kStatFields; i += blockDim.x) state.stats[i] = 0;
        for (int i = threadIdx.x; i < channels * kStatFields; i += blockDim.x) state.channel_stats[i] = 0;
        for (int i = threadIdx.x; i < channels * 2; i += blockDim.x) {
            state.channel_timestamps_ns[i] = 0;
            state.receive_expand_overlap[i] = 0;
        }
        for (int i = threadIdx.x; i < 2; i += blockDim.x) {
            state.transport_timestamps_ns[i] = 0;
            state.receive_prefix_state[i] = 0;
        }
        for (int i = threadIdx.x; i < (channels + 1) * 2; i += blockDim.x) state.prefix_tx_timestamps_ns[i] = 0;
        // Ticket queues of the transport kernel: counters back to zero, totals
        // unknown.  The rings' tags carry the epoch and need no clearing.
        TransportQueues& q = *state.queues;
        QueueCounter* globals[] = {&q.rx_tail, &q.tx_tail, &q.rx_head, &q.tx_head, &q.abort, &q.local_head, &q.finished};
        if (threadIdx.x < 7) {
            globals[threadIdx.x]->value = 0;
            globals[threadIdx.x]->total = -1;
        }
        for (int i = threadIdx.x; i < channels; i += blockDim.x) {
            q.rx_retired[i].value = q.tx_retired[i].value = q.rx_finished[i].value = 0;
            q.rx_retired[i].total = q.tx_retired[i].total = q.rx_finished[i].total = -1;
        }
        // Abort signals are terminal, and the previous count mailbox must have
        // been consumed.  The host loads are only issued here: their values are
        // first looked at after the layout, so the round trip over the host link
        // hides behind it (a use right here would make every thread wait for it).
        const int per_rank = abort_flags_per_rank(z);
#pragma unroll
        for (int i = 0; i < kAbortLoadsPerThread; ++i) {
            const int index = threadIdx.x + i * int(blockDim.x);
            if (index < ranks * per_rank) abort_words[i] = host_load(abort_flag_at(z, state.seg[index / per_rank], index % per_rank));
        }
        // (Relay mode with many domains has more flags than that: the rest is read the plain way.)
        for (int index = threadIdx.x + kAbortLoadsPerThread * int(blockDim.x); index < ranks * per_rank; index += blockDim.x)
            abort_words[0] |= host_load(abort_flag_at(z, state.seg[index / per_rank], index % per_rank));
        if (wave == 0 && tag > 1 && lane < ranks && lane != state.local_rank) consumed_word = host_load(signal_at(own, z.counts_consumed_offset, lane));
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
    if (!state.reuse_plan && chunk < chunks) {
        for (int i = threadIdx.x; i < bins * chunk_waves; i += blockDim.x) masks[i] = 0;
        for (int i = threadIdx.x; i < channels * ranks; i += blockDim.x) chan_counts[i] = 0;
        for (int i = threadIdx.x; i < channels; i += blockDim.x) chan_remote[i] = 0;
        for (int i = threadIdx.x; i < channels * domains; i += blockDim.x) chan_relay[i] = 0;
        if (threadIdx.x == 0) *first_error = 0x7FFFFFFF;
        __syncthreads();
        const int tokens = state.num_tokens;
        const int token = (chunk * chunk_waves + wave) * kWave + lane;
        const bool participant = wave < chunk_waves;
        const bool live = participant && token < tokens;
        const int channel = token % channels;
        // All route ids of the token in registers, loaded back to back.
        int64_t raw[kTopk];
        int expert[kTopk];
#pragma unroll
        for (int branch = 0; branch < kTopk; ++branch) raw[branch] = (live && branch < topk) ? state.topk_idx[size_t(token) * topk + branch] : -1;
        uint32_t destination_mask = 0;
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
        __syncthreads();
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
        // Base of this chunk: totals of every earlier chunk.
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
        if (!stalled) {
            for (int bin = threadIdx.x; bin < bins; bin += blockDim.x) {
                int sum = 0;
                for (int earlier = 0; earlier < chunk; ++earlier)
                    sum += device_load(chunk_records + size_t(earlier) * record.stride() + record.counts() + bin);
                base[bin] = sum;
            }
        }
        __syncthreads();
        if (live && !stalled) {
            const uint64_t below = lanes_below(lane);
            state.plan_mask[token] = destination_mask;
            for (int rank = 0; rank < ranks; ++rank) {
                int ordinal = -1;
                const size_t at = size_t(wave) * bins + rank;
                if ((destination_mask >> rank) & 1u) ordinal = base[rank] + prefix[at] + __popcll(masks[at] & below);
                state.plan_rank_ord[size_t(token) * ranks + rank] = ordinal;
            }
#pragma unroll
            for (int branch = 0; branch < kTopk; ++branch) {
                if (branch < topk) {
                    int ordinal = -1;
                    if (expert[branch] >= 0) {
                        const size_t at = size_t(wave) * bins + ranks + expert[branch];
                        ordinal = base[ranks + expert[branch]] + prefix[at] + __popcll(masks[at] & below);
                    }
                    state.plan_exp_idx[size_t(token) * topk + branch] = expert[branch];
                    state.plan_exp_ord[size_t(token) * topk + branch] = ordinal;
                }
            }
        }
    }
    if (!leader) return;
    PCIE_EP_PROFILE(profile.first(kPrologueLayoutNs);)

    // ---- leader: totals of the whole plan ------------------------------------------------
    if (!state.reuse_plan) {
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
            const int fields = record.error_key();  // counts, channel counts, channel remote tokens, relay counts
            for (int field = threadIdx.x; field < fields; field += blockDim.x) {
                int sum = 0;
                for (int other = 0; other < chunks; ++other) sum += device_load(chunk_records + size_t(other) * record.stride() + field);
                if (field < bins) state.plan_counts[field] = sum;
                else if (field < record.chan_remote()) state.plan_chan_counts[field - record.chan_counts()] = sum;
                else if (field < record.chan_relay()) state.plan_chan_remote[field - record.chan_remote()] = sum;
                else state.plan_chan_relay[field - record.chan_relay()] = sum;
            }
            if (threadIdx.x == 0) {
                int key = 0x7FFFFFFF;
                for (int other = 0; other < chunks; ++other) {
                    const int candidate = device_load(chunk_records + size_t(other) * record.stride() + record.error_key());
                    key = candidate < key ? candidate : key;
                }
                if (key != 0x7FFFFFFF) record_error(state, kErrInvalidRouting, key / 64, key % 64);
            }
        }
    }

    PCIE_EP_PROFILE(profile.first(kPrologueTotalsNs);)
    // ---- epoch verdict -----------------------------------------------------------------
    // Everything the leader's threads hand to each other below (plan totals, the
    // error record) stays inside this workgroup: the barriers order it, no cache
    // write-back is needed before the kernel ends.
    bool aborted = false;
#pragma unroll
    for (int i = 0; i < kAbortLoadsPerThread; ++i) aborted |= abort_words[i] != 0;
    bool consumed = consumed_word == tag - 1;
    const bool any_abort = __syncthreads_or(aborted);
    PCIE_EP_PROFILE(profile.first(kPrologueVerdictNs);)
    if (threadIdx.x == 0) {
        *state.epoch = tag;
        if (tag >= 0x100000000ull) record_error(state, kErrEpochExhausted);
        else if (stalled) record_error(state, kErrRingProgressWait);
        else if (any_abort) record_error(state, kErrAlreadyAborted);
        // Any error here (including invalid routing found above) is terminal for this buffer.
        if (load_error_code(state)) host_store_release(signal_at(own, z.channel_abort_offset), tag);
    }
    __syncthreads();
    const uint64_t epoch = tag;
    __shared__ int mailbox_failed;
    if (threadIdx.x == 0) mailbox_failed = 0;
    __syncthreads();
    if (load_error_code(state)) {
        PCIE_EP_PROFILE(profile.save(state.profiling, profile_row, threadIdx.x);)
        return;
    }

    // ---- previous count mailbox must be consumed by every peer --------------------------
    // (advanced_layout.cuh:60-88): only then may the counts be overwritten.
    if (wave == 0 && epoch > 1) {
        HealthCheck health(state, now_ticks());
        while (!__all(consumed)) {
            if (health.poll(state, lane)) {
                if (lane == 0) {
                    record_error(state, kErrCountsMailboxWait);
                    host_store_release(signal_at(own, z.channel_abort_offset), epoch);
                    mailbox_failed = 1;
                }
                break;
            }
            backoff();
            if (!consumed) consumed = host_load(signal_at(own, z.counts_consumed_offset, lane)) == epoch - 1;
        }
    }
    __syncthreads();
    PCIE_EP_PROFILE(profile.first(kPrologueMailboxFreeNs);)
    if (mailbox_failed) {
        PCIE_EP_PROFILE(profile.save(state.profiling, profile_row, threadIdx.x);)
        return;
    }
    // Transmit tickets of this dispatch: every own token with a remote destination.
    if (threadIdx.x == 0) {
        int remote_tokens = 0;
        for (int channel = 0; channel < channels; ++channel) remote_tokens += state.plan_chan_remote[channel];
        state.queues->tx_head.total = remote_tokens;
    }
    publish_counts(state, epoch PCIE_EP_PROFILE(, profile));
    PCIE_EP_PROFILE(profile.save(state.profiling, profile_row, threadIdx.x);)
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

int prologue_chunks(const SegmentLayout& z, int tokens) {
    const int chunk_tokens = prologue_chunk_waves(z) * kWave;
    return (tokens + chunk_tokens - 1) / chunk_tokens;
}

size_t prologue_flag_bytes(const SegmentLayout& z) { return align_up(size_t(prologue_chunks(z, z.dims.max_tokens)) * 8, 256); }

size_t prologue_scratch_bytes(const SegmentLayout& z) {
    const ChunkRecord record{z.dims.num_ranks + z.dims.num_experts, z.dims.channels, z.dims.num_ranks, z.dims.domains};
    return prologue_flag_bytes(z) + size_t(prologue_chunks(z, z.dims.max_tokens)) * record.stride() * 4;
}

hipError_t launch_prologue(const DeviceState& state, hipStream_t stream) {
    const int waves = prologue_chunk_waves(state.z);
    const size_t bytes = prologue_lds_bytes(state.z, waves);
    const bool narrow = state.z.dims.topk <= 8;
    if (bytes > 64 * 1024) return hipErrorInvalidValue;  // cannot happen within the supported dimensions
    // At least 256 threads so the clear / publish loops stay short.
    const int threads = waves * kWave < 256 ? 256 : waves * kWave;
    if (threads > kPrologueMaxThreads) return hipErrorInvalidValue;
    const int chunks = state.reuse_plan ? 0 : prologue_chunks(state.z, state.num_tokens);
    const dim3 grid(chunks > 1 ? chunks : 1);
    if (narrow) hipLaunchKernelGGL(prologue_kernel<8>, grid, dim3(threads), bytes, stream, state, waves, chunks);
    else hipLaunchKernelGGL(prologue_kernel<kMaxTopk>, grid, dim3(threads), bytes, stream, state, waves, chunks);
    return hipGetLastError();
}

}  // namespace pcie_ep

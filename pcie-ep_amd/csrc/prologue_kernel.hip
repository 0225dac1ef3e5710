// Prologue kernel: epoch begin, route validation, stable layout and count
// publication, fused into one single-workgroup launch.
//
// Replaces five launches of the reference's eager dispatch
// (csrc/buffers/advanced.hpp:472-486): advanced_begin_epoch
// (advanced_layout.cuh:9-89), advanced_route_flags (:287-309),
// advanced_stable_ordinals (:311-356), advanced_prepare_channels_parallel
// (:358-425) and publish_counts (layout.cuh:7-29).
//
// Layout method (wave64): tokens are processed in chunks of W wavefronts.  For
// every bin (P destination ranks, then E experts) and every wavefront of the
// chunk a 64-bit hit mask is built in LDS (rank bins from ballots, expert bins
// with one LDS OR per branch).  A thread per bin then turns the W popcounts
// into exclusive prefixes on top of the running total, and every token reads
// back `prefix[bin][wave] + popcount(mask[bin][wave] & lanes_below)` — its
// stable ordinal.  Work is O(T*K), not O((P+E)*T*K), and bit-identical to a
// serial scan because ordinals only depend on which earlier tokens hit a bin.
#include "device_common.h"
#include "launch.h"

namespace pcie_ep {

namespace {

__device__ void publish_counts(const DeviceState& state, uint64_t epoch) {
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
        mailbox_at(z, own, destination)[field] = value;
    }
    // Every writer fences its own stores; the leader publishes after the join
    // (a leader-only fence would not cover the other writers: layout.cuh:21-28).
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) store_release_system(signal_at(own, z.counts_ready_offset), epoch);
}

}  // namespace

__global__ void __launch_bounds__(1024) prologue_kernel(DeviceState state, int chunk_waves) {
    extern __shared__ __align__(16) unsigned char lds[];
    const SegmentLayout& z = state.z;
    const int ranks = z.dims.num_ranks, experts = z.dims.num_experts, topk = z.dims.topk;
    const int channels = z.dims.channels, local = z.local_experts;
    const int bins = ranks + experts;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    char* own = state.seg[state.local_rank];

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
    {
        TransportQueues& q = *state.queues;
        QueueCounter* globals[] = {&q.rx_tail, &q.tx_tail, &q.rx_head, &q.tx_head, &q.abort};
        if (threadIdx.x < 5) {
            globals[threadIdx.x]->value = 0;
            globals[threadIdx.x]->total = -1;
        }
        for (int i = threadIdx.x; i < channels; i += blockDim.x) {
            q.rx_retired[i].value = q.tx_retired[i].value = q.rx_finished[i].value = 0;
            q.rx_retired[i].total = q.tx_retired[i].total = q.rx_finished[i].total = -1;
        }
    }

    // Abort signals are terminal.  Issue the loads now; the verdict is taken
    // after the layout so their PCIe latency hides behind it.
    bool aborted = false;
    {
        const int per_rank = 1 + channels;
        for (int index = threadIdx.x; index < ranks * per_rank; index += blockDim.x) {
            char* segment = state.seg[index / per_rank];
            const int flag = index % per_rank;
            const uint64_t* signal = flag == 0 ? signal_at(segment, z.abort_offset) : signal_at(segment, z.channel_abort_offset, flag - 1);
            aborted |= load_acquire_system(signal) != 0;
        }
    }
    __syncthreads();  // diagnostics are clear before anyone can record an error

    // ---- stable layout ---------------------------------------------------------------
    if (!state.reuse_plan) {
        uint64_t* masks = reinterpret_cast<uint64_t*>(lds);                       // [bins][W]
        int* prefix = reinterpret_cast<int*>(masks + size_t(bins) * chunk_waves);  // [bins][W]
        int* base = prefix + size_t(bins) * chunk_waves;                           // [bins]
        int* chan_counts = base + bins;                                            // [C][P]
        int* chan_remote = chan_counts + channels * ranks;                         // [C]
        for (int i = threadIdx.x; i < bins; i += blockDim.x) base[i] = 0;
        for (int i = threadIdx.x; i < channels * ranks; i += blockDim.x) chan_counts[i] = 0;
        for (int i = threadIdx.x; i < channels; i += blockDim.x) chan_remote[i] = 0;
        const int tokens = state.num_tokens;
        const int chunk_tokens = chunk_waves * kWave;
        const bool participant = wave < chunk_waves;
        for (int begin = 0; begin < tokens; begin += chunk_tokens) {
            for (int i = threadIdx.x; i < bins * chunk_waves; i += blockDim.x) masks[i] = 0;
            __syncthreads();
            const int token = begin + wave * kWave + lane;
            const bool live = participant && token < tokens;
            uint32_t destination_mask = 0;
#pragma unroll 4
            for (int branch = 0; branch < kMaxTopk; ++branch) {
                if (branch >= topk) break;
                int expert = -1;
                if (live) {
                    // Invalid: < -1, >= E, or equal to an earlier id of the same
                    // token (advanced_layout.cuh:296-307).  -1 is a legal skip.
                    const int64_t raw = state.topk_idx[size_t(token) * topk + branch];
                    bool invalid = raw < -1 || raw >= experts;
                    for (int previous = 0; previous < branch; ++previous)
                        invalid |= raw >= 0 && raw == state.topk_idx[size_t(token) * topk + previous];
                    if (invalid) record_error(state, kErrInvalidRouting, token, branch);
                    else expert = int(raw);
                    state.plan_exp_idx[size_t(token) * topk + branch] = expert;
                    if (expert >= 0) {
                        destination_mask |= 1u << (expert / local);
                        atomicOr(reinterpret_cast<unsigned long long*>(masks + size_t(ranks + expert) * chunk_waves + wave), 1ull << lane);
                    }
                }
            }
            if (participant) {
                for (int rank = 0; rank < ranks; ++rank) {
                    const uint64_t hits = __ballot((destination_mask >> rank) & 1u);
                    if (lane == 0) masks[size_t(rank) * chunk_waves + wave] = hits;
                }
            }
            __syncthreads();
            for (int bin = threadIdx.x; bin < bins; bin += blockDim.x) {
                int running = base[bin];
                for (int w = 0; w < chunk_waves; ++w) {
                    prefix[size_t(bin) * chunk_waves + w] = running;
                    running += __popcll(masks[size_t(bin) * chunk_waves + w]);
                }
                base[bin] = running;
            }
            __syncthreads();
            if (live) {
                const uint64_t below = lanes_below(lane);
                state.plan_mask[token] = destination_mask;
                for (int rank = 0; rank < ranks; ++rank) {
                    int ordinal = -1;
                    if ((destination_mask >> rank) & 1u)
                        ordinal = prefix[size_t(rank) * chunk_waves + wave] + __popcll(masks[size_t(rank) * chunk_waves + wave] & below);
                    state.plan_rank_ord[size_t(token) * ranks + rank] = ordinal;
                }
#pragma unroll 4
                for (int branch = 0; branch < kMaxTopk; ++branch) {
                    if (branch >= topk) break;
                    const int expert = state.plan_exp_idx[size_t(token) * topk + branch];
                    int ordinal = -1;
                    if (expert >= 0) {
                        const size_t at = size_t(ranks + expert) * chunk_waves + wave;
                        ordinal = prefix[at] + __popcll(masks[at] & below);
                    }
                    state.plan_exp_ord[size_t(token) * topk + branch] = ordinal;
                }
                // Channel c owns tokens c, c + C, ...; counts include the own rank
                // (advanced_layout.cuh:385-412).
                const int channel = token % channels;
                for (int rank = 0; rank < ranks; ++rank)
                    if ((destination_mask >> rank) & 1u) atomicAdd(chan_counts + channel * ranks + rank, 1);
                if (destination_mask & ~(1u << state.local_rank)) atomicAdd(chan_remote + channel, 1);
            }
            __syncthreads();
        }
        for (int i = threadIdx.x; i < bins; i += blockDim.x) state.plan_counts[i] = base[i];
        for (int i = threadIdx.x; i < channels * ranks; i += blockDim.x) state.plan_chan_counts[i] = chan_counts[i];
        for (int i = threadIdx.x; i < channels; i += blockDim.x) state.plan_chan_remote[i] = chan_remote[i];
        __threadfence();
    }

    // ---- epoch verdict -----------------------------------------------------------------
    const bool any_abort = __syncthreads_or(aborted);
    if (threadIdx.x == 0) {
        const uint64_t epoch = *state.epoch + 1;
        *state.epoch = epoch;
        if (epoch >= 0x100000000ull) {
            record_error(state, kErrEpochExhausted);
            store_release_system(signal_at(own, z.channel_abort_offset), epoch);
        } else if (any_abort) {
            record_error(state, kErrAlreadyAborted);
            store_release_system(signal_at(own, z.channel_abort_offset), epoch);
        } else if (load_error_code(state)) {
            // Invalid routing found above: terminal for this buffer.
            store_release_system(signal_at(own, z.channel_abort_offset), epoch);
        }
        __threadfence();
    }
    __syncthreads();
    const uint64_t epoch = *state.epoch;
    __shared__ int mailbox_failed;
    if (threadIdx.x == 0) mailbox_failed = 0;
    __syncthreads();
    if (load_error_code(state)) return;

    // ---- previous count mailbox must be consumed by every peer --------------------------
    // (advanced_layout.cuh:60-88): only then may the counts be overwritten.
    if (wave == 0 && epoch > 1) {
        bool consumed = lane >= ranks || lane == state.local_rank;
        HealthCheck health(state, now_ticks());
        while (true) {
            if (!consumed)
                consumed = load_acquire_system(signal_at(own, z.counts_consumed_offset, lane)) == epoch - 1;
            if (__all(consumed)) break;
            if (health.poll(state, lane)) {
                if (lane == 0) {
                    record_error(state, kErrCountsMailboxWait);
                    store_release_system(signal_at(own, z.channel_abort_offset), epoch);
                    mailbox_failed = 1;
                }
                break;
            }
            backoff();
        }
    }
    __syncthreads();
    if (mailbox_failed) return;
    // Transmit tickets of this dispatch: every own token with a remote destination.
    if (threadIdx.x == 0) {
        int remote_tokens = 0;
        for (int channel = 0; channel < channels; ++channel) remote_tokens += state.plan_chan_remote[channel];
        state.queues->tx_head.total = remote_tokens;
    }
    publish_counts(state, epoch);
}

size_t prologue_lds_bytes(const SegmentLayout& z, int chunk_waves) {
    const size_t bins = size_t(z.dims.num_ranks) + z.dims.num_experts;
    return bins * chunk_waves * 12 + bins * 4 + size_t(z.dims.channels) * z.dims.num_ranks * 4 + size_t(z.dims.channels) * 4 + 64;
}

int prologue_chunk_waves(const SegmentLayout& z) {
    int waves = 16;
    while (waves > 1 && prologue_lds_bytes(z, waves) > 144 * 1024) waves /= 2;
    return waves;
}

hipError_t launch_prologue(const DeviceState& state, hipStream_t stream) {
    const int waves = prologue_chunk_waves(state.z);
    const size_t bytes = prologue_lds_bytes(state.z, waves);
    static bool raised = false;
    if (!raised && bytes > 64 * 1024) {
        hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(prologue_kernel),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (status != hipSuccess) return status;
        raised = true;
    }
    // At least 256 threads so the clear / publish loops stay short.
    const int threads = waves * kWave < 256 ? 256 : waves * kWave;
    hipLaunchKernelGGL(prologue_kernel, dim3(1), dim3(threads), bytes, stream, state, waves);
    return hipGetLastError();
}

}  // namespace pcie_ep

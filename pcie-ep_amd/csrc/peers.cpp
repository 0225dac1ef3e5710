// Host peer emulator (see peers.h).  Plain C++20: no GPU call is made here; the
// segments are pinned host memory the GPU maps.
#include "peers.h"

#include <algorithm>
#include <chrono>
#include <cstring>

#include "fp8.h"

#if defined(__x86_64__)
#include <emmintrin.h>
#endif

namespace pcie_ep {

namespace {

inline uint64_t acquire(uint64_t* address) { return std::atomic_ref<uint64_t>(*address).load(std::memory_order_acquire); }
inline void release(uint64_t* address, uint64_t value) { std::atomic_ref<uint64_t>(*address).store(value, std::memory_order_release); }
inline double now_seconds() {
    return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
// Staging copy of an emulated source.  A real peer is another GPU whose rows reach
// this memory as DMA writes: they land in memory (or the shared last-level cache),
// never in a core's private cache.  A plain memcpy would leave the rows modified in
// the staging core's cache, and every read of the receiving GPU would first have to
// be snooped out of that core - the emulator would then decide how fast small
// dispatches run.  Streaming (non-temporal) stores put the rows where a device
// would, and the fence orders them before the descriptor's release store.
inline void stage_bytes(char* destination, const void* source, size_t bytes) {
#if defined(__x86_64__)
    if (reinterpret_cast<uintptr_t>(destination) % 16 == 0 && bytes % 16 == 0) {
        const char* from = static_cast<const char*>(source);
        for (size_t at = 0; at < bytes; at += 16)
            _mm_stream_si128(reinterpret_cast<__m128i*>(destination + at), _mm_loadu_si128(reinterpret_cast<const __m128i*>(from + at)));
        _mm_sfence();
        return;
    }
#endif
    std::memcpy(destination, source, bytes);
}

inline void cpu_relax() {
#if defined(__x86_64__)
    __builtin_ia32_pause();
#endif
}

}  // namespace

int host_source_layout(const int64_t* topk_idx, int tokens, int topk, int num_ranks, int num_experts, uint32_t* mask,
                       int32_t* rank_ordinals, int32_t* expert_indices, int32_t* expert_ordinals, int32_t* counts) {
    // Serial form of the reference's route validation and stable ordinals
    // (csrc/kernels/host_staged/advanced_layout.cuh:287-356).
    const int local = num_experts / num_ranks;
    std::fill(counts, counts + num_ranks + num_experts, 0);
    int error = 0;
    for (int token = 0; token < tokens; ++token) {
        uint32_t destinations = 0;
        for (int branch = 0; branch < topk; ++branch) {
            const int64_t raw = topk_idx[size_t(token) * topk + branch];
            bool invalid = raw < -1 || raw >= num_experts;
            for (int previous = 0; previous < branch; ++previous)
                invalid |= raw >= 0 && raw == topk_idx[size_t(token) * topk + previous];
            if (invalid) error = kErrInvalidRouting;
            const int expert = invalid ? -1 : int(raw);
            expert_indices[size_t(token) * topk + branch] = expert;
            if (expert >= 0) destinations |= 1u << (expert / local);
        }
        mask[token] = destinations;
        for (int rank = 0; rank < num_ranks; ++rank)
            rank_ordinals[size_t(token) * num_ranks + rank] = (destinations >> rank) & 1u ? counts[rank]++ : -1;
        for (int branch = 0; branch < topk; ++branch) {
            const int expert = expert_indices[size_t(token) * topk + branch];
            expert_ordinals[size_t(token) * topk + branch] = expert >= 0 ? counts[num_ranks + expert]++ : -1;
        }
    }
    return error;
}

void host_quantize_fp8(const uint16_t* x, uint8_t* codes, float* scales, int tokens, int hidden) {
    for (int token = 0; token < tokens; ++token) {
        const uint16_t* row = x + size_t(token) * hidden;
        float amax = 0.0f;
        for (int i = 0; i < hidden; ++i) {
            const float magnitude = bits_float((uint32_t(row[i]) << 16) & 0x7FFFFFFFu);
            amax = magnitude > amax ? magnitude : amax;
        }
        const float scale = fp8_scale_from_amax(amax);
        const float inverse = 1.0f / scale;
        for (int i = 0; i < hidden; ++i) codes[size_t(token) * hidden + i] = fp8_quantize_element(row[i], inverse);
        scales[token] = scale;
    }
}

void host_dequantize_fp8(const uint8_t* codes, const float* scales, uint16_t* out, int tokens, int hidden) {
    for (int token = 0; token < tokens; ++token)
        for (int i = 0; i < hidden; ++i)
            out[size_t(token) * hidden + i] = fp8_dequantize_element(codes[size_t(token) * hidden + i], scales[token]);
}

PeerEmulator::PeerEmulator(const SegmentLayout& layout, int local_rank, char* const* segments, char* const* replica, int threads,
                           int timeout_ms, const RelayOptions& relay)
    : z_(layout), me_(local_rank), timeout_ms_(timeout_ms), ranks_(layout.dims.num_ranks) {
    for (int rank = 0; rank < kMaxRanks; ++rank) seg_[rank] = rank < z_.dims.num_ranks ? segments[rank] : nullptr;
    for (int rank = 0; rank < z_.dims.num_ranks; ++rank)
        for (int domain = 0; domain < z_.dims.domains; ++domain) replica_[rank][domain] = replica[rank * kMaxDomains + domain];
    if (z_.dims.domains) {
        // The relay workers an emulated source's own process would run.  Only the
        // GPU consumes what they publish: the other receivers are not simulated.
        RelayOptions options = relay;
        options.live_ranks = 1u << me_;
        options.workers_per_domain = 1;
        options.pin = false;
        for (int rank = 0; rank < z_.dims.num_ranks; ++rank)
            if (rank != me_) relays_.push_back(std::make_unique<NumaRelay>(z_, rank, seg_, replica_[rank], options));
    }
    const int channels = z_.dims.channels;
    for (auto& state : ranks_) {
        state.remote.resize(channels);
        state.channel_counts.assign(size_t(channels) * z_.dims.num_ranks, 0);
        state.counts.assign(size_t(z_.dims.num_ranks) + z_.dims.num_experts, 0);
        state.slot_generation.assign(size_t(channels) * z_.dims.payload_slots, 0);
        state.slot_token.assign(size_t(channels) * z_.dims.payload_slots, -1);
        state.pending_sequence.assign(size_t(channels) * z_.dims.payload_slots, 0);
        state.pending_listed.assign(size_t(channels) * z_.dims.payload_slots, 0);
        state.cursor.assign(channels, 0);
        state.sent.assign(channels, 0);
        state.expected.assign(channels, 0);
        state.consumed.assign(channels, 0);
    }
    // A rank's two roles share no state, so they may run on different threads:
    // the tasks are the peers' source roles followed by their receiver roles,
    // dealt round; up to one thread per peer a rank's roles meet on one thread.
    const int peers = z_.dims.num_ranks - 1;
    if (threads > 2 * peers) threads = 2 * peers;
    if (threads < 1) threads = 1;
    assignment_.resize(threads);
    int next = 0;
    for (int role : {kSourceRole, kReceiverRole})
        for (int rank = 0; rank < z_.dims.num_ranks; ++rank)
            if (rank != me_) assignment_[next++ % threads].push_back({rank, role});
    thread_done_.assign(threads, 0);
    for (int index = 0; index < threads; ++index) threads_.emplace_back([this, index] { thread_main(index); });
}

PeerEmulator::~PeerEmulator() {
    for (auto& relay : relays_) relay->stop_and_join();
    {
        std::lock_guard<std::mutex> lock(mutex_);
        stop_ = true;
        cancel_.store(true);
    }
    wake_.notify_all();
    for (auto& thread : threads_) thread.join();
}

void PeerEmulator::fail(const std::string& message) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (!failed_.exchange(true)) failure_ = message;
}

int PeerEmulator::set_source(int rank, const uint16_t* x, const int64_t* topk_idx, const float* weights, int tokens, std::string& error) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (rank < 0 || rank >= z_.dims.num_ranks || rank == me_) { error = "peer rank is out of range or is the GPU's own rank"; return -1; }
    if (tokens < 0 || tokens > z_.dims.max_tokens) { error = "peer token count exceeds the prepared capacity"; return -1; }
    if (served_ != target_) { error = "peer inputs cannot change while epochs are being served"; return -3; }
    Rank& state = ranks_[rank];
    const int topk = z_.dims.topk, ranks = z_.dims.num_ranks, hidden = z_.dims.hidden, channels = z_.dims.channels;
    state.tokens = tokens;
    state.x.assign(x, x + size_t(tokens) * hidden);
    state.has_weights = weights != nullptr;
    if (weights) state.weights.assign(weights, weights + size_t(tokens) * topk);
    else state.weights.assign(size_t(tokens) * topk, 1.0f);
    state.mask.assign(tokens, 0);
    state.rank_ordinals.assign(size_t(tokens) * ranks, -1);
    state.expert_indices.assign(size_t(tokens) * topk, -1);
    state.expert_ordinals.assign(size_t(tokens) * topk, -1);
    const int status = host_source_layout(topk_idx, tokens, topk, ranks, z_.dims.num_experts, state.mask.data(),
                                          state.rank_ordinals.data(), state.expert_indices.data(), state.expert_ordinals.data(),
                                          state.counts.data());
    if (status) { error = "peer routing is invalid (duplicate, < -1 or >= num_experts)"; return -1; }
    std::fill(state.channel_counts.begin(), state.channel_counts.end(), 0);
    for (auto& list : state.remote) list.clear();
    for (int token = 0; token < tokens; ++token) {
        const int channel = token % channels;
        for (int destination = 0; destination < ranks; ++destination)
            if ((state.mask[token] >> destination) & 1u) ++state.channel_counts[size_t(channel) * ranks + destination];
        if (state.mask[token] & ~(1u << rank)) state.remote[channel].push_back(token);
    }
    ++state.generation;
    return 0;
}

int PeerEmulator::start(int epochs, uint32_t flags, std::string& error) {
    {
        std::lock_guard<std::mutex> lock(mutex_);
        if (epochs < 1) { error = "epochs must be positive"; return -1; }
        if (failed_.load()) { error = "the peer emulator has failed: " + failure_; return -5; }
        if (served_ != target_) { error = "previous epochs are still being served"; return -3; }
        flags_ = flags;
        cancel_.store(false);
        target_ += uint64_t(epochs);
    }
    wake_.notify_all();
    return 0;
}

void PeerEmulator::cancel() {
    std::unique_lock<std::mutex> lock(mutex_);
    cancel_.store(true);
    finished_.wait(lock, [this] {
        for (uint64_t done : thread_done_) if (done != target_) return false;
        return true;
    });
    served_ = target_;
}

int PeerEmulator::inject_fault(int rank, int fault) {
    if (rank < 0 || rank >= z_.dims.num_ranks || rank == me_ || fault < 0 || fault > kFaultSlotOutOfRange) return -1;
    ranks_[rank].fault.store(fault);
    return 0;
}

int PeerEmulator::wait_staged(int timeout_ms, std::string& error) {
    const double deadline = now_seconds() + timeout_ms * 1e-3;
    uint64_t epoch;
    {
        std::lock_guard<std::mutex> lock(mutex_);
        if (served_ == target_) return 0;
        epoch = served_ + 1;
    }
    while (true) {
        bool staged = true;
        for (int rank = 0; rank < z_.dims.num_ranks; ++rank)
            if (rank != me_ && ranks_[rank].staged_epoch.load(std::memory_order_acquire) < epoch) staged = false;
        if (staged) return 0;
        if (failed_.load()) { std::lock_guard<std::mutex> lock(mutex_); error = failure_; return -5; }
        if (now_seconds() > deadline) { error = "timed out waiting for the peer sources to stage"; return -4; }
        std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
}

int PeerEmulator::wait(int timeout_ms, std::string& error) {
    std::unique_lock<std::mutex> lock(mutex_);
    // A deadline on the system clock: this form of the wait goes through
    // pthread_cond_timedwait, which thread-checking tools understand.
    const bool finished = finished_.wait_until(lock, std::chrono::system_clock::now() + std::chrono::milliseconds(timeout_ms), [this] {
        for (uint64_t done : thread_done_) if (done != target_) return false;
        return true;
    });
    if (!finished) { error = "timed out waiting for the peer emulator"; return -4; }
    served_ = target_;
    if (failed_.load()) { error = failure_; return -5; }
    return 0;
}

void PeerEmulator::thread_main(int index) {
    uint64_t done = 0;
    while (true) {
        {
            std::unique_lock<std::mutex> lock(mutex_);
            wake_.wait(lock, [&] { return stop_ || target_ > done; });
            if (stop_) return;
        }
        std::string error;
        const bool ok = !cancel_.load() && !failed_.load() && serve_epoch(index, done + 1, error);
        if (!ok && !error.empty()) fail(error);
        {
            std::lock_guard<std::mutex> lock(mutex_);
            // After a failure or a cancel the remaining epochs are abandoned.
            done = ok ? done + 1 : target_;
            thread_done_[index] = done;
        }
        finished_.notify_all();
    }
}

bool PeerEmulator::serve_epoch(int index, uint64_t epoch, std::string& error) {
    const auto& mine = assignment_[index];
    for (const Task& task : mine) {
        Rank& state = ranks_[task.rank];
        if (task.role == kSourceRole) {
            state.source_phase = 0;
            std::fill(state.cursor.begin(), state.cursor.end(), 0);
            std::fill(state.sent.begin(), state.sent.end(), 0);
            for (int slot_index : state.pending_slots) {
                state.pending_sequence[slot_index] = 0;
                state.pending_listed[slot_index] = 0;
            }
            state.pending_slots.clear();
            continue;
        }
        state.receiver_phase = 0;
        std::fill(state.consumed.begin(), state.consumed.end(), 0);
        state.receive_total = state.receive_done = 0;
        if (flags_ & kPeerCapture) {
            state.cap_tokens.clear(); state.cap_rank_ordinals.clear(); state.cap_expert_idx.clear();
            state.cap_expert_ordinals.clear(); state.cap_payload.clear(); state.cap_scales.clear();
            state.cap_weights.clear(); state.cap_masks.clear();
        }
    }
    std::vector<char> task_done(mine.size(), 0);
    double last_progress = now_seconds();
    while (true) {
        bool progressed = false, all_done = true;
        for (size_t i = 0; i < mine.size(); ++i) {
            if (task_done[i]) continue;
            const int rank = mine[i].rank;
            bool done = false;
            if (mine[i].role == kSourceRole) {
                bool quiescent = false;
                progressed |= source_progress(rank, epoch, done, quiescent, error);
                if (!error.empty()) return false;
                if (done || quiescent) {
                    uint64_t seen = ranks_[rank].staged_epoch.load(std::memory_order_relaxed);
                    if (seen < epoch) ranks_[rank].staged_epoch.store(epoch, std::memory_order_release);
                }
            } else {
                progressed |= receiver_progress(rank, epoch, done, error);
                if (!error.empty()) return false;
            }
            task_done[i] = done;
            all_done &= done;
        }
        if (all_done) return true;
        if (cancel_.load() || failed_.load()) return false;
        if (progressed) last_progress = now_seconds();
        else {
            if (now_seconds() - last_progress > timeout_ms_ * 1e-3) {
                std::string detail;
                for (size_t i = 0; i < mine.size(); ++i) {
                    const Rank& state = ranks_[mine[i].rank];
                    if (mine[i].role == kSourceRole)
                        detail += " rank " + std::to_string(mine[i].rank) + ": source phase " + std::to_string(state.source_phase) +
                                  (task_done[i] ? " done;" : ";");
                    else
                        detail += " rank " + std::to_string(mine[i].rank) + ": receiver phase " + std::to_string(state.receiver_phase) + " (" +
                                  std::to_string(state.receive_done) + "/" + std::to_string(state.receive_total) + ")" +
                                  (task_done[i] ? " done;" : ";");
                }
                error = "peer emulator made no progress for " + std::to_string(timeout_ms_) + " ms in epoch " + std::to_string(epoch) + ":" + detail;
                return false;
            }
            cpu_relax();
        }
    }
}

void PeerEmulator::publish_token(Rank& state, int rank, uint64_t epoch, int channel, int token, int slot, int ordinal, int fault) {
    const int topk = z_.dims.topk, ranks = z_.dims.num_ranks, hidden = z_.dims.hidden;
    char* own = seg_[rank];
    char* base = slot_at(z_, own, channel, slot);
    const size_t slot_index = size_t(channel) * z_.dims.payload_slots + slot;
    const bool falsify = fault == kFaultRankOrdinalOutOfRange || fault == kFaultExpertOrdinalOutOfRange;
    // Rows that did not change since the slot was last written are left in place
    // unless the caller asked for every epoch to be staged afresh.
    if ((flags_ & kPeerRestage) || falsify || state.slot_generation[slot_index] != state.generation || state.slot_token[slot_index] != token) {
        float scale = 1.0f;
        const uint16_t* row = state.x.data() + size_t(token) * hidden;
        if (z_.dims.wire_fp8) {
            std::vector<uint8_t>& codes = state.stage_codes;
            codes.resize((size_t(hidden) + 15) / 16 * 16);
            host_quantize_fp8(row, codes.data(), &scale, 1, hidden);
            if (hidden % 16 == 0) stage_bytes(base, codes.data(), size_t(hidden));
            else std::memcpy(base, codes.data(), size_t(hidden));
        } else {
            stage_bytes(base, row, size_t(hidden) * 2);
        }
        // The slot metadata is composed on the side and staged the same way.
        alignas(16) char meta[kMetaBranchOffset + 12 * kMaxTopk + 16] = {};
        SlotMetaHeader header{};
        header.token_index = token;
        header.destination_mask = state.mask[token];
        header.scale = scale;
        std::memcpy(meta, &header, sizeof header);
        int32_t* rank_ordinals = reinterpret_cast<int32_t*>(meta + kMetaRankOrdinalsOffset);
        for (int r = 0; r < kMaxRanks; ++r) rank_ordinals[r] = r < ranks ? state.rank_ordinals[size_t(token) * ranks + r] : -1;
        int32_t* branch = reinterpret_cast<int32_t*>(meta + kMetaBranchOffset);
        std::memcpy(branch, state.expert_indices.data() + size_t(token) * topk, size_t(topk) * 4);
        std::memcpy(branch + topk, state.expert_ordinals.data() + size_t(token) * topk, size_t(topk) * 4);
        std::memcpy(branch + 2 * topk, state.weights.data() + size_t(token) * topk, size_t(topk) * 4);
        state.slot_generation[slot_index] = state.generation;
        state.slot_token[slot_index] = token;
        if (falsify) {
            // Fault hooks: an ordinal outside the counts this source announced.
            if (fault == kFaultRankOrdinalOutOfRange) rank_ordinals[me_] = state.counts[me_];
            else
                for (int k = 0; k < topk; ++k)
                    if (branch[k] >= 0 && branch[k] / z_.local_experts == me_) branch[topk + k] = 1 << 20;
            state.slot_token[slot_index] = -1;  // stage the true row again next time
        }
        stage_bytes(base + z_.meta_offset, meta, size_t(z_.meta_bytes));
    }
    Descriptor* descriptor = descriptor_at(z_, own, channel, endpoint_of(z_.dims, rank, me_), ordinal);
    descriptor->payload_slot = fault == kFaultSlotOutOfRange ? z_.dims.payload_slots : slot;
    // The token identifies the payload (its sequence is sequence(epoch, token));
    // the fault hook publishes a token that does not match the slot's metadata.
    descriptor->token_index = fault == kFaultWrongPayloadSequence ? token + 1 : token;
    release(&descriptor->ready, sequence(epoch, ordinal));
    state.pending_sequence[slot_index] = sequence(epoch, token);
    if (!state.pending_listed[slot_index]) {
        state.pending_listed[slot_index] = 1;
        state.pending_slots.push_back(int(slot_index));
    }
}

// Source role of rank `rank`: feed the GPU's receive side.
bool PeerEmulator::source_progress(int rank, uint64_t epoch, bool& done, bool& quiescent, std::string& error) {
    Rank& state = ranks_[rank];
    char* own = seg_[rank];
    const int channels = z_.dims.channels, ranks = z_.dims.num_ranks, local = z_.local_experts;
    const int slots = z_.dims.payload_slots, descriptors = z_.dims.descriptor_slots;
    const int fault = state.fault.load(std::memory_order_relaxed);
    bool progressed = false;
    if (state.source_phase == 0) {
        // The GPU must have consumed the previous mailbox before it is rewritten
        // (advanced_layout.cuh:60-88 from the source's point of view).
        if (epoch > 1 && acquire(signal_at(own, z_.counts_consumed_offset, me_)) != epoch - 1) { quiescent = true; return false; }
        // ... and so must this source's relay flows have (advanced_dispatch.cuh:213-225).
        if (epoch > 1 && !relays_drained(rank, epoch - 1)) { quiescent = true; return false; }
        // Relay mode: rows for the GPU travel through the relay endpoint of the
        // GPU's domain when this source sits in another one.
        for (int domain = 0; domain < z_.dims.domains; ++domain) {
            const bool carries = reads_replica(z_.dims, rank, me_) && domain == z_.dims.rank_domain[me_];
            for (int channel = 0; channel < channels; ++channel)
                relay_mailbox_at(z_, own, domain)[channel] = carries ? state.channel_counts[size_t(channel) * ranks + me_] : 0;
        }
        for (int destination = 0; destination < ranks; ++destination) {
            int32_t* block = mailbox_at(z_, own, destination);
            block[0] = state.counts[destination];
            for (int expert = 0; expert < local; ++expert) block[1 + expert] = state.counts[ranks + destination * local + expert];
            for (int channel = 0; channel < channels; ++channel)
                block[1 + local + channel] = state.channel_counts[size_t(channel) * ranks + destination];
        }
        if (fault != kFaultWithholdCountsReady) release(signal_at(own, z_.counts_ready_offset), epoch);
        state.source_phase = 1;
        progressed = true;
    }
    const int endpoint = endpoint_of(z_.dims, rank, me_);
    if (state.source_phase == 1) {
        bool all_published = true;
        for (int channel = 0; channel < channels; ++channel) {
            const auto& list = state.remote[channel];
            int& cursor = state.cursor[channel];
            while (cursor < int(list.size())) {
                const int token = list[cursor];
                if ((state.mask[token] >> me_) & 1u) {
                    const int slot = cursor % slots;
                    // The slot may be rewritten only after the GPU ACKed the last row
                    // that was published to it here.  Occupants bound for other
                    // emulated ranks are never written, so the previous ring
                    // occupant is not necessarily the one whose ACK matters.
                    const size_t slot_index = size_t(channel) * slots + slot;
                    if (state.pending_sequence[slot_index]) {
                        if (acquire(ack_at(z_, own, channel, slot, endpoint)) != state.pending_sequence[slot_index]) break;
                        state.pending_sequence[slot_index] = 0;
                    }
                    const int ordinal = state.sent[channel];
                    if (!credit_covers(acquire(credit_at(z_, own, channel, endpoint)), epoch, ordinal, descriptors)) break;
                    // Row faults apply to the last row this source sends to the GPU on the channel.
                    const bool last = state.sent[channel] + 1 == state.channel_counts[size_t(channel) * ranks + me_];
                    publish_token(state, rank, epoch, channel, token, slot, ordinal, last ? fault : kFaultNone);
                    ++state.sent[channel];
                }
                // Tokens bound only for other emulated ranks need no transfer here:
                // those receivers are not simulated, their ACKs count as immediate.
                ++cursor;
                progressed = true;
            }
            all_published &= cursor == int(list.size());
        }
        if (all_published) state.source_phase = 2;
        else if (!progressed) quiescent = true;
    }
    if (state.source_phase == 2) {
        // Tail drain: every slot published to the GPU must be ACKed before the
        // next epoch may overwrite it (advanced_dispatch.cuh:229-285).
        quiescent = true;
        size_t kept = 0;
        for (int slot_index : state.pending_slots) {
            const uint64_t expected = state.pending_sequence[slot_index];
            if (expected && acquire(ack_at(z_, own, slot_index / z_.dims.payload_slots, slot_index % z_.dims.payload_slots, endpoint)) != expected) {
                state.pending_slots[kept++] = slot_index;
            } else {
                state.pending_sequence[slot_index] = 0;
                state.pending_listed[slot_index] = 0;
                progressed = true;
            }
        }
        state.pending_slots.resize(kept);
        // The epoch is over for this source once its relay flows are drained too.
        if (state.pending_slots.empty() && relays_drained(rank, epoch)) {
            state.source_phase = 3;
            done = true;
        }
    }
    if (state.source_phase == 3) done = true;
    (void)error;
    return progressed;
}

// Receiver role of rank `rank`: absorb the GPU's transmit side.
bool PeerEmulator::receiver_progress(int rank, uint64_t epoch, bool& done, std::string& error) {
    Rank& state = ranks_[rank];
    char* gpu = seg_[me_];
    const int channels = z_.dims.channels, local = z_.local_experts, topk = z_.dims.topk;
    const int fault = state.fault.load(std::memory_order_relaxed);
    const bool replica = reads_replica(z_.dims, me_, rank);
    const int domain = z_.dims.domains ? z_.dims.rank_domain[rank] : 0;
    bool progressed = false;
    if (state.receiver_phase == 0) {
        if (acquire(signal_at(gpu, z_.counts_ready_offset)) != epoch) return false;
        const int32_t* block = mailbox_at(z_, gpu, rank);
        state.receive_total = 0;
        for (int channel = 0; channel < channels; ++channel) {
            state.expected[channel] = block[1 + local + channel];
            state.receive_total += state.expected[channel];
        }
        if (state.receive_total != block[0]) {
            error = "GPU mailbox is inconsistent for rank " + std::to_string(rank) + ": channel counts sum to " +
                    std::to_string(state.receive_total) + " but the unique count is " + std::to_string(block[0]);
            return false;
        }
        std::atomic_thread_fence(std::memory_order_seq_cst);
        if (fault != kFaultWithholdCountsConsumed) release(signal_at(gpu, z_.counts_consumed_offset, rank), epoch);
        state.receiver_phase = 1;
        progressed = true;
    }
    if (state.receiver_phase == 1) {
        for (int channel = 0; channel < channels; ++channel) {
            while (state.consumed[channel] < state.expected[channel]) {
                const int ordinal = state.consumed[channel];
                // A receiver of another domain than the GPU's reads the replica ring
                // that the GPU's relay workers fill for its domain.
                Descriptor* descriptor = replica ? replica_descriptor_at(z_, gpu, channel, domain, rank, ordinal)
                                                 : descriptor_at(z_, gpu, channel, rank, ordinal);
                if (acquire(&descriptor->ready) != sequence(epoch, ordinal)) break;
                const int slot = descriptor->payload_slot, token = descriptor->token_index;
                const uint64_t payload_sequence = sequence(epoch, token);
                if (slot < 0 || slot >= (replica ? z_.dims.replica_slots : z_.dims.payload_slots) || token < 0 || token >= z_.dims.max_tokens) {
                    error = "GPU published a descriptor with an out-of-range slot or token";
                    return false;
                }
                const char* base = replica ? replica_slot_at(z_, replica_[me_][domain], channel, slot) : slot_at(z_, gpu, channel, slot);
                SlotMetaHeader header;
                std::memcpy(&header, base + z_.meta_offset, sizeof header);
                if (header.token_index != token) {
                    error = "GPU payload sequence does not match its slot metadata (rank " + std::to_string(rank) + ", channel " +
                            std::to_string(channel) + ", ordinal " + std::to_string(ordinal) + ")";
                    return false;
                }
                if (!((header.destination_mask >> rank) & 1u)) {
                    error = "GPU sent a token to a rank outside its destination mask";
                    return false;
                }
                if (flags_ & kPeerReadRows) {
                    const uint64_t* words = reinterpret_cast<const uint64_t*>(base);
                    uint64_t sum = 0;
                    for (int i = 0; i < z_.payload_bytes / 8; ++i) sum += words[i];
                    state.read_checksum += sum;
                }
                if (flags_ & kPeerCapture) {
                    const char* meta = base + z_.meta_offset;
                    const int32_t* branch = reinterpret_cast<const int32_t*>(meta + kMetaBranchOffset);
                    state.cap_tokens.push_back(token);
                    state.cap_rank_ordinals.push_back(reinterpret_cast<const int32_t*>(meta + kMetaRankOrdinalsOffset)[rank]);
                    state.cap_masks.push_back(header.destination_mask);
                    state.cap_scales.push_back(header.scale);
                    state.cap_payload.insert(state.cap_payload.end(), reinterpret_cast<const uint8_t*>(base),
                                             reinterpret_cast<const uint8_t*>(base) + z_.payload_bytes);
                    state.cap_expert_idx.insert(state.cap_expert_idx.end(), branch, branch + topk);
                    state.cap_expert_ordinals.insert(state.cap_expert_ordinals.end(), branch + topk, branch + 2 * topk);
                    const float* weights = reinterpret_cast<const float*>(branch + 2 * topk);
                    state.cap_weights.insert(state.cap_weights.end(), weights, weights + topk);
                }
                std::atomic_thread_fence(std::memory_order_seq_cst);
                const bool last = state.receive_done + 1 == state.receive_total;
                if (!(fault == kFaultWithholdLastAck && last))
                    release(replica ? replica_ack_at(z_, gpu, channel, domain, slot, rank) : ack_at(z_, gpu, channel, slot, rank), payload_sequence);
                release(replica ? replica_credit_at(z_, gpu, channel, domain, rank) : credit_at(z_, gpu, channel, rank), sequence(epoch, ordinal));
                ++state.consumed[channel];
                ++state.receive_done;
                progressed = true;
            }
        }
        if (state.receive_done == state.receive_total) {
            state.receiver_phase = 2;
            done = true;
        }
    }
    if (state.receiver_phase == 2) done = true;
    return progressed;
}

bool PeerEmulator::relays_drained(int rank, uint64_t epoch) const {
    for (int channel = 0; channel < z_.dims.channels; ++channel)
        for (int domain = 0; domain < z_.dims.domains; ++domain)
            if (acquire(signal_at(seg_[rank], z_.relay_drained_offset, flow_index(z_, channel, domain))) != epoch) return false;
    return true;
}

int64_t PeerEmulator::captured_count(int rank) {
    if (rank < 0 || rank >= z_.dims.num_ranks || rank == me_) return -1;
    std::lock_guard<std::mutex> lock(mutex_);
    return int64_t(ranks_[rank].cap_tokens.size());
}

int PeerEmulator::captured_copy(int rank, int32_t* tokens, int32_t* rank_ordinals, uint8_t* payload, float* scales, int32_t* expert_idx,
                                int32_t* expert_ordinals, float* weights, uint32_t* masks) {
    if (rank < 0 || rank >= z_.dims.num_ranks || rank == me_) return -1;
    std::lock_guard<std::mutex> lock(mutex_);
    const Rank& state = ranks_[rank];
    auto copy = [](auto* destination, const auto& source) {
        if (destination && !source.empty()) std::memcpy(destination, source.data(), source.size() * sizeof(source[0]));
    };
    copy(tokens, state.cap_tokens);
    copy(rank_ordinals, state.cap_rank_ordinals);
    copy(payload, state.cap_payload);
    copy(scales, state.cap_scales);
    copy(expert_idx, state.cap_expert_idx);
    copy(expert_ordinals, state.cap_expert_ordinals);
    copy(weights, state.cap_weights);
    copy(masks, state.cap_masks);
    return 0;
}

}  // namespace pcie_ep

// Host-side peer emulator: CPU threads that play the other logical ranks of the
// dispatch on the same pinned segments the GPU uses.
//
// The closest precedent in the reference for CPU code taking part in the ring
// protocol is its NUMA relay worker (csrc/comm/numa_relay.hpp:18-35 acquire/
// release helpers, :240-340 descriptor consume / ACK / credit).  The emulator
// follows the same discipline: every signal is read with an acquire load and
// written with a release store through std::atomic_ref, each signal has one
// writer, and a rank's progress step never blocks, so tiny rings cannot
// deadlock against the GPU.
#pragma once

#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "relay.h"
#include "wire.h"

namespace pcie_ep {

// Route plan of one source computed on the host.  Returns 0 or kErrInvalidRouting.
int host_source_layout(const int64_t* topk_idx, int tokens, int topk, int num_ranks, int num_experts, uint32_t* mask,
                       int32_t* rank_ordinals, int32_t* expert_indices, int32_t* expert_ordinals, int32_t* counts);
void host_quantize_fp8(const uint16_t* x, uint8_t* codes, float* scales, int tokens, int hidden);
void host_dequantize_fp8(const uint8_t* codes, const float* scales, uint16_t* out, int tokens, int hidden);

enum PeerFault : int {
    kFaultNone = 0,
    kFaultWithholdCountsReady = 1,
    kFaultWithholdCountsConsumed = 2,
    kFaultWithholdLastAck = 3,
    kFaultWrongPayloadSequence = 4,
    kFaultRankOrdinalOutOfRange = 5,    // last row: unique-row ordinal beyond the announced count
    kFaultExpertOrdinalOutOfRange = 6,  // last row: expert ordinal beyond the announced count
    kFaultSlotOutOfRange = 7,           // last row: the descriptor names a payload slot beyond the ring
};

// Flags of PeerEmulator::start.
enum PeerFlag : uint32_t {
    kPeerCapture = 1u,   // receivers keep a copy of every row the GPU sent
    kPeerRestage = 2u,   // sources rewrite payload and metadata of every slot in every epoch
    kPeerReadRows = 4u,  // receivers read every byte of the rows the GPU sent
};

class PeerEmulator {
public:
    // `replica[rank * kMaxDomains + domain]` is the replica payload region of
    // `rank` for `domain` (relay mode; unused otherwise).  In relay mode every
    // emulated source gets relay workers of its own, as its process would have.
    PeerEmulator(const SegmentLayout& layout, int local_rank, char* const* segments, char* const* replica, int threads, int timeout_ms,
                 const RelayOptions& relay);
    ~PeerEmulator();

    int set_source(int rank, const uint16_t* x, const int64_t* topk_idx, const float* weights, int tokens, std::string& error);
    int start(int epochs, uint32_t flags, std::string& error);
    int wait_staged(int timeout_ms, std::string& error);
    int wait(int timeout_ms, std::string& error);
    void cancel();
    int inject_fault(int rank, int fault);

    int64_t captured_count(int rank);
    int captured_copy(int rank, int32_t* tokens, int32_t* rank_ordinals, uint8_t* payload, float* scales, int32_t* expert_idx,
                      int32_t* expert_ordinals, float* weights, uint32_t* masks);

private:
    struct Rank {
        // Inputs and plan (guarded by `mutex_` while no epoch is being served).
        int tokens = 0;
        bool has_weights = false;
        uint64_t generation = 0;
        std::vector<uint16_t> x;
        std::vector<float> weights;
        std::vector<uint32_t> mask;
        std::vector<int32_t> rank_ordinals, expert_indices, expert_ordinals, counts;
        std::vector<std::vector<int>> remote;      // per channel: tokens with a remote destination, ascending
        std::vector<int> channel_counts;           // [C][P]
        std::vector<uint64_t> slot_generation;     // [C*Q]: generation whose bytes sit in the slot
        std::vector<int> slot_token;               // [C*Q]
        // Source flow of the epoch being served.
        int source_phase = 0;
        std::vector<int> cursor, sent;             // per channel
        std::vector<uint64_t> pending_sequence;    // [C*Q]: sequence published to the GPU whose ACK is outstanding, 0 = none
        std::vector<int> pending_slots;            // slot indices listed for the tail drain
        std::vector<char> pending_listed;          // [C*Q]
        // Receiver flow.
        int receiver_phase = 0;
        std::vector<int> expected, consumed;       // per channel
        int64_t receive_total = 0, receive_done = 0;
        // Captured rows of the last served epoch.
        std::vector<int32_t> cap_tokens, cap_rank_ordinals, cap_expert_idx, cap_expert_ordinals;
        std::vector<uint8_t> cap_payload;
        std::vector<float> cap_scales, cap_weights;
        std::vector<uint32_t> cap_masks;
        std::atomic<int> fault{0};
        uint64_t read_checksum = 0;  // sink of kPeerReadRows
        std::vector<uint8_t> stage_codes;  // FP8 codes of the row being staged
        std::atomic<uint64_t> staged_epoch{0};
    };

    // One role of one emulated rank: the unit of work a thread is given.
    enum Role : int { kSourceRole = 0, kReceiverRole = 1 };
    struct Task { int rank; int role; };

    void thread_main(int index);
    bool serve_epoch(int index, uint64_t epoch, std::string& error);
    bool source_progress(int rank, uint64_t epoch, bool& done, bool& quiescent, std::string& error);
    bool receiver_progress(int rank, uint64_t epoch, bool& done, std::string& error);
    void publish_token(Rank& state, int rank, uint64_t epoch, int channel, int token, int slot, int ordinal, int fault);
    void fail(const std::string& message);

    bool relays_drained(int rank, uint64_t epoch) const;

    SegmentLayout z_;
    int me_;
    char* seg_[kMaxRanks];
    char* replica_[kMaxRanks][kMaxDomains] = {};
    std::vector<std::unique_ptr<NumaRelay>> relays_;  // one per emulated source (relay mode)
    int timeout_ms_;
    std::vector<Rank> ranks_;
    std::vector<std::thread> threads_;
    std::vector<std::vector<Task>> assignment_;
    std::vector<uint64_t> thread_done_;  // epochs completed per thread (under mutex_)
    std::mutex mutex_;
    std::condition_variable wake_, finished_;
    uint64_t served_ = 0;   // epochs fully served by every thread
    uint64_t target_ = 0;   // epochs requested
    uint32_t flags_ = 0;
    bool stop_ = false;
    std::atomic<bool> cancel_{false};
    std::atomic<bool> failed_{false};
    std::string failure_;
};

}  // namespace pcie_ep

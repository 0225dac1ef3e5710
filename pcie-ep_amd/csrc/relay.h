// NUMA relay workers: CPU threads of a source rank that move its rows from the
// source ring into the replica ring of every other NUMA domain, so that the
// receivers of that domain read memory of their own node and a row crosses the
// socket interconnect once however many ranks of the domain it is bound for.
//
// Replaces NumaRelay of the reference (csrc/comm/numa_relay.hpp:59-427).  One
// object serves ONE source segment.  Per NUMA domain it starts
// `workers_per_domain` threads; a worker owns the (channel, domain) flows of a
// disjoint set of channels.  A flow's progress step never blocks: a full replica
// ring or missing credit of one channel lets the worker go on with its other
// channels (numa_relay.hpp:57-58).
//
// Protocol of a flow (channel c, domain n), per epoch:
//   * the epoch starts when the source's counts_ready shows it; the number of
//     rows to expect is the relay mailbox entry [n][c];
//   * rows arrive as descriptors on endpoint P + n of channel c; for each the
//     worker checks the slot's identity, waits until replica slot `i mod R` has
//     been released by every rank it was last published to and until every
//     targeted rank has a free replica descriptor entry, copies payload +
//     metadata, publishes one replica descriptor per targeted rank of the
//     domain, then ACKs the source slot and returns the descriptor credit on
//     behalf of endpoint P + n;
//   * after the last row, once every replica slot is released, it stores the
//     epoch to relay_drained[c][n]: the source may then start its next epoch.
// Failures store a non-zero code to relay_failed[c][n], which every GPU's
// health scan reads (101 epoch changed before the flow was drained, 102 timeout,
// 103 bad slot, 104 identity mismatch, 105 no target in the domain, 106 worker
// exception: numa_relay.hpp:216-220 and the codes in :240-340).
#pragma once

#include <atomic>
#include <cstdint>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "wire.h"

namespace pcie_ep {

struct RelayOptions {
    int workers_per_domain = 1;
    int timeout_ms = 30000;
    uint64_t delay_ns = 0;
    std::vector<int> cpus;             // CPUs workers may be pinned to; empty = any allowed CPU of the domain's node
    int domain_node[kMaxDomains] = {}; // physical NUMA node of every domain
    // Ranks that really consume replica rows.  All ranks in a deployment; the
    // host peer emulator restricts its sources' relays to the one real GPU.
    uint32_t live_ranks = 0xFFFFFFFFu;
    bool pin = true;
};

struct RelayFlowRecord {
    int32_t channel, domain, worker, cpu;
    int32_t expected_tokens, error;
    uint64_t epoch, copied_tokens, copied_payload_bytes, copy_time_ns_total, credit_wait_probes_total, drained_epoch;
    uint64_t copies_total, payload_bytes_total;
};

class NumaRelay {
public:
    // `replica` holds the replica payload region of this source for every domain.
    NumaRelay(const SegmentLayout& layout, int rank, char* const* segments, char* const* replica, const RelayOptions& options);
    ~NumaRelay();
    NumaRelay(const NumaRelay&) = delete;
    NumaRelay& operator=(const NumaRelay&) = delete;

    void stop_and_join();
    void set_delay(uint64_t delay_ns) { delay_ns_.store(delay_ns, std::memory_order_relaxed); }
    int flows() const;
    int workers() const { return int(workers_.size()); }
    // Snapshot of every flow (at most `capacity` records); returns the number written.
    int diagnostics(RelayFlowRecord* records, int capacity) const;
    std::string worker_errors() const;
    uint64_t ready_epoch() const;

private:
    struct Flow {
        int channel, domain;
        uint64_t epoch = 0, started_ns = 0, delayed_until_ns = 0;
        int expected = 0, copied = 0;
        bool drained = false;
        int sent[kMaxRanks] = {};
        std::vector<uint64_t> replica_sequences;  // per replica slot: what was last published in it ...
        std::vector<uint32_t> replica_masks;      // ... and to which ranks
        std::atomic<uint64_t> diagnostic_epoch{0}, diagnostic_copies{0}, diagnostic_bytes{0};
        std::atomic<uint64_t> copies_total{0}, bytes_total{0}, waits_total{0}, copy_time_ns{0};
        std::atomic<int> diagnostic_expected{0}, failure{0};
        Flow(int c, int n, int slots) : channel(c), domain(n), replica_sequences(slots, 0), replica_masks(slots, 0) {}
    };
    struct Worker {
        int domain = 0, index = 0;
        std::atomic<int> cpu{-1};  // written by the worker thread when it pins itself, read by diagnostics()
        std::string runtime_error;
        mutable std::mutex guard;
        std::vector<std::unique_ptr<Flow>> flows;
        std::thread thread;
    };

    void run(Worker& worker);
    void pin(Worker& worker);
    bool progress(Flow& flow);
    void fail(Flow& flow, int code);
    bool peer_aborted() const;
    bool replica_released(const Flow& flow, int slot) const;

    SegmentLayout z_;
    int rank_;
    char* own_;
    char* seg_[kMaxRanks] = {};
    char* replica_[kMaxDomains] = {};
    RelayOptions options_;
    std::vector<std::unique_ptr<Worker>> workers_;
    std::atomic<bool> stopping_{false};
    std::atomic<uint64_t> delay_ns_{0};
};

// CPUs of a NUMA node (/sys/devices/system/node/nodeN/cpulist); empty when the node does not exist.
std::vector<int> numa_node_cpus(int node);
bool numa_node_exists(int node);

}  // namespace pcie_ep

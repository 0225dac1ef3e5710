// CPU-only exercise of the NUMA relay workers' failure paths: one NumaRelay (the
// relay of source rank 0 in a world of two ranks in two domains) runs on a
// hand-built segment in ordinary memory, and this program plays the source and
// the receiving rank around it.  Every case ends with the relay's threads
// joined.  Built with the host compiler under the address/undefined and the
// thread sanitizer (tests/test_host_protocol.py).
//
// The codes are those a relay flow stores to relay_failed[channel][domain]
// (relay.cpp; the reference's worker fails a flow the same way,
// csrc/comm/numa_relay.hpp:240-340):
//   101 the source began a new epoch before the flow had drained the last one
//   102 the flow made no progress for timeout_ms
//   103 a descriptor names a payload slot outside the ring
//   104 the slot's metadata holds another token than the descriptor
//   105 a row for this domain has no destination in it
//   106 the worker thread ended with an exception (here: it cannot be pinned)
#include <sched.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "relay.h"

using namespace pcie_ep;

namespace {

constexpr int kRanks = 2, kTokens = 8, kHidden = 32, kTopk = 2, kExperts = 4, kChannels = 1, kSlots = 2, kDescriptors = 2;
constexpr int kFar = 1;  // the domain of rank 1: the flow the cases drive

inline uint64_t acquire(uint64_t* address) { return std::atomic_ref<uint64_t>(*address).load(std::memory_order_acquire); }
inline void release(uint64_t* address, uint64_t value) { std::atomic_ref<uint64_t>(*address).store(value, std::memory_order_release); }

int fail(const std::string& message) {
    std::fprintf(stderr, "FAILED: %s\n", message.c_str());
    return 1;
}

struct World {
    SegmentLayout z;
    char* segments[kMaxRanks] = {};
    char* replica[kMaxDomains] = {};
    World() {
        Dimensions dims{kRanks, kTokens, kHidden, kTopk, kExperts, kChannels, kSlots, kDescriptors, /*wire_fp8*/ 0};
        dims.domains = 2;
        dims.replica_slots = 2;
        dims.rank_domain[0] = 0;
        dims.rank_domain[1] = 1;
        z = make_segment_layout(dims);
        for (int rank = 0; rank < kRanks; ++rank) segments[rank] = zeroed(z.size_bytes);
        for (int domain = 0; domain < dims.domains; ++domain) replica[domain] = zeroed(z.replica_region_bytes);
    }
    ~World() {
        for (char* pointer : segments) std::free(pointer);
        for (char* pointer : replica) std::free(pointer);
    }
    static char* zeroed(size_t bytes) {
        void* pointer = std::aligned_alloc(kPageBytes, align_up(bytes, kPageBytes));
        std::memset(pointer, 0, align_up(bytes, kPageBytes));
        return static_cast<char*>(pointer);
    }
    char* own() { return segments[0]; }
    // The source announces an epoch in which the far flow carries `expected` rows.
    void begin_epoch(uint64_t epoch, int expected) {
        relay_mailbox_at(z, own(), 0)[0] = 0;
        relay_mailbox_at(z, own(), kFar)[0] = expected;
        release(signal_at(own(), z.counts_ready_offset), epoch);
    }
    // A source that begins an epoch although a flow has not drained the last one (the relay
    // mailbox, which such a flow may still be reading, keeps its contents).
    void begin_epoch_early(uint64_t epoch) { release(signal_at(own(), z.counts_ready_offset), epoch); }
    // The source publishes row `ordinal` of the far flow: slot contents, then the descriptor of endpoint P + domain.
    void publish(uint64_t epoch, int ordinal, int slot, int token, int header_token, uint32_t mask) {
        if (slot >= 0 && slot < kSlots) {
            char* base = slot_at(z, own(), 0, slot);
            std::memset(base, 0x40 + token, size_t(z.payload_bytes));
            SlotMetaHeader header{};
            header.token_index = header_token;
            header.destination_mask = mask;
            header.scale = 1.0f;
            std::memcpy(base + z.meta_offset, &header, sizeof header);
        }
        Descriptor* descriptor = descriptor_at(z, own(), 0, kRanks + kFar, ordinal);
        descriptor->payload_slot = slot;
        descriptor->token_index = token;
        release(&descriptor->ready, sequence(epoch, ordinal));
    }
    uint64_t failed() { return acquire(signal_at(own(), z.relay_failed_offset, flow_index(z, 0, kFar))); }
    uint64_t drained(int domain) { return acquire(signal_at(own(), z.relay_drained_offset, flow_index(z, 0, domain))); }
};

template <typename Condition>
bool eventually(Condition condition, int milliseconds = 5000) {
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(milliseconds);
    while (!condition()) {
        if (std::chrono::steady_clock::now() > deadline) return false;
        std::this_thread::sleep_for(std::chrono::microseconds(200));
    }
    return true;
}

RelayOptions options(int timeout_ms) {
    RelayOptions result;
    result.timeout_ms = timeout_ms;
    result.pin = false;
    return result;
}

int first_allowed_cpu() {
    cpu_set_t allowed;
    CPU_ZERO(&allowed);
    if (sched_getaffinity(0, sizeof allowed, &allowed)) return -1;
    for (int cpu = 0; cpu < CPU_SETSIZE; ++cpu)
        if (CPU_ISSET(cpu, &allowed)) return cpu;
    return -1;
}

// A row goes through: copied to the replica ring, announced to rank 1, ACKed by it, the flow drains.  The
// workers are pinned (to a CPU the caller names: the far domain's node does not exist on a one-node machine).
int happy_path_pinned() {
    World w;
    RelayOptions pinned = options(20000);
    pinned.pin = true;
    pinned.domain_node[0] = 0;
    pinned.domain_node[1] = 1 << 20;  // a node no machine has: its CPU list is empty
    const int cpu = first_allowed_cpu();
    if (cpu < 0) return fail("no allowed CPU");
    pinned.cpus = {cpu};
    NumaRelay relay(w.z, 0, w.segments, w.replica, pinned);
    w.begin_epoch(1, 1);
    w.publish(1, 0, 1, 5, 5, 1u << 1);
    Descriptor* outgoing = replica_descriptor_at(w.z, w.own(), 0, kFar, 1, 0);
    if (!eventually([&] { return acquire(&outgoing->ready) == sequence(1, 0); })) return fail("the relay did not publish the replica descriptor: " + relay.worker_errors());
    if (outgoing->token_index != 5) return fail("replica descriptor names another token");
    const char* copy = replica_slot_at(w.z, w.replica[kFar], 0, outgoing->payload_slot);
    if (static_cast<unsigned char>(copy[0]) != 0x45 || static_cast<unsigned char>(copy[w.z.payload_bytes - 1]) != 0x45) return fail("replica payload differs");
    // The relay publishes the replica descriptor first and ACKs the source slot right after.
    if (!eventually([&] { return acquire(ack_at(w.z, w.own(), 0, 1, kRanks + kFar)) == sequence(1, 5); }))
        return fail("the source slot was not ACKed on behalf of the relay endpoint");
    // Rank 1 consumes the replica row.
    release(replica_ack_at(w.z, w.own(), 0, kFar, outgoing->payload_slot, 1), sequence(1, 5));
    release(replica_credit_at(w.z, w.own(), 0, kFar, 1), sequence(1, 0));
    if (!eventually([&] { return w.drained(kFar) == 1 && w.drained(0) == 1; })) return fail("the flows did not drain");
    if (w.failed()) return fail("unexpected failure code " + std::to_string(w.failed()));
    std::vector<RelayFlowRecord> records(8);
    const int flows = relay.diagnostics(records.data(), int(records.size()));
    for (int i = 0; i < flows; ++i)
        if (records[i].cpu != cpu) return fail("worker not pinned to the requested CPU");
    return 0;
}

// True once every flow of the relay has taken up `epoch`.
bool flows_entered(const NumaRelay& relay, uint64_t epoch) {
    std::vector<RelayFlowRecord> records(8);
    const int flows = relay.diagnostics(records.data(), int(records.size()));
    for (int i = 0; i < flows; ++i)
        if (records[i].epoch != epoch) return false;
    return flows > 0;
}

int expect_code(const char* name, uint64_t code, int timeout_ms, void (*drive)(World&, const NumaRelay&)) {
    World w;
    {
        NumaRelay relay(w.z, 0, w.segments, w.replica, options(timeout_ms));
        drive(w, relay);
        if (!eventually([&] { return w.failed() != 0; })) return fail(std::string(name) + ": no failure code was stored");
        if (w.failed() != code) return fail(std::string(name) + ": code " + std::to_string(w.failed()) + ", expected " + std::to_string(code));
        // Nothing was copied or announced for the failed row.
        if (acquire(&replica_descriptor_at(w.z, w.own(), 0, kFar, 1, 0)->ready)) return fail(std::string(name) + ": a replica descriptor was published");
        if (!relay.worker_errors().empty()) return fail(std::string(name) + ": worker exception " + relay.worker_errors());
    }  // the destructor joins the workers
    return 0;
}

// A failed flow stays failed: it copies nothing in a later epoch, and because it never drained,
// the next epoch the source announces is recorded as 101.
int failure_is_sticky() {
    World w;
    NumaRelay relay(w.z, 0, w.segments, w.replica, options(20000));
    w.begin_epoch(1, 1);
    w.publish(1, 0, kSlots, 3, 3, 1u << 1);
    if (!eventually([&] { return w.failed() == 103; })) return fail("sticky: expected 103 first");
    w.begin_epoch_early(2);
    w.publish(2, 0, 0, 3, 3, 1u << 1);
    if (!eventually([&] { return w.failed() == 101; })) return fail("sticky: expected 101 for the epoch after a failure, got " + std::to_string(w.failed()));
    std::this_thread::sleep_for(std::chrono::milliseconds(20));
    if (acquire(&replica_descriptor_at(w.z, w.own(), 0, kFar, 1, 0)->ready)) return fail("sticky: a failed flow copied a row");
    // The other flow of the relay is not affected.
    if (!eventually([&] { return w.drained(0) == 2; })) return fail("sticky: the healthy flow did not drain epoch 2");
    return 0;
}

// A worker that cannot be pinned where it was told to ends with an exception: 106 on all its flows.
int worker_exception() {
    World w;
    RelayOptions pinned = options(20000);
    pinned.pin = true;
    pinned.domain_node[0] = pinned.domain_node[1] = 1 << 20;
    pinned.cpus = {CPU_SETSIZE - 1 + 100000};  // no such CPU
    NumaRelay relay(w.z, 0, w.segments, w.replica, pinned);
    if (!eventually([&] { return w.failed() == 106; })) return fail("worker exception: expected 106, got " + std::to_string(w.failed()));
    if (relay.worker_errors().find("no allowed CPU") == std::string::npos) return fail("worker exception: message is '" + relay.worker_errors() + "'");
    return 0;
}

}  // namespace

int main() {
    int status = happy_path_pinned();
    if (!status) std::printf("happy path with pinned workers ok\n");
    if (!status) status = expect_code("epoch changed before the drain", 101, 20000, [](World& w, const NumaRelay& relay) {
        w.begin_epoch(1, 1);  // one row expected, none published
        // The next epoch begins once the flows are inside this one (a flow that first looks after the second
        // announcement would simply start there).
        eventually([&] { return flows_entered(relay, 1); });
        w.begin_epoch_early(2);
    });
    if (!status) status = expect_code("no progress", 102, 60, [](World& w, const NumaRelay&) { w.begin_epoch(1, 1); });
    if (!status) status = expect_code("slot outside the ring", 103, 20000, [](World& w, const NumaRelay&) {
        w.begin_epoch(1, 1);
        w.publish(1, 0, kSlots, 2, 2, 1u << 1);
    });
    if (!status) status = expect_code("identity mismatch", 104, 20000, [](World& w, const NumaRelay&) {
        w.begin_epoch(1, 1);
        w.publish(1, 0, 0, 2, 6, 1u << 1);
    });
    if (!status) status = expect_code("no destination in the domain", 105, 20000, [](World& w, const NumaRelay&) {
        w.begin_epoch(1, 1);
        w.publish(1, 0, 0, 2, 2, 1u << 0);
    });
    if (!status) std::printf("failure codes 101-105 ok\n");
    if (!status) status = failure_is_sticky();
    if (!status) status = worker_exception();
    if (!status) std::printf("relay failure test passed\n");
    return status;
}

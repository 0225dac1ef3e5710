// NUMA relay workers (see relay.h).  Plain C++20, no GPU call: the segments are
// pinned host memory that the GPUs map.
#include "relay.h"

#include <pthread.h>
#include <sched.h>

#include <algorithm>
#include <chrono>
#include <cstring>
#include <fstream>
#include <sstream>

namespace pcie_ep {

namespace {

inline uint64_t acquire(uint64_t* address) { return std::atomic_ref<uint64_t>(*address).load(std::memory_order_acquire); }
inline void release(uint64_t* address, uint64_t value) { std::atomic_ref<uint64_t>(*address).store(value, std::memory_order_release); }
inline uint64_t now_ns() {
    return uint64_t(std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count());
}

}  // namespace

bool numa_node_exists(int node) {
    if (node < 0) return false;
    return std::ifstream("/sys/devices/system/node/node" + std::to_string(node) + "/cpulist").good();
}

std::vector<int> numa_node_cpus(int node) {
    std::vector<int> cpus;
    std::ifstream file("/sys/devices/system/node/node" + std::to_string(node) + "/cpulist");
    std::string text;
    if (!(file >> text)) return cpus;
    std::stringstream ranges(text);
    std::string range;
    while (std::getline(ranges, range, ',')) {
        const size_t dash = range.find('-');
        const int first = std::stoi(range.substr(0, dash));
        const int last = dash == std::string::npos ? first : std::stoi(range.substr(dash + 1));
        for (int cpu = first; cpu <= last; ++cpu) cpus.push_back(cpu);
    }
    return cpus;
}

NumaRelay::NumaRelay(const SegmentLayout& layout, int rank, char* const* segments, char* const* replica, const RelayOptions& options)
    : z_(layout), rank_(rank), own_(segments[rank]), options_(options), delay_ns_(options.delay_ns) {
    for (int r = 0; r < z_.dims.num_ranks; ++r) seg_[r] = segments[r];
    for (int n = 0; n < z_.dims.domains; ++n) replica_[n] = replica[n];
    const int per_domain = std::max(1, std::min(options_.workers_per_domain, z_.dims.channels));
    for (int domain = 0; domain < z_.dims.domains; ++domain) {
        for (int index = 0; index < per_domain; ++index) {
            auto worker = std::make_unique<Worker>();
            worker->domain = domain;
            worker->index = index;
            // Worker `index` of a domain owns channels index, index + W, ...
            for (int channel = index; channel < z_.dims.channels; channel += per_domain)
                worker->flows.push_back(std::make_unique<Flow>(channel, domain, z_.dims.replica_slots));
            workers_.push_back(std::move(worker));
        }
    }
    for (auto& worker : workers_) {
        Worker* pointer = worker.get();
        pointer->thread = std::thread([this, pointer] { run(*pointer); });
    }
}

NumaRelay::~NumaRelay() { stop_and_join(); }

void NumaRelay::stop_and_join() {
    stopping_.store(true, std::memory_order_release);
    for (auto& worker : workers_)
        if (worker->thread.joinable()) worker->thread.join();
}

int NumaRelay::flows() const {
    int total = 0;
    for (const auto& worker : workers_) total += int(worker->flows.size());
    return total;
}

uint64_t NumaRelay::ready_epoch() const { return acquire(signal_at(own_, z_.counts_ready_offset)); }

int NumaRelay::diagnostics(RelayFlowRecord* records, int capacity) const {
    int written = 0;
    for (size_t w = 0; w < workers_.size(); ++w) {
        const Worker& worker = *workers_[w];
        for (const auto& flow : worker.flows) {
            if (written >= capacity) return written;
            RelayFlowRecord& r = records[written++];
            r.channel = flow->channel;
            r.domain = flow->domain;
            r.worker = int(w);
            r.cpu = worker.cpu.load(std::memory_order_relaxed);
            r.epoch = flow->diagnostic_epoch.load(std::memory_order_acquire);
            r.expected_tokens = flow->diagnostic_expected.load(std::memory_order_relaxed);
            r.copied_tokens = flow->diagnostic_copies.load(std::memory_order_relaxed);
            r.copied_payload_bytes = flow->diagnostic_bytes.load(std::memory_order_relaxed);
            r.copy_time_ns_total = flow->copy_time_ns.load(std::memory_order_relaxed);
            r.credit_wait_probes_total = flow->waits_total.load(std::memory_order_relaxed);
            r.drained_epoch = acquire(signal_at(own_, z_.relay_drained_offset, flow_index(z_, flow->channel, flow->domain)));
            r.error = flow->failure.load(std::memory_order_relaxed);
            r.copies_total = flow->copies_total.load(std::memory_order_relaxed);
            r.payload_bytes_total = flow->bytes_total.load(std::memory_order_relaxed);
        }
    }
    return written;
}

std::string NumaRelay::worker_errors() const {
    std::string all;
    for (const auto& worker : workers_) {
        std::lock_guard<std::mutex> lock(worker->guard);
        if (!worker->runtime_error.empty()) all += (all.empty() ? "" : "; ") + worker->runtime_error;
    }
    return all;
}

// Pin the worker to one allowed CPU of its domain's node (numa_relay.hpp:178-199).
// A node that does not exist on this machine has no CPU list: the worker is then
// pinned among the CPUs the caller asked for (relay_cpu_affinity) if there are any,
// and left unpinned otherwise - the reference refuses such a map ("no allowed CPU on
// requested relay NUMA node", numa_relay.hpp:192-206), which would rule out every
// logical NUMA map on a one-node machine.  A request none of whose CPUs is allowed
// fails as in the reference.
void NumaRelay::pin(Worker& worker) {
    if (!options_.pin) return;
    const std::vector<int> node_cpus = numa_node_cpus(options_.domain_node[worker.domain]);
    if (node_cpus.empty() && options_.cpus.empty()) return;
    cpu_set_t allowed;
    CPU_ZERO(&allowed);
    if (pthread_getaffinity_np(pthread_self(), sizeof allowed, &allowed) != 0) throw std::runtime_error("cannot query relay thread CPU affinity");
    std::vector<int> candidates;
    for (int cpu : node_cpus.empty() ? options_.cpus : node_cpus) {
        const bool wanted = options_.cpus.empty() || std::find(options_.cpus.begin(), options_.cpus.end(), cpu) != options_.cpus.end();
        if (cpu >= 0 && cpu < CPU_SETSIZE && CPU_ISSET(cpu, &allowed) && wanted) candidates.push_back(cpu);
    }
    if (candidates.empty()) throw std::runtime_error("no allowed CPU on requested relay NUMA node");
    const int chosen = candidates[size_t(rank_ * options_.workers_per_domain + worker.index) % candidates.size()];
    worker.cpu.store(chosen, std::memory_order_relaxed);
    cpu_set_t target;
    CPU_ZERO(&target);
    CPU_SET(chosen, &target);
    if (const int status = pthread_setaffinity_np(pthread_self(), sizeof target, &target))
        throw std::runtime_error("cannot pin relay worker: " + std::to_string(status));
}

void NumaRelay::fail(Flow& flow, int code) {
    flow.failure.store(code, std::memory_order_relaxed);
    release(signal_at(own_, z_.relay_failed_offset, flow_index(z_, flow.channel, flow.domain)), uint64_t(code));
}

bool NumaRelay::peer_aborted() const {
    for (int rank = 0; rank < z_.dims.num_ranks; ++rank) {
        if (acquire(signal_at(seg_[rank], z_.abort_offset))) return true;
        for (int channel = 0; channel < z_.dims.channels; ++channel)
            if (acquire(signal_at(seg_[rank], z_.channel_abort_offset, channel))) return true;
    }
    return false;
}

// A replica slot is free again once every rank it was last published to has ACKed it.
bool NumaRelay::replica_released(const Flow& flow, int slot) const {
    const uint64_t published = flow.replica_sequences[slot];
    const uint32_t targets = flow.replica_masks[slot];
    for (int rank = 0; rank < z_.dims.num_ranks; ++rank)
        if (((targets >> rank) & 1u) && acquire(replica_ack_at(z_, own_, flow.channel, flow.domain, slot, rank)) != published) return false;
    return true;
}

// One non-blocking step of a flow; true when it advanced.
bool NumaRelay::progress(Flow& flow) {
    const uint64_t ready_epoch = acquire(signal_at(own_, z_.counts_ready_offset));
    if (!ready_epoch) return false;  // nothing has been dispatched yet: no work and no timeout origin
    const int endpoint = z_.dims.num_ranks + flow.domain;
    if (ready_epoch != flow.epoch) {
        // The source may only start an epoch after this flow reported the previous one drained.
        if (flow.epoch && !flow.drained) {
            fail(flow, 101);
            return false;
        }
        flow.epoch = ready_epoch;
        flow.started_ns = now_ns();
        flow.expected = relay_mailbox_at(z_, own_, flow.domain)[flow.channel];
        flow.copied = 0;
        flow.drained = false;
        flow.delayed_until_ns = 0;
        std::fill(std::begin(flow.sent), std::end(flow.sent), 0);
        std::fill(flow.replica_sequences.begin(), flow.replica_sequences.end(), 0);
        std::fill(flow.replica_masks.begin(), flow.replica_masks.end(), 0u);
        flow.diagnostic_expected.store(flow.expected, std::memory_order_relaxed);
        flow.diagnostic_copies.store(0, std::memory_order_relaxed);
        flow.diagnostic_bytes.store(0, std::memory_order_relaxed);
        flow.diagnostic_epoch.store(flow.epoch, std::memory_order_release);
    }
    if (flow.drained || flow.failure.load(std::memory_order_relaxed)) return false;
    if (now_ns() - flow.started_ns > uint64_t(options_.timeout_ms) * 1000000ull) {
        fail(flow, 102);
        return false;
    }
    if (flow.copied == flow.expected) {
        for (int slot = 0; slot < z_.dims.replica_slots; ++slot)
            if (!replica_released(flow, slot)) return false;
        release(signal_at(own_, z_.relay_drained_offset, flow_index(z_, flow.channel, flow.domain)), flow.epoch);
        flow.drained = true;
        return true;
    }

    // Next row of the flow: descriptor `copied` of endpoint P + domain.
    Descriptor* incoming = descriptor_at(z_, own_, flow.channel, endpoint, flow.copied);
    if (acquire(&incoming->ready) != sequence(flow.epoch, flow.copied)) return false;
    const int source_slot = incoming->payload_slot, token = incoming->token_index;
    if (source_slot < 0 || source_slot >= z_.dims.payload_slots) {
        fail(flow, 103);
        return false;
    }
    const char* source = slot_at(z_, own_, flow.channel, source_slot);
    SlotMetaHeader header;
    std::memcpy(&header, source + z_.meta_offset, sizeof header);
    if (header.token_index != token) {
        fail(flow, 104);
        return false;
    }
    const uint64_t payload_sequence = sequence(flow.epoch, token);
    const int replica_slot = flow.copied % z_.dims.replica_slots;
    if (!replica_released(flow, replica_slot)) {
        flow.waits_total.fetch_add(1, std::memory_order_relaxed);
        return false;
    }
    uint32_t targets = 0;
    for (int rank = 0; rank < z_.dims.num_ranks; ++rank) {
        if (rank == rank_ || z_.dims.rank_domain[rank] != flow.domain || !((header.destination_mask >> rank) & 1u)) continue;
        if (!((options_.live_ranks >> rank) & 1u)) continue;
        targets |= 1u << rank;
        const uint64_t credit = acquire(replica_credit_at(z_, own_, flow.channel, flow.domain, rank));
        if (!credit_covers(credit, flow.epoch, flow.sent[rank], z_.dims.descriptor_slots)) {
            flow.waits_total.fetch_add(1, std::memory_order_relaxed);
            return false;
        }
    }
    if (!targets) {
        fail(flow, 105);
        return false;
    }
    if (const uint64_t delay = delay_ns_.load(std::memory_order_relaxed); delay && !flow.delayed_until_ns) flow.delayed_until_ns = now_ns() + delay;
    if (flow.delayed_until_ns && now_ns() < flow.delayed_until_ns) return false;
    flow.delayed_until_ns = 0;

    // Copy payload and slot metadata (one contiguous range of the slot) into the replica slot.
    char* destination = replica_slot_at(z_, replica_[flow.domain], flow.channel, replica_slot);
    const uint64_t begin = now_ns();
    std::memcpy(destination, source, size_t(z_.payload_bytes));
    std::memcpy(destination + z_.meta_offset, source + z_.meta_offset, size_t(z_.meta_bytes));
    flow.copy_time_ns.fetch_add(now_ns() - begin, std::memory_order_relaxed);
    for (int rank = 0; rank < z_.dims.num_ranks; ++rank) {
        if (!((targets >> rank) & 1u)) continue;
        Descriptor* outgoing = replica_descriptor_at(z_, own_, flow.channel, flow.domain, rank, flow.sent[rank]);
        outgoing->payload_slot = replica_slot;
        outgoing->token_index = token;
        release(&outgoing->ready, sequence(flow.epoch, flow.sent[rank]));
        ++flow.sent[rank];
    }
    flow.replica_sequences[replica_slot] = payload_sequence;
    flow.replica_masks[replica_slot] = targets;
    // The CPU is done with the source slot: ACK it and return the descriptor
    // entry on behalf of the relay endpoint.
    release(ack_at(z_, own_, flow.channel, source_slot, endpoint), payload_sequence);
    release(credit_at(z_, own_, flow.channel, endpoint), sequence(flow.epoch, flow.copied));
    ++flow.copied;
    flow.diagnostic_copies.store(uint64_t(flow.copied), std::memory_order_relaxed);
    flow.diagnostic_bytes.store(uint64_t(flow.copied) * uint64_t(z_.payload_bytes), std::memory_order_relaxed);
    flow.copies_total.fetch_add(1, std::memory_order_relaxed);
    flow.bytes_total.fetch_add(uint64_t(z_.payload_bytes), std::memory_order_relaxed);
    return true;
}

void NumaRelay::run(Worker& worker) {
    try {
        pin(worker);
        uint64_t idle_passes = 0;
        while (!stopping_.load(std::memory_order_acquire)) {
            // The abort flags of every rank are 1 + C words each: look at them now
            // and then, not between any two rows.
            if ((idle_passes & 0x3F) == 0 && peer_aborted()) return;
            bool advanced = false;
            for (auto& flow : worker.flows) advanced |= progress(*flow);
            if (advanced) {
                idle_passes = 1;
            } else {
                ++idle_passes;
                std::this_thread::yield();
            }
        }
    } catch (const std::exception& error) {
        {
            std::lock_guard<std::mutex> lock(worker.guard);
            worker.runtime_error = error.what();
        }
        for (auto& flow : worker.flows) fail(*flow, 106);
    }
}

}  // namespace pcie_ep

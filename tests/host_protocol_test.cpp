// CPU-only exercise of the host side of the ring protocol: two peer emulators
// play the two ranks of a P = 2 world against each other on ordinary memory, in
// direct mode and through NUMA relay workers.  No GPU and no HIP call: the
// program is built with the host compiler (with the address/undefined or the
// thread sanitizer) from peers.cpp, relay.cpp and the wire-format headers.
//
// Emulator A stands for "the GPU is rank 0" and therefore runs rank 1; emulator
// B stands for "the GPU is rank 1" and runs rank 0.  A's source role of rank 1
// feeds B's receiver role of rank 0 through segment 1, and vice versa, so every
// host-side path is driven by a real counterpart: count mailboxes, payload
// slots, descriptor queues, credits, ACKs, and in relay mode the relay workers,
// replica rings, replica ACKs/credits and relay_drained.
//
// usage: host_protocol_test <direct|relay> [epochs]
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "peers.h"

using namespace pcie_ep;

namespace {

constexpr int kRanks = 2, kTokens = 45, kHidden = 96, kTopk = 2, kExperts = 8, kChannels = 3;

struct Inputs {
    std::vector<uint16_t> x;
    std::vector<int64_t> idx;
    std::vector<float> weights;
};

Inputs make_inputs(int rank, int tokens, int salt) {
    Inputs in;
    in.x.resize(size_t(tokens) * kHidden);
    in.idx.resize(size_t(tokens) * kTopk);
    in.weights.resize(size_t(tokens) * kTopk);
    uint32_t state = 0x9E3779B9u * uint32_t(rank + 1) + uint32_t(salt) * 7919u;
    auto next = [&] {
        state = state * 1664525u + 1013904223u;
        return state >> 8;
    };
    for (auto& value : in.x) value = uint16_t(0x3C00u + next() % 0x0400u);  // finite BF16 patterns
    for (int token = 0; token < tokens; ++token) {
        const int first = int(next() % kExperts);
        int second = int(next() % kExperts);
        if (second == first) second = (second + 1) % kExperts;
        in.idx[size_t(token) * kTopk] = token % 7 == 3 ? -1 : first;  // some unused branches
        in.idx[size_t(token) * kTopk + 1] = second;
        in.weights[size_t(token) * kTopk] = float(next() % 1000) / 1000.0f;
        in.weights[size_t(token) * kTopk + 1] = float(next() % 1000) / 1000.0f;
    }
    return in;
}

char* zeroed(size_t bytes) {
    void* pointer = std::aligned_alloc(kPageBytes, align_up(bytes, kPageBytes));
    std::memset(pointer, 0, align_up(bytes, kPageBytes));
    return static_cast<char*>(pointer);
}

int fail(const std::string& message) {
    std::fprintf(stderr, "FAILED: %s\n", message.c_str());
    return 1;
}

// What `receiver` captured from `sender` must be exactly the sender's tokens
// with the receiver's destination bit, each once, with the sender's bytes.
int check_captured(PeerEmulator& emulator, int receiver, const Inputs& sent, int tokens, const SegmentLayout& z) {
    std::vector<uint32_t> mask(tokens);
    std::vector<int32_t> rank_ordinals(size_t(tokens) * kRanks), expert_indices(size_t(tokens) * kTopk), expert_ordinals(size_t(tokens) * kTopk);
    std::vector<int32_t> counts(kRanks + kExperts);
    if (host_source_layout(sent.idx.data(), tokens, kTopk, kRanks, kExperts, mask.data(), rank_ordinals.data(), expert_indices.data(),
                           expert_ordinals.data(), counts.data()))
        return fail("invalid routing in the test inputs");
    const int64_t got = emulator.captured_count(receiver);
    if (got != counts[receiver]) return fail("rank " + std::to_string(receiver) + " captured " + std::to_string(got) + " rows, expected " + std::to_string(counts[receiver]));
    std::vector<int32_t> cap_tokens(got), cap_ordinals(got), cap_idx(size_t(got) * kTopk), cap_ord(size_t(got) * kTopk);
    std::vector<uint8_t> payload(size_t(got) * z.payload_bytes);
    std::vector<float> scales(got), weights(size_t(got) * kTopk);
    std::vector<uint32_t> masks(got);
    emulator.captured_copy(receiver, cap_tokens.data(), cap_ordinals.data(), payload.data(), scales.data(), cap_idx.data(), cap_ord.data(),
                           weights.data(), masks.data());
    std::vector<char> seen(tokens, 0);
    for (int64_t row = 0; row < got; ++row) {
        const int token = cap_tokens[row];
        if (token < 0 || token >= tokens || seen[token] || !((mask[token] >> receiver) & 1u)) return fail("unexpected or repeated token in the captured rows");
        seen[token] = 1;
        if (cap_ordinals[row] != rank_ordinals[size_t(token) * kRanks + receiver] || masks[row] != mask[token]) return fail("captured ordinal or mask differs");
        if (std::memcmp(payload.data() + size_t(row) * z.payload_bytes, sent.x.data() + size_t(token) * kHidden, size_t(z.payload_bytes)))
            return fail("captured payload differs from what the source sent");
        for (int k = 0; k < kTopk; ++k) {
            if (cap_idx[size_t(row) * kTopk + k] != expert_indices[size_t(token) * kTopk + k] ||
                cap_ord[size_t(row) * kTopk + k] != expert_ordinals[size_t(token) * kTopk + k] ||
                std::memcmp(&weights[size_t(row) * kTopk + k], &sent.weights[size_t(token) * kTopk + k], 4))
                return fail("captured branch metadata differs");
        }
    }
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    const bool relay = argc > 1 && std::string(argv[1]) == "relay";
    const int epochs = argc > 2 ? std::atoi(argv[2]) : 4;
    const int threads = argc > 3 ? std::atoi(argv[3]) : 1;  // 2: the peer's source and receiver roles on a thread each
    Dimensions dims{kRanks, kTokens, kHidden, kTopk, kExperts, kChannels, /*payload_slots*/ 2, /*descriptor_slots*/ 1, /*wire_fp8*/ 0};
    if (relay) {
        dims.domains = 2;
        dims.replica_slots = 3;
        dims.rank_domain[0] = 0;
        dims.rank_domain[1] = 1;
    }
    const SegmentLayout z = make_segment_layout(dims);
    char* segments[kMaxRanks] = {};
    char* replica[kMaxRanks * kMaxDomains] = {};
    for (int rank = 0; rank < kRanks; ++rank) {
        segments[rank] = zeroed(z.size_bytes);
        for (int domain = 0; domain < dims.domains; ++domain) replica[rank * kMaxDomains + domain] = zeroed(z.replica_region_bytes);
    }
    RelayOptions options;
    options.timeout_ms = 20000;
    options.pin = false;
    int status = 0;
    {
        PeerEmulator gpu_is_rank0(z, 0, segments, replica, threads, 20000, options);  // runs rank 1
        PeerEmulator gpu_is_rank1(z, 1, segments, replica, threads, 20000, options);  // runs rank 0
        std::string error;
        for (int epoch = 0; epoch < epochs && !status; ++epoch) {
            // Token counts change from epoch to epoch, including an empty source.
            const int tokens0 = epoch % 3 == 2 ? 0 : kTokens - epoch, tokens1 = kTokens - 2 * epoch;
            const Inputs in0 = make_inputs(0, tokens0, epoch), in1 = make_inputs(1, tokens1, epoch);
            if (gpu_is_rank1.set_source(0, in0.x.data(), in0.idx.data(), in0.weights.data(), tokens0, error) ||
                gpu_is_rank0.set_source(1, in1.x.data(), in1.idx.data(), in1.weights.data(), tokens1, error))
                status = fail("set_source: " + error);
            if (!status && (gpu_is_rank0.start(1, kPeerCapture | kPeerRestage, error) || gpu_is_rank1.start(1, kPeerCapture | kPeerReadRows, error)))
                status = fail("start: " + error);
            if (!status && (gpu_is_rank0.wait(30000, error) || gpu_is_rank1.wait(30000, error))) status = fail("wait: " + error);
            // Rank 1 (run by A) received what rank 0 (run by B) sent, and vice versa.
            if (!status) status = check_captured(gpu_is_rank0, 1, in0, tokens0, z);
            if (!status) status = check_captured(gpu_is_rank1, 0, in1, tokens1, z);
            if (!status) std::printf("epoch %d ok: %d + %d tokens, %s\n", epoch + 1, tokens0, tokens1, relay ? "relay" : "direct");
        }
    }
    for (char* pointer : segments) std::free(pointer);
    for (char* pointer : replica) std::free(pointer);
    if (!status) std::printf("host protocol test passed\n");
    return status;
}

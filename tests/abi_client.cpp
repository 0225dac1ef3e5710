// Stand-alone client of the C ABI: no Python, no torch.  It includes only
// include/pcie_ep_amd.h and the HIP runtime API, creates a runtime for logical
// rank 0 of 2 (the other rank is one host peer thread), dispatches once with
// small rings that wrap, and checks every output against a direct evaluation of
// the dispatch semantics (expert-major rows, sources in rank order, tokens in
// order; csrc/kernels/host_staged/advanced_layout.cuh:94-154, :207-215 of the
// reference).  Exit status 0 = all checks passed.
//
// Built by pcie-ep_amd/build.py next to the library; run by
// tests/test_gpu_abi_client.py.
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "pcie_ep_amd.h"

namespace {

constexpr int kRanks = 2, kTokens = 24, kHidden = 64, kTopk = 2, kExperts = 4, kLocal = kExperts / kRanks;

#define CHECK(condition, ...)                      \
    do {                                           \
        if (!(condition)) {                        \
            std::fprintf(stderr, "FAILED: ");      \
            std::fprintf(stderr, __VA_ARGS__);     \
            std::fprintf(stderr, "\n");            \
            return 1;                              \
        }                                          \
    } while (0)
#define HIP(call) CHECK((call) == hipSuccess, "%s", #call)
#define ABI(call) CHECK((call) == 0, "%s: %s", #call, pcie_ep_last_error())

uint16_t payload(int source, int token, int column) { return uint16_t((source * 9001 + token * 131 + column * 7 + 1) & 0x3FFF); }
int64_t route(int source, int token, int branch) {
    // Two distinct experts per token, spread over both ranks; every third token of rank 1 skips a branch.
    const int first = (token * 3 + source) % kExperts;
    if (branch == 0) return first;
    if (source == 1 && token % 3 == 0) return -1;
    return (first + 1 + token % 3) % kExperts;
}
float weight(int source, int token, int branch) { return 0.125f * float(source + 1) + 0.01f * float(token) + 0.5f * float(branch); }

template <typename T>
T* device_array(size_t count) {
    void* pointer = nullptr;
    if (hipMalloc(&pointer, count * sizeof(T) + 16) != hipSuccess) std::exit(3);
    if (hipMemset(pointer, 0xEE, count * sizeof(T)) != hipSuccess) std::exit(3);
    return static_cast<T*>(pointer);
}
template <typename T>
std::vector<T> to_host(const T* device, size_t count) {
    std::vector<T> host(count);
    if (hipMemcpy(host.data(), device, count * sizeof(T), hipMemcpyDeviceToHost) != hipSuccess) std::exit(3);
    return host;
}

}  // namespace

int main() {
    CHECK(pcie_ep_abi_version() == PCIE_EP_ABI_VERSION, "ABI version");
    pcie_ep_config config{};
    config.num_ranks = kRanks;
    config.max_tokens = kTokens;
    config.hidden = kHidden;
    config.topk = kTopk;
    config.num_experts = kExperts;
    config.channels = 2;
    config.payload_slots = 4;  // 12 tokens per channel: the rings wrap
    config.descriptor_slots = 3;
    config.timeout_ms = 5000;
    config.fuse_receive_expand = 1;
    config.peer_threads = 1;
    config.staging_numa_node = -1;
    pcie_ep_sizes sizes{};
    ABI(pcie_ep_query_sizes(&config, &sizes));
    CHECK(sizes.unique_rows == kRanks * kTokens && sizes.local_experts == kLocal, "sizes");
    pcie_ep_runtime* runtime = nullptr;
    ABI(pcie_ep_runtime_create(&config, &runtime));

    // Inputs of both ranks.
    std::vector<uint16_t> x[kRanks];
    std::vector<int64_t> idx[kRanks];
    std::vector<float> w[kRanks];
    for (int s = 0; s < kRanks; ++s) {
        for (int t = 0; t < kTokens; ++t) {
            for (int c = 0; c < kHidden; ++c) x[s].push_back(payload(s, t, c));
            for (int k = 0; k < kTopk; ++k) {
                idx[s].push_back(route(s, t, k));
                w[s].push_back(weight(s, t, k));
            }
        }
    }
    ABI(pcie_ep_peer_set_source(runtime, 1, x[1].data(), idx[1].data(), w[1].data(), kTokens));
    ABI(pcie_ep_peers_start(runtime, 1, 1u));

    const size_t n = size_t(sizes.unique_rows), m = size_t(sizes.expanded_rows);
    pcie_ep_dispatch_args args{};
    auto* dx = device_array<uint16_t>(size_t(kTokens) * kHidden);
    auto* didx = device_array<int64_t>(size_t(kTokens) * kTopk);
    auto* dw = device_array<float>(size_t(kTokens) * kTopk);
    HIP(hipMemcpy(dx, x[0].data(), x[0].size() * 2, hipMemcpyHostToDevice));
    HIP(hipMemcpy(didx, idx[0].data(), idx[0].size() * 8, hipMemcpyHostToDevice));
    HIP(hipMemcpy(dw, w[0].data(), w[0].size() * 4, hipMemcpyHostToDevice));
    args.x = dx;
    args.topk_idx = didx;
    args.topk_weights = dw;
    args.num_tokens = kTokens;
    args.alignment = 1;
    args.expand = 1;
    args.plan = device_array<char>(size_t(sizes.plan_bytes));
    args.unique_payload = device_array<uint16_t>(n * kHidden);
    args.unique_topk_idx = device_array<int64_t>(n * kTopk);
    args.unique_topk_weights = device_array<float>(n * kTopk);
    args.unique_source_meta = device_array<int64_t>(n * 3);
    args.unique_expert_ordinals = device_array<int32_t>(n * kTopk);
    auto* rows = device_array<uint16_t>(m * kHidden);
    auto* row_expert = device_array<int64_t>(m);
    auto* row_weight = device_array<float>(m);
    auto* row_meta = device_array<int64_t>(m * 3);
    args.expanded_payload = rows;
    args.expanded_expert_idx = row_expert;
    args.expanded_weights = row_weight;
    args.expanded_source_meta = row_meta;
    args.expanded_capacity_rows = int64_t(m);
    args.unique_count = device_array<int64_t>(1);
    args.expanded_count = device_array<int64_t>(1);
    args.expert_prefix = device_array<int32_t>(kLocal);
    args.expert_counts = device_array<int32_t>(kLocal);
    args.expert_offsets = device_array<int32_t>(kLocal + 1);
    args.source_offsets = device_array<int32_t>(kRanks + 1);
    args.source_expert_prefix = device_array<int32_t>(kRanks * kLocal);
    args.errors = device_array<int64_t>(8);
    args.stats = device_array<int64_t>(8);
    args.transport_timestamps_ns = device_array<int64_t>(2);
    args.expected_receive_counts = device_array<int32_t>(size_t(config.channels) * kRanks);
    args.channel_stats = device_array<int64_t>(size_t(config.channels) * 8);
    args.channel_timestamps_ns = device_array<int64_t>(size_t(config.channels) * 2);
    args.receive_expand_overlap = device_array<int64_t>(size_t(config.channels) * 2);
    args.receive_prefix_state = device_array<uint64_t>(2);
    args.prefix_tx_timestamps_ns = device_array<int64_t>(size_t(config.channels + 1) * 2);

    hipStream_t stream = nullptr;
    HIP(hipStreamCreate(&stream));
    ABI(pcie_ep_dispatch(runtime, &args, stream));
    HIP(hipStreamSynchronize(stream));
    ABI(pcie_ep_peers_wait(runtime, 10000));

    // ---- expected result, evaluated directly ------------------------------------------
    struct Row { int source, token, branch, expert; };
    std::vector<Row> expected;
    std::vector<int> counts(kLocal, 0), offsets(kLocal + 1, 0);
    for (int e = 0; e < kLocal; ++e) {
        offsets[e] = int(expected.size());
        for (int s = 0; s < kRanks; ++s)
            for (int t = 0; t < kTokens; ++t)
                for (int k = 0; k < kTopk; ++k)
                    if (route(s, t, k) == e) {  // rank 0 owns experts 0 .. kLocal-1
                        expected.push_back({s, t, k, e});
                        ++counts[e];
                    }
    }
    offsets[kLocal] = int(expected.size());
    int unique[kRanks] = {0, 0}, sent_to_peer = 0;
    for (int s = 0; s < kRanks; ++s)
        for (int t = 0; t < kTokens; ++t) {
            bool local = false, remote = false;
            for (int k = 0; k < kTopk; ++k) {
                const int64_t e = route(s, t, k);
                if (e >= 0 && e < kLocal) local = true;
                if (e >= kLocal) remote = true;
            }
            unique[s] += local;
            if (s == 0) sent_to_peer += remote;
        }

    const auto errors = to_host(args.errors, 8);
    CHECK(errors[0] == 0, "device error %lld", static_cast<long long>(errors[0]));
    CHECK(to_host(args.unique_count, 1)[0] == unique[0] + unique[1], "unique_count");
    CHECK(to_host(args.expanded_count, 1)[0] == int64_t(expected.size()), "expanded_count");
    const auto got_counts = to_host(args.expert_counts, kLocal);
    const auto got_offsets = to_host(args.expert_offsets, kLocal + 1);
    const auto got_sources = to_host(args.source_offsets, kRanks + 1);
    for (int e = 0; e < kLocal; ++e) CHECK(got_counts[e] == counts[e] && got_offsets[e] == offsets[e], "expert %d counts/offsets", e);
    CHECK(got_offsets[kLocal] == offsets[kLocal], "expert_offsets end");
    CHECK(got_sources[0] == 0 && got_sources[1] == unique[0] && got_sources[2] == unique[0] + unique[1], "source_offsets");
    const auto got_rows = to_host(rows, expected.size() * kHidden);
    const auto got_expert = to_host(row_expert, expected.size());
    const auto got_weight = to_host(row_weight, expected.size());
    const auto got_meta = to_host(row_meta, expected.size() * 3);
    for (size_t r = 0; r < expected.size(); ++r) {
        const Row& want = expected[r];
        CHECK(got_expert[r] == want.expert, "row %zu expert", r);
        CHECK(got_meta[r * 3] == want.source && got_meta[r * 3 + 1] == want.token && got_meta[r * 3 + 2] == want.branch, "row %zu source_meta", r);
        const float expected_weight = weight(want.source, want.token, want.branch);
        CHECK(std::memcmp(&got_weight[r], &expected_weight, 4) == 0, "row %zu weight", r);
        for (int c = 0; c < kHidden; ++c)
            CHECK(got_rows[r * kHidden + c] == payload(want.source, want.token, c), "row %zu column %d payload", r, c);
    }
    const auto stats = to_host(args.stats, 8);
    CHECK(stats[0] == sent_to_peer && stats[1] == unique[1], "stats: writes %lld reads %lld", static_cast<long long>(stats[0]),
          static_cast<long long>(stats[1]));
    int64_t captured = -1;
    ABI(pcie_ep_peer_captured_count(runtime, 1, &captured));
    CHECK(captured == sent_to_peer, "peer received %lld rows, expected %d", static_cast<long long>(captured), sent_to_peer);

    ABI(pcie_ep_runtime_destroy(runtime));
    std::printf("abi_client ok: %zu expanded rows, %d + %d unique rows, %d rows sent to the peer\n", expected.size(), unique[0], unique[1],
                sent_to_peer);
    return 0;
}

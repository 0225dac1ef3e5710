// Publication / acknowledgement litmus on pinned, fine-grained host memory.
//
// The whole dispatch rests on one hand-off: a writer stores a payload into
// mapped host memory, waits for its own stores, and then stores a sequence
// word; a reader that has seen the sequence word reads the payload and must
// find all of it.  The reference checks that discipline between two GPUs with
// a stand-alone program (tests/mapped_litmus.cu, tests/MAPPED_LITMUS.md: one
// payload slot, READY and ACK words 128 bytes apart, sequences from 1, a delay
// on the last thread to widen the window, a million round trips).  This is the
// same experiment for one MI355X and the host: the other end of the slot is a
// CPU thread, and the GPU end uses exactly the access primitives of the
// transport kernel (device_common.h) - buffer stores and loads with the
// system-scope cache policy, s_waitcnt on the wave's own operations, relaxed
// system-scope loads and stores of the sequence words - not acquire/release
// fences, which the hot path avoids.
//
//   mode 0  a wavefront produces, the CPU consumes   (TX worker -> peer)
//   mode 1  a workgroup of four wavefronts produces: every writer waits for its
//           own stores, the workgroup joins, the leader publishes
//           (publish_counts -> peer)
//   mode 2  the CPU produces, a wavefront consumes    (peer -> RX worker)
//   mode 3  the CPU produces, a workgroup consumes
//   mode 4  a wavefront produces, a wavefront of ANOTHER kernel on another stream
//           consumes                                  (TX worker -> RX worker of a peer
//           GPU: the hand-off a deployment performs, and the reference's experiment
//           proper - both ends are kernels, the slot lies in host memory between them)
//   mode 5  a workgroup produces, a workgroup of another kernel consumes
//   mode 0, 1, 4 or 5 with flag 16: negative control - the producer publishes the
//           sequence word WITHOUT waiting for its payload stores.  On an idle link
//           posted writes of one compute unit arrive in order and nothing shows; with
//           other traffic on the link the CPU finds words of an earlier round within
//           thousands of rounds.  It shows that the experiment can fail, and that
//           the wait it drops is needed, not merely sufficient.
// The two kernels of modes 4 and 5 run on two streams with disjoint compute-unit
// masks, which have hardware queues of their own (two ordinary streams may be put
// on one queue, one kernel behind the other, and the first would wait in vain).
// One slot, strict alternation: the producer waits for ACK == sequence before
// it overwrites the payload.  Every wait is bounded; a side that fails raises
// the abort word the other side polls, so the kernel always ends.
#include <atomic>
#include <chrono>
#include <cstring>

#include <string>

#include "../../include/pcie_ep_amd.h"
#include "device_common.h"
#include "launch.h"

namespace pcie_ep {

namespace {

constexpr int kLitmusOk = 0, kLitmusReadyTimeout = 1, kLitmusAckTimeout = 2, kLitmusPeerAborted = 3, kLitmusMismatch = 4;

struct LitmusShared {
    char* payload;        // mapped host memory, `vectors` 16-byte vectors
    uint64_t* ready;      // host: 128-byte separated sequence words
    uint64_t* ack;
    uint64_t* abort_word;
    int64_t* result;      // device memory: code, iteration, vector index
    int64_t iterations;
    int vectors;
    uint64_t writer_delay_ticks, reader_delay_ticks, timeout_ticks;
};

// What vector `index` of the payload holds in round `sequence`: every 32-bit
// word depends on both, so a stale vector of any earlier round is detected.
__host__ __device__ inline void litmus_pattern(uint64_t sequence, uint32_t index, uint32_t out[4]) {
    const uint32_t low = uint32_t(sequence), high = uint32_t(sequence >> 32);
    out[0] = low * 2654435761u ^ index;
    out[1] = (low + index * 40503u) ^ high;
    out[2] = ~low + index * 7u;
    out[3] = (index ^ 0xA5A5A5A5u) + low * 3u;
}

// Lane/thread 0 waits until `word` carries `sequence`; returns 0, or the failure code.
__device__ int litmus_wait(const LitmusShared& s, const uint64_t* word, uint64_t sequence, int timeout_code) {
    const uint64_t start = now_ticks();
    while (host_load(word) != sequence) {
        if (host_load(s.abort_word) != 0) return kLitmusPeerAborted;
        if (now_ticks() - start > s.timeout_ticks) return timeout_code;
        backoff();
    }
    return kLitmusOk;
}

__device__ void litmus_fail(const LitmusShared& s, int code, int64_t iteration, int64_t index) {
    s.result[0] = code;
    s.result[1] = iteration;
    s.result[2] = index;
    // Tell the CPU side (it polls this word in its own waits).
    host_store_release(s.abort_word, uint64_t(code));
}

template <bool kWorkgroup, bool kPublishEarly>
__global__ void __launch_bounds__(kRowKernelThreads) litmus_producer_kernel(LitmusShared s) {
    __shared__ int verdict;
    const int thread = threadIdx.x, threads = blockDim.x;
    const __amdgpu_buffer_rsrc_t slot = host_resource(s.payload, uint32_t(s.vectors) * 16u);
    for (int64_t round = 1; round <= s.iterations; ++round) {
        // The last thread stores late: the others' stores are long acknowledged
        // when its own go out, which the leader's publication must still cover.
        if (thread == threads - 1) test_delay(s.writer_delay_ticks);
        for (int index = thread; index < s.vectors; index += threads) {
            uint32_t words[4];
            litmus_pattern(uint64_t(round), uint32_t(index), words);
            host_store_b128(slot, uint32_t(index) * 16u, u32x4{words[0], words[1], words[2], words[3]});
        }
        // Every writer waits for its own stores (the counters are wave-wide);
        // across wavefronts the join carries that to the leader.
        if (!kPublishEarly) wait_memory_ops();
        if (kWorkgroup) __syncthreads();
        int code = kLitmusOk;
        if (thread == 0) {
            if (kPublishEarly) __hip_atomic_store(s.ready, uint64_t(round), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            else host_store_release(s.ready, uint64_t(round));
            code = litmus_wait(s, s.ack, uint64_t(round), kLitmusAckTimeout);
            if (code) litmus_fail(s, code, round, -1);
        }
        if (kWorkgroup) {
            if (thread == 0) verdict = code;
            __syncthreads();
            code = verdict;
            __syncthreads();
        } else {
            code = broadcast_first(code);
        }
        if (code) return;
    }
}

template <bool kWorkgroup>
__global__ void __launch_bounds__(kRowKernelThreads) litmus_consumer_kernel(LitmusShared s) {
    __shared__ int verdict;
    __shared__ int first_bad;
    const int thread = threadIdx.x, threads = blockDim.x;
    const __amdgpu_buffer_rsrc_t slot = host_resource(s.payload, uint32_t(s.vectors) * 16u);
    for (int64_t round = 1; round <= s.iterations; ++round) {
        int code = kLitmusOk;
        if (thread == 0) {
            code = litmus_wait(s, s.ready, uint64_t(round), kLitmusReadyTimeout);
            if (code) litmus_fail(s, code, round, -1);
            first_bad = 0x7FFFFFFF;
        }
        // The payload loads below are issued after the sequence word has been seen:
        // the leader's load has returned, and the others learn it through the join
        // (or, inside one wavefront, through the broadcast of its value).
        if (kWorkgroup) {
            if (thread == 0) verdict = code;
            __syncthreads();
            code = verdict;
        } else {
            code = broadcast_first(code);
        }
        if (code) return;
        if (thread == threads - 1) test_delay(s.reader_delay_ticks);
        int bad = 0x7FFFFFFF;
        for (int index = thread; index < s.vectors; index += threads) {
            uint32_t words[4];
            litmus_pattern(uint64_t(round), uint32_t(index), words);
            const u32x4 seen = host_load_b128(slot, uint32_t(index) * 16u);
            if ((seen[0] != words[0] || seen[1] != words[1] || seen[2] != words[2] || seen[3] != words[3]) && index < bad) bad = index;
        }
        if (bad != 0x7FFFFFFF) atomicMin(&first_bad, bad);
        // Every reader's loads have returned before the slot is given back.
        wait_memory_ops();
        if (kWorkgroup) __syncthreads();
        else fence_lds();
        if (thread == 0) {
            if (first_bad != 0x7FFFFFFF) {
                code = kLitmusMismatch;
                litmus_fail(s, code, round, first_bad);
            } else {
                host_store_release(s.ack, uint64_t(round));
            }
        }
        if (kWorkgroup) {
            if (thread == 0) verdict = code;
            __syncthreads();
            code = verdict;
            __syncthreads();
        } else {
            code = broadcast_first(code);
        }
        if (code) return;
    }
}

using Clock = std::chrono::steady_clock;

// CPU end of the slot.  Sequence words through acquire / release atomics; the
// payload through ordinary accesses ordered by them.
struct HostSide {
    char* payload;
    std::atomic_ref<uint64_t> ready, ack, abort_word;
    int vectors;
    int timeout_ms;
    int wait(std::atomic_ref<uint64_t>& word, uint64_t sequence, int timeout_code) {
        const auto start = Clock::now();
        uint32_t spins = 0;
        while (word.load(std::memory_order_acquire) != sequence) {
            if (abort_word.load(std::memory_order_acquire) != 0) return kLitmusPeerAborted;
            if ((++spins & 0xFFF) == 0 && std::chrono::duration_cast<std::chrono::milliseconds>(Clock::now() - start).count() > timeout_ms)
                return timeout_code;
        }
        return kLitmusOk;
    }
};

}  // namespace

// Runs one litmus; returns 0 or a PCIE_EP_E_* code with `error` filled in.  The
// C entry point (pcie_ep_litmus, runtime.hip) validates nothing else.
int run_litmus(int device, int mode, int64_t iterations, int payload_bytes, int writer_delay_ns, int reader_delay_ns, int timeout_ms,
               pcie_ep_litmus_result* out, std::string& error) {
    const auto fail = [&](int code, const char* message) {
        error = message;
        return code;
    };
    const bool publish_early = (mode & 16) != 0;
    mode &= ~16;
    const bool both_kernels = mode == 4 || mode == 5;
    if (!out || mode < 0 || mode > 5 || (publish_early && (mode == 2 || mode == 3)) || iterations < 1 || payload_bytes < 16 || payload_bytes % 16 || payload_bytes > (1 << 24) ||
        writer_delay_ns < 0 || reader_delay_ns < 0 || timeout_ms < 1)
        return fail(PCIE_EP_E_INVALID, "bad litmus arguments");
    std::memset(out, 0, sizeof *out);
    if (hipSetDevice(device) != hipSuccess) return fail(PCIE_EP_E_HIP, "hipSetDevice failed");
    int clock_khz = 0;
    if (hipDeviceGetAttribute(&clock_khz, hipDeviceAttributeWallClockRate, device) != hipSuccess || clock_khz <= 0)
        return fail(PCIE_EP_E_HIP, "the device does not report its wall clock rate");
    // The same kind of memory as the segments: pinned, fine-grained, mapped.
    const size_t bytes = 4 * 128 + size_t(payload_bytes);
    char* host = nullptr;
    int64_t* result = nullptr;
    hipStream_t stream = nullptr, consumer_stream = nullptr;
    hipError_t status = hipHostMalloc(reinterpret_cast<void**>(&host), bytes, hipHostMallocCoherent | hipHostMallocMapped | hipHostMallocPortable);
    if (status == hipSuccess) std::memset(host, 0, bytes);
    // Two result records: [0..2] the kernel that the calling thread talks to (or the
    // consumer kernel), [3..5] the producer kernel of the kernel-to-kernel modes.
    if (status == hipSuccess) status = hipMalloc(reinterpret_cast<void**>(&result), 6 * sizeof(int64_t));
    if (status == hipSuccess) status = hipMemset(result, 0, 6 * sizeof(int64_t));
    if (status == hipSuccess && !both_kernels) status = hipStreamCreate(&stream);
    if (status == hipSuccess && both_kernels) {
        // Producer on the first half of the compute units, consumer on the second.
        int units = 0;
        status = hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device);
        if (status == hipSuccess && units < 2) return fail(PCIE_EP_E_INVALID, "the kernel-to-kernel litmus needs two compute units");
        uint32_t first[32] = {}, second[32] = {};
        const int words = (units + 31) / 32 < 32 ? (units + 31) / 32 : 32;
        for (int unit = 0; unit < units && unit < 1024; ++unit) (unit < units / 2 ? first : second)[unit / 32] |= 1u << (unit % 32);
        if (status == hipSuccess) status = hipExtStreamCreateWithCUMask(&stream, uint32_t(words), first);
        if (status == hipSuccess) status = hipExtStreamCreateWithCUMask(&consumer_stream, uint32_t(words), second);
    }
    int64_t host_result[3] = {0, 0, -1};
    double elapsed = 0.0;
    if (status == hipSuccess) {
        LitmusShared shared{};
        shared.ready = reinterpret_cast<uint64_t*>(host);
        shared.ack = reinterpret_cast<uint64_t*>(host + 128);
        shared.abort_word = reinterpret_cast<uint64_t*>(host + 256);
        shared.payload = host + 512;
        shared.result = result;
        shared.iterations = iterations;
        shared.vectors = payload_bytes / 16;
        shared.writer_delay_ticks = uint64_t(writer_delay_ns) * uint64_t(clock_khz) / 1000000ull;
        shared.reader_delay_ticks = uint64_t(reader_delay_ns) * uint64_t(clock_khz) / 1000000ull;
        shared.timeout_ticks = uint64_t(timeout_ms) * uint64_t(clock_khz);
        const bool gpu_produces = mode < 2 || both_kernels, workgroup = (mode & 1) != 0;
        const dim3 grid(1), block(workgroup ? kRowKernelThreads : kWave);
        const auto start = Clock::now();
        if (both_kernels) {
            // The consumer first: it only waits; then the producer, with a result record of its own.
            if (workgroup) hipLaunchKernelGGL(litmus_consumer_kernel<true>, grid, block, 0, consumer_stream, shared);
            else hipLaunchKernelGGL(litmus_consumer_kernel<false>, grid, block, 0, consumer_stream, shared);
            status = hipGetLastError();
            shared.result = result + 3;
        }
        if (status != hipSuccess) {
        } else if (gpu_produces) {
            if (workgroup && publish_early) hipLaunchKernelGGL((litmus_producer_kernel<true, true>), grid, block, 0, stream, shared);
            else if (workgroup) hipLaunchKernelGGL((litmus_producer_kernel<true, false>), grid, block, 0, stream, shared);
            else if (publish_early) hipLaunchKernelGGL((litmus_producer_kernel<false, true>), grid, block, 0, stream, shared);
            else hipLaunchKernelGGL((litmus_producer_kernel<false, false>), grid, block, 0, stream, shared);
        } else {
            if (workgroup) hipLaunchKernelGGL(litmus_consumer_kernel<true>, grid, block, 0, stream, shared);
            else hipLaunchKernelGGL(litmus_consumer_kernel<false>, grid, block, 0, stream, shared);
        }
        if (status == hipSuccess) status = hipGetLastError();
        if (status == hipSuccess && both_kernels) {
            status = hipStreamSynchronize(stream);
            const hipError_t other = hipStreamSynchronize(consumer_stream);
            if (status == hipSuccess) status = other;
            elapsed = std::chrono::duration<double>(Clock::now() - start).count();
        } else if (status == hipSuccess) {
            HostSide side{shared.payload, std::atomic_ref<uint64_t>(*shared.ready), std::atomic_ref<uint64_t>(*shared.ack),
                          std::atomic_ref<uint64_t>(*shared.abort_word), shared.vectors, timeout_ms};
            auto* words = reinterpret_cast<volatile uint32_t*>(shared.payload);
            for (int64_t round = 1; round <= iterations && host_result[0] == 0; ++round) {
                if (gpu_produces) {
                    int code = side.wait(side.ready, uint64_t(round), kLitmusReadyTimeout);
                    for (int index = 0; index < shared.vectors && !code; ++index) {
                        uint32_t want[4];
                        litmus_pattern(uint64_t(round), uint32_t(index), want);
                        for (int word = 0; word < 4; ++word)
                            if (words[index * 4 + word] != want[word]) {
                                code = kLitmusMismatch;
                                host_result[2] = index;
                                break;
                            }
                    }
                    if (code) {
                        host_result[0] = code;
                        host_result[1] = round;
                        if (code != kLitmusPeerAborted) side.abort_word.store(uint64_t(code), std::memory_order_release);
                    } else {
                        side.ack.store(uint64_t(round), std::memory_order_release);
                    }
                } else {
                    for (int index = 0; index < shared.vectors; ++index) {
                        uint32_t value[4];
                        litmus_pattern(uint64_t(round), uint32_t(index), value);
                        for (int word = 0; word < 4; ++word) words[index * 4 + word] = value[word];
                    }
                    side.ready.store(uint64_t(round), std::memory_order_release);
                    const int code = side.wait(side.ack, uint64_t(round), kLitmusAckTimeout);
                    if (code) {
                        host_result[0] = code;
                        host_result[1] = round;
                        if (code != kLitmusPeerAborted) side.abort_word.store(uint64_t(code), std::memory_order_release);
                    }
                }
            }
            status = hipStreamSynchronize(stream);
            elapsed = std::chrono::duration<double>(Clock::now() - start).count();
        }
        int64_t device_result[6] = {0, 0, -1, 0, 0, -1};
        if (status == hipSuccess) status = hipMemcpy(device_result, result, sizeof device_result, hipMemcpyDeviceToHost);
        if (both_kernels) {
            // The producer kernel's verdict takes the place of the CPU side's.
            host_result[0] = device_result[3];
            host_result[1] = device_result[4];
            host_result[2] = device_result[3] ? device_result[5] : -1;
        }
        out->gpu_code = int32_t(device_result[0]);
        out->gpu_iteration = device_result[1];
        out->gpu_index = device_result[0] ? device_result[2] : -1;
        out->host_code = int32_t(host_result[0]);
        out->host_iteration = host_result[1];
        out->host_index = host_result[2];
        out->completed = (device_result[0] == 0 && host_result[0] == 0) ? iterations : 0;
        out->seconds = elapsed;
    }
    if (stream) (void)hipStreamDestroy(stream);
    if (consumer_stream) (void)hipStreamDestroy(consumer_stream);
    if (result) (void)hipFree(result);
    if (host) (void)hipHostFree(host);
    if (status != hipSuccess) return fail(PCIE_EP_E_HIP, hipGetErrorString(status));
    return 0;
}

}  // namespace pcie_ep

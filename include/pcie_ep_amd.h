/* C ABI of the MI355X host-staged expert-dispatch runtime.
 *
 * This is the drop-in boundary for the reference's native extension: every
 * entry point below names the reference interface it replaces (paths relative
 * to the reference checkout).  Signatures use plain pointers and sizes only;
 * device pointers are ordinary HIP device addresses and `stream` is a
 * `hipStream_t` passed as `void*`.
 *
 * Error convention: functions returning `int` return 0 on success and a
 * negative `PCIE_EP_E_*` code otherwise; `pcie_ep_last_error()` then holds a
 * message whose text mirrors the reference's `TORCH_CHECK` messages so that a
 * binding can raise the same exception types.  Device-side protocol errors are
 * never reported here: they land in the `errors[8]` output array with the
 * reference's numeric codes (csrc/kernels/host_staged/common.cuh:26-38).
 */
#ifndef PCIE_EP_AMD_H
#define PCIE_EP_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PCIE_EP_ABI_VERSION 2

#define PCIE_EP_E_INVALID (-1)   /* bad argument / unsupported dimensions (ValueError / RuntimeError) */
#define PCIE_EP_E_HIP (-2)       /* a HIP runtime call failed */
#define PCIE_EP_E_STATE (-3)     /* runtime closed, or call not legal in this state */
#define PCIE_EP_E_TIMEOUT (-4)   /* a host-side wait timed out */
#define PCIE_EP_E_PROTOCOL (-5)  /* the host peer emulator observed a protocol violation */

typedef struct pcie_ep_runtime pcie_ep_runtime;

/* Replaces the (directory, rank, p, t, h, k, e, options) constructor arguments
 * of AdvancedRuntime (csrc/buffers/advanced.hpp:107) and the option dict parsed
 * by AdvancedConfig (csrc/comm/advanced_shared_memory.hpp:55-112). */
typedef struct pcie_ep_config {
    int32_t num_ranks;          /* P logical ranks, 1..16 */
    int32_t local_rank;         /* the rank this GPU plays */
    int32_t max_tokens;         /* num_max_tokens_per_rank */
    int32_t hidden;
    int32_t topk;               /* 1..32 */
    int32_t num_experts;        /* divisible by num_ranks, <= 4096 */
    int32_t channels;           /* 1..32 */
    int32_t payload_slots;      /* Q per channel */
    int32_t descriptor_slots;   /* L per (channel, destination) */
    int32_t wire_fp8;           /* 0 BF16 wire, 1 E4M3FN + FP32 scale per token */
    int32_t timeout_ms;         /* device-side protocol timeout */
    int32_t fuse_receive_expand;/* 1: receive waves scatter to expert rows; 0: unique rows + expand kernel */
    int32_t tx_waves;           /* tx_waves + rx_waves = payload wavefronts per payload workgroup, 0 = default (2 each). */
    int32_t rx_waves;           /* The kernel decides row by row which direction a wavefront serves; the two values only add up. */
    int32_t peer_threads;       /* host threads standing in for the other ranks; 0 = none */
    int32_t staging_numa_node;  /* NUMA node for the pinned segments, -1 = first touch */
    int32_t device;             /* HIP device ordinal */
    int32_t worker_groups;      /* payload workgroups of the transport kernel, spread over the XCDs;
                                   0 = default (as many as keep 2.7 MB of rows in flight: 48 for 14 KB rows, at most 96),
                                   -1 = none (control workgroups move the rows) */
    int32_t receive_expand_mode;/* 0 pipelined, 1 vectorized, 2 scalar (pcie_ep/config.py:58-60): selects what the
                                   receive_expand_overlap diagnostic holds, the rows are moved the same way */
    int32_t numa_mode;          /* 0 direct; 1 relay: ranks on another NUMA domain are reached through host relay
                                   workers and replica rings (csrc/comm/numa_relay.hpp) */
    int32_t replica_slots;      /* R per (channel, NUMA domain), relay mode */
    int32_t relay_workers_per_numa; /* host relay threads per NUMA domain, 1..channels */
    int32_t relay_cpu_count;    /* entries of relay_cpus in use; 0 = any CPU the process may run on */
    int32_t split_launch;       /* 0: one launch per dispatch where the prologue fits into the transport launch (top-k <= 8, default
                                   launch shape, at most 64 chunks of 256 tokens); 1: always a prologue launch of its own */
    int32_t reserved[4];
    int32_t rank_numa_nodes[16];/* physical NUMA node of every rank, -1 = unknown (one domain) */
    int32_t relay_cpus[64];     /* CPUs the relay workers may be pinned to */
    uint64_t relay_delay_ns;    /* test hook: delay before each relay copy */
} pcie_ep_config;

/* Capacities and byte sizes a caller needs to allocate pools
 * (csrc/buffers/advanced.hpp:296-326, :21-41). */
typedef struct pcie_ep_sizes {
    int64_t unique_rows;        /* P * Tmax */
    int64_t expanded_rows;      /* unique_rows * min(K, E/P) + (E/P) * 255 */
    int64_t plan_bytes;         /* one route-plan blob */
    int64_t segment_bytes;      /* one pinned source segment */
    int64_t slot_stride;        /* bytes between payload slots */
    int32_t local_experts;
    int32_t payload_bytes;      /* wire bytes of one row */
    int32_t meta_bytes;         /* per-slot token metadata bytes */
    int32_t mailbox_dwords;
    int32_t transport_threads;  /* workgroup size of the transport kernel */
    int32_t transport_workgroups; /* control + payload workgroups; 1..32 more do the local bypass */
    int32_t num_domains;        /* NUMA domains of a relay configuration, 0 in direct mode */
    int32_t reserved[3];
    int64_t replica_region_bytes; /* one replica payload region (per rank and domain), relay mode */
} pcie_ep_sizes;

/* One dispatch: inputs, the route plan to fill or reuse, and every output of
 * one result pool.  Field-for-field the tensors AdvancedRuntime binds in
 * bind_state (csrc/buffers/advanced.hpp:420-470).  All pointers are device
 * pointers that stay valid until the stream has executed the dispatch. */
typedef struct pcie_ep_dispatch_args {
    const void* x;                   /* bf16 [T, H] */
    const int64_t* topk_idx;         /* [T, K] global expert ids, -1 unused */
    const float* topk_weights;       /* [T, K] or NULL */
    int32_t num_tokens;              /* T <= max_tokens */
    int32_t alignment;               /* 1..256 */
    int32_t expand;                  /* do_expand */
    int32_t zero_padding;
    int32_t reuse_plan;              /* 1: `plan` already holds this routing (cached layout) */
    int32_t reserved0;
    void* plan;                      /* plan_bytes */
    void* unique_payload;            /* bf16 [unique_rows, H] */
    int64_t* unique_topk_idx;        /* [unique_rows, K] */
    float* unique_topk_weights;      /* [unique_rows, K] */
    int64_t* unique_source_meta;     /* [unique_rows, 3] */
    int32_t* unique_expert_ordinals; /* [unique_rows, K] */
    void* expanded_payload;          /* bf16 [expanded_rows, H] */
    int64_t* expanded_expert_idx;    /* [expanded_rows] */
    float* expanded_weights;         /* [expanded_rows] */
    int64_t* expanded_source_meta;   /* [expanded_rows, 3] */
    int64_t* unique_count;           /* [1] */
    int64_t* expanded_count;         /* [1] */
    int32_t* expert_prefix;          /* [E/P] */
    int32_t* expert_counts;          /* [E/P] */
    int32_t* expert_offsets;         /* [E/P + 1] */
    int32_t* source_offsets;         /* [P + 1] */
    int32_t* source_expert_prefix;   /* [P, E/P] */
    int64_t* errors;                 /* [8] */
    int64_t* stats;                  /* [8] */
    int64_t* transport_timestamps_ns;/* [2] */
    int32_t* expected_receive_counts;/* [C, P] */
    int64_t* channel_stats;          /* [C, 8] */
    int64_t* channel_timestamps_ns;  /* [C, 2] */
    int64_t* receive_expand_overlap; /* [C, 2] */
    uint64_t* receive_prefix_state;  /* [2] */
    int64_t* prefix_tx_timestamps_ns;/* [C + 1, 2] */
    int64_t expanded_capacity_rows;  /* rows actually allocated for expanded_* */
} pcie_ep_dispatch_args;

int pcie_ep_abi_version(void);

/* Pure host arithmetic, usable without a GPU.  Replaces the capacity formulas
 * of allocate_workspace (advanced.hpp:296-298) and the segment size of
 * make_advanced_shared_memory_layout (advanced_common.cuh:42-84). */
int pcie_ep_query_sizes(const pcie_ep_config* config, pcie_ep_sizes* sizes);

/* Replaces create_advanced_segments + prepare_advanced_segment +
 * AdvancedRuntime::AdvancedRuntime (csrc/comm/advanced_shared_memory.hpp:143-212,
 * csrc/buffers/advanced.hpp:107-124): allocates and zeroes the P pinned
 * fine-grained host segments, the device workspace and, when
 * `peer_threads > 0`, the host peer emulator. */
int pcie_ep_runtime_create(const pcie_ep_config* config, pcie_ep_runtime** runtime);

/* The pinned segments of a whole EP world as a set that several runtimes share:
 * one segment per rank (pcie_ep_sizes.segment_bytes each) and, in relay mode, the
 * replica payload regions [rank * 8 + domain] (pcie_ep_sizes.replica_region_bytes
 * each).  Pointers are what the GPU uses (for pinned, mapped host memory the host
 * address).  Replaces the set of /dev/shm segments a rank creates and its peers
 * map (create_advanced_segments / AdvancedSharedMemory,
 * csrc/comm/advanced_shared_memory.hpp:143-233). */
typedef struct pcie_ep_segments {
    void* segment[16];
    void* replica[16 * 8];
} pcie_ep_segments;

/* Allocates (pinned, fine-grained, GPU-mapped, zeroed; NUMA placement as
 * pcie_ep_runtime_create does it) and frees such a set in this process. */
int pcie_ep_segments_create(const pcie_ep_config* config, pcie_ep_segments* segments);
int pcie_ep_segments_destroy(pcie_ep_segments* segments);

/* pcie_ep_runtime_create for rank `config->local_rank` on segments it does not
 * own: every other rank of `segments` is a runtime of its own (another stream,
 * another process that mapped the same memory, another GPU), so `peer_threads`
 * must be 0 and no emulator is started.  The set must outlive the runtime and
 * must have been zeroed before its first user.  Replaces the attach path of the
 * reference's runtime (attach_advanced_segments / register_advanced_segments,
 * csrc/comm/advanced_shared_memory.hpp:235-288; its use by the constructor,
 * csrc/buffers/advanced.hpp:107-124). */
int pcie_ep_runtime_attach(const pcie_ep_config* config, const pcie_ep_segments* segments, pcie_ep_runtime** runtime);

/* Replaces AdvancedRuntime::close (advanced.hpp:229-240).  The caller must have
 * synchronised every stream that ran a dispatch. */
int pcie_ep_runtime_destroy(pcie_ep_runtime* runtime);

/* Replaces AdvancedRuntime::dispatch / launch_dispatch (advanced.hpp:126-156,
 * :472-523): enqueues the dispatch kernels on `stream`, never synchronises and
 * never allocates, so it may be called under stream capture.  Dispatches of one
 * runtime share its epoch, ticket rings and scratch: they must execute one after
 * the other (same stream, or streams ordered by events), and calls on one
 * runtime must not be made from two threads at once (the reference serialises
 * submissions the same way: pcie_ep/buffers/ep.py:101, :283). */
int pcie_ep_dispatch(pcie_ep_runtime* runtime, const pcie_ep_dispatch_args* args, void* stream);

/* The same dispatch with the transport scratch (ticket queues, prologue chunk
 * flags and records, ring history) taken from a fixed array in the library's
 * device image instead of the runtime's own allocations.  No counterpart in the
 * reference: it is for callers that cannot allocate device memory or do not want
 * a runtime's scratch allocations in their address map (code under graph
 * capture, serving loops, harnesses that forbid hipMalloc).  It calls no
 * allocating routine.  Limits: the scratch a configuration needs (about 0.4 MB at
 * the defaults; it grows with max_tokens and num_experts) must fit the 4 MiB
 * array, otherwise PCIE_EP_E_INVALID.  Every runtime on one GPU shares that GPU's
 * array and each call clears the part that must start at zero, so calls of
 * different runtimes that overlap in time on one GPU race; per-kernel timing
 * (pcie_ep_set_kernel_timing) is not recorded by this entry point. */
int pcie_ep_dispatch_static_scratch(pcie_ep_runtime* runtime, const pcie_ep_dispatch_args* args, void* stream);

/* Residency of the transport kernel on `compute_units` compute units (0 = the whole
 * device): `needed` = control + payload workgroups of one dispatch, which wait for
 * each other through device memory and must therefore all be running at once;
 * `resident` = workgroups of that kernel the units hold together (occupancy of the
 * kernel times the units).  A caller that confines the dispatch stream to a
 * compute-unit mask must keep resident >= needed, otherwise every dispatch ends
 * with device code 15 after the timeout.  No counterpart in the reference (its
 * kernels take `num_sms`-style footprints on trust). */
int pcie_ep_transport_residency(pcie_ep_runtime* runtime, int32_t compute_units, int32_t* needed, int32_t* resident);

/* Thread-local message of the last failing call (runtime may be NULL). */
const char* pcie_ep_last_error(void);

/* Test-only hooks (advanced.hpp:158-180; csrc/runtime.cu:23-27). */
int pcie_ep_set_test_delays(pcie_ep_runtime* runtime, uint64_t metadata_ns, uint64_t tx_ns, uint64_t rx_ns, uint64_t scatter_ns);
int pcie_ep_set_test_prefix_delay_ns(pcie_ep_runtime* runtime, uint64_t delay_ns);
int pcie_ep_set_test_control_abort_after_ns(pcie_ep_runtime* runtime, uint64_t delay_ns);
int pcie_ep_set_test_skip_counts_ack_source(pcie_ep_runtime* runtime, int32_t source);
/* Overwrite the device-side epoch counter (synchronises the device).  Only for
 * testing epoch exhaustion (error 20 once the epoch would reach 2^32:
 * csrc/kernels/host_staged/advanced_layout.cuh:44-48); no counterpart in the
 * reference, which has no test of that path. */
int pcie_ep_set_test_epoch(pcie_ep_runtime* runtime, uint64_t epoch);

/* ---- NUMA relay (numa_mode = 1) ------------------------------------------- */

/* One (channel, domain) flow of this rank's relay workers; the per-flow record
 * of NumaRelay::diagnostics (csrc/comm/numa_relay.hpp:133-175). */
typedef struct pcie_ep_relay_flow {
    int32_t channel;
    int32_t numa_domain;
    int32_t worker;             /* index of the worker thread that owns the flow */
    int32_t cpu;                /* CPU that worker is pinned to, -1 = not pinned */
    int32_t expected_tokens;    /* rows the flow carries in `epoch` */
    int32_t error;              /* 0, or 101..106 (also stored in relay_failed) */
    uint64_t epoch;
    uint64_t copied_tokens;     /* in `epoch` */
    uint64_t copied_payload_bytes;
    uint64_t copy_time_ns_total;
    uint64_t credit_wait_probes_total;
    uint64_t drained_epoch;     /* relay_drained[channel][domain] */
    uint64_t copies_total;      /* since creation */
    uint64_t payload_bytes_total;
} pcie_ep_relay_flow;

/* The per-runtime part of AdvancedRuntime::relay_diagnostics (advanced.hpp:182-213). */
typedef struct pcie_ep_relay_summary {
    int32_t enabled;
    int32_t rank;
    int32_t num_domains;
    int32_t workers;
    int32_t flows;              /* flows that exist; at most `capacity` records were written */
    int32_t source_page_node;   /* node a sampled page of this rank's payload slots resides on, or -errno */
    int32_t rank_numa_nodes[16];
    int32_t domain_numa_nodes[8];   /* physical node of every domain */
    int32_t domain_bound[8];        /* 1: that node exists here and the domain's replica regions were bound to it */
    int32_t replica_page_node[8];   /* node a sampled page of this rank's replica region of the domain resides on, or -errno */
    uint64_t epoch;             /* this rank's counts_ready */
    uint64_t copies;            /* rows copied in `epoch`, all flows */
    uint64_t payload_bytes;     /* payload bytes copied in `epoch` (metadata and scales excluded) */
    uint64_t copies_total;
    uint64_t payload_bytes_total;
    int64_t slot_stride;
    int64_t segment_bytes;
    int64_t replica_region_bytes;
} pcie_ep_relay_summary;

/* Replaces AdvancedRuntime::relay_diagnostics (advanced.hpp:182-213; csrc/runtime.cu:22).
 * `flows` may be NULL when capacity is 0.  With numa_mode = 0 only `enabled`,
 * `rank` and the sizes are filled. */
int pcie_ep_relay_diagnostics(pcie_ep_runtime* runtime, pcie_ep_relay_summary* summary, pcie_ep_relay_flow* flows, int32_t capacity);
/* Replaces AdvancedRuntime::set_relay_delay_ns (advanced.hpp:164-167; csrc/runtime.cu:27):
 * test hook, delays every relay copy of this rank.  PCIE_EP_E_STATE when the relay is not enabled. */
int pcie_ep_set_relay_delay_ns(pcie_ep_runtime* runtime, uint64_t delay_ns);

/* Replaces get_device_numa_node (advanced_shared_memory.hpp:120-131). */
int pcie_ep_device_numa_node(int32_t device);

/* Host-visible protocol words, for failure tests that force a condition from
 * the CPU (the reference's destructor does the same store: advanced.hpp:258-261).
 * which: 0 abort, 1 channel_abort[index], 2 counts_ready, 3 counts_consumed[index],
 * 4 relay_failed[index], 5 relay_drained[index] (relay mode; index = channel * domains + domain). */
int pcie_ep_host_signal_store(pcie_ep_runtime* runtime, int32_t segment_rank, int32_t which, int32_t index, uint64_t value);
int pcie_ep_host_signal_load(pcie_ep_runtime* runtime, int32_t segment_rank, int32_t which, int32_t index, uint64_t* value);

/* ---- Stand-alone kernels (same device code the dispatch uses) ------------ */

/* Replaces quantize_transport_payload (csrc/kernels/host_staged/quantization.cuh:34-71):
 * bf16 [T,H] -> E4M3FN codes [T,H] + FP32 scale [T]. */
int pcie_ep_quantize_fp8(const void* x, uint8_t* codes, float* scales, int32_t tokens, int32_t hidden, void* stream);
/* Replaces dequantize_fp8_to_bf16 (quantization.cuh:21-24) over whole rows. */
int pcie_ep_dequantize_fp8(const uint8_t* codes, const float* scales, void* out, int32_t tokens, int32_t hidden, void* stream);
/* Replaces scatter_expert_inputs (csrc/kernels/host_staged/dispatch.cuh:8-65): expands
 * the unique rows of `args` into its expert-major outputs using the prefixes
 * already present in `args` (what a non-fused dispatch launches last). */
int pcie_ep_expand_unique(pcie_ep_runtime* runtime, const pcie_ep_dispatch_args* args, void* stream);

/* Launches an instantiated HIP graph (a hipGraphExec_t, e.g. the one a captured
 * dispatch was turned into) on `stream`.  For hosts whose graph object can only
 * replay on "the current stream" of their framework: switching that stream around
 * every replay costs more CPU time than a small dispatch takes on the GPU.
 * No counterpart in the reference (its graph.py:150-202 replays through PyTorch). */
int pcie_ep_graph_launch(void* graph_exec, void* stream);

/* Per-kernel timing with HIP events recorded on the dispatch stream (off by
 * default; must stay off for a dispatch that is being captured into a graph).
 * pcie_ep_get_kernel_times waits for the last timed dispatch and returns the
 * milliseconds of {prologue, transport, separate expand or 0}; the prologue reads 0
 * where it rides in the transport launch (the default wherever it fits).
 * No counterpart in the reference (its harness wraps events around the whole
 * dispatch: benchmarks/benchmark.py:165-198). */
int pcie_ep_set_kernel_timing(pcie_ep_runtime* runtime, int32_t enable);
int pcie_ep_get_kernel_times(pcie_ep_runtime* runtime, float* milliseconds3);

/* Per-role timing records of the last dispatch, from a library built with
 * -DPCIE_EP_ENABLE_PROFILING=1 (`python pcie-ep_amd/build.py --profiling`; the default
 * build contains no profiling code and reports 0 rows).  Replaces the `profiling`
 * output tensor of the reference's PCIE_EP_ENABLE_PROFILING build
 * (csrc/kernels/host_staged/advanced_common.cuh:126-181; docs/pcie-ep/
 * profiling-instrumentation.md): one record of `fields` (32) int64 per role wavefront,
 * rows ordered TX control [0, C), RX control [C, 2C), payload wavefronts
 * [2C, 2C + W), prologue leader [2C + W], epoch begin [2C + W + 1], producer of the
 * receive prefixes [2C + W + 2] (the last two where they are roles of their own, else
 * zero); the field meanings are the ProfileField /
 * PrologueProfileField enums of csrc/device_common.h, mirrored in pcie_ep/profiling.py.
 * pcie_ep_profile_read synchronises the device (a diagnostic wait outside the dispatch
 * path, like the reference's handle.profiling.cpu()). */
int pcie_ep_profile_shape(pcie_ep_runtime* runtime, int32_t* rows, int32_t* fields, int32_t* channels, int32_t* payload_wavefronts);
int pcie_ep_profile_read(pcie_ep_runtime* runtime, int64_t* records);

/* Pinned-copy bandwidth of this box (GB/s, best of `repeats`), the denominator
 * for "% of x16 peak".  No counterpart in the reference. */
int pcie_ep_measure_pinned_copy(int32_t device, int64_t bytes, int32_t repeats, double* h2d_gbps, double* d2h_gbps);
/* The same between pinned host memory and HBM, but moved by a kernel with
 * `wavefronts` wavefronts in flight (16 KiB each) through the accesses the
 * transport kernel uses for host slots: what kernel-initiated traffic can reach
 * on the host link (host -> device reads, device -> host writes), and a kernel
 * of known host traffic for scaling counters.  No counterpart in the reference. */
int pcie_ep_measure_kernel_host_copy(int32_t device, int64_t bytes, int32_t repeats, int32_t wavefronts, double* read_gbps,
                                     double* write_gbps);
/* Read+write rate (GB/s, bytes read plus bytes written, best of `repeats`) of a
 * plain device-to-device copy of `bytes` (a multiple of 16) done by a kernel
 * with the row movers' access shape: the practical ceiling the expand kernel is
 * compared with, and a kernel of known traffic for scaling memory counters.
 * No counterpart in the reference. */
int pcie_ep_measure_device_copy(int32_t device, int64_t bytes, int32_t repeats, double* gbps);

/* Read+write rate (GB/s; best of three batches of `repeats` back-to-back launches) of the expand kernel's traffic shape
 * without its metadata: every wavefront reads one row of `row_bytes` and writes
 * it once, `extra_per_1024` of every 1024 rows twice.  pattern 0 writes in linear
 * order, 1 into `streams` interleaved sequential streams (what expert-major
 * placement of source-ordered rows produces), 2 hashed, 3 reads the rows only,
 * 4 writes them only (one row per wavefront each).  The practical HBM
 * ceiling for a write-heavy row scatter on this part.  No counterpart in the
 * reference. */
int pcie_ep_measure_row_scatter(int32_t device, int32_t rows, int32_t row_bytes, int32_t extra_per_1024, int32_t pattern, int32_t streams,
                                int32_t repeats, double* gbps);

/* Publication / acknowledgement litmus on the kind of memory the segments are
 * made of (pinned, fine-grained, mapped), with the access primitives of the
 * transport kernel: the experiment of the reference's stand-alone two-GPU
 * program (tests/mapped_litmus.cu, tests/MAPPED_LITMUS.md - one payload slot,
 * READY and ACK words 128 bytes apart, sequences from 1, a delayed last thread)
 * between this GPU and the calling CPU thread.  mode 0: one wavefront produces,
 * the CPU consumes; 1: a workgroup of four wavefronts produces; 2: the CPU
 * produces, one wavefront consumes; 3: a workgroup consumes; 4: one wavefront
 * produces and a wavefront of another kernel, on another stream, consumes (both
 * ends on the GPU, the slot in host memory between them: the hand-off between
 * two GPUs of a deployment, which is what the reference's program runs); 5: the
 * same between two workgroups.  In modes 4 and 5 the gpu_* fields are the
 * consumer kernel's verdict and the host_* fields the producer kernel's.  Every
 * round the consumer compares every word of the payload with what the round must
 * hold.  Mode 0, 1, 4 or 5 with PCIE_EP_LITMUS_PUBLISH_EARLY added is the negative control:
 * the producer publishes READY without waiting for its payload stores; with
 * other traffic on the host link the consumer then finds stale words (code 4),
 * which shows that the experiment can fail and that the wait is needed.
 * Codes: 0 passed, 1 READY timeout, 2 ACK timeout, 3 the other side gave up,
 * 4 payload mismatch (index = first bad 16-byte vector).  Every wait on either
 * side is bounded by timeout_ms, so the kernel always ends. */
#define PCIE_EP_LITMUS_PUBLISH_EARLY 16
typedef struct pcie_ep_litmus_result {
    int64_t completed;      /* rounds both sides completed without error (0 on any failure) */
    int32_t gpu_code;       /* what the GPU side found */
    int32_t host_code;      /* what the CPU side found */
    int64_t gpu_iteration;  /* round of the GPU side's failure */
    int64_t gpu_index;      /* vector of a mismatch the GPU side found, else -1 */
    int64_t host_iteration;
    int64_t host_index;
    double seconds;         /* wall clock of all rounds */
} pcie_ep_litmus_result;
int pcie_ep_litmus(int32_t device, int32_t mode, int64_t iterations, int32_t payload_bytes, int32_t writer_delay_ns, int32_t reader_delay_ns,
                   int32_t timeout_ms, pcie_ep_litmus_result* result);

/* ---- Host peer emulator ---------------------------------------------------
 * On one GPU the other logical ranks are host threads that follow the ring
 * protocol on the same pinned segments, the way the reference's CPU relay
 * workers do (csrc/comm/numa_relay.hpp:18-35, :240-340).  As sources they stage
 * payload, metadata, descriptors and counts for rows destined to the GPU's
 * rank; as receivers they consume the GPU's descriptors, optionally capture
 * the rows, and return ACKs and credits. */

/* Give rank `rank` (!= local_rank) its inputs for the following epochs; host
 * pointers, copied.  `weights` may be NULL (1.0 is sent, as the reference does:
 * advanced_dispatch.cuh:73).  tokens may be 0. */
int pcie_ep_peer_set_source(pcie_ep_runtime* runtime, int32_t rank, const void* x_bf16, const int64_t* topk_idx,
                            const float* weights, int32_t tokens);
/* Serve the next `epochs` dispatches.  flags: bit 0 capture the rows received
 * from the GPU; bit 1 stage every source slot afresh in every epoch (by default
 * a slot whose row did not change since it was last written is only
 * re-announced, so repeated epochs of one workload cause no host-memory writes
 * besides descriptors); bit 2 the emulated receivers read every byte of the
 * rows the GPU sent (by default they read the slot metadata only). */
int pcie_ep_peers_start(pcie_ep_runtime* runtime, int32_t epochs, uint32_t flags);
/* Block until every emulated source has staged all it can for the first
 * pending epoch without GPU progress (used to pre-stage before timing). */
int pcie_ep_peers_wait_staged(pcie_ep_runtime* runtime, int32_t timeout_ms);
/* Block until all started epochs are served; returns PCIE_EP_E_PROTOCOL /
 * PCIE_EP_E_TIMEOUT with a message on failure. */
int pcie_ep_peers_wait(pcie_ep_runtime* runtime, int32_t timeout_ms);
/* Abandon outstanding epochs (after a GPU-side failure). */
int pcie_ep_peers_cancel(pcie_ep_runtime* runtime);
/* Rows rank `rank` received from the GPU in the last served epoch: count, then
 * copies (row order = arrival order per channel; `tokens[i]` identifies the row).
 * payload is wire bytes [count, payload_bytes]; idx/ordinals/weights are [count, K]. */
int pcie_ep_peer_captured_count(pcie_ep_runtime* runtime, int32_t rank, int64_t* count);
int pcie_ep_peer_captured_copy(pcie_ep_runtime* runtime, int32_t rank, int32_t* tokens, int32_t* rank_ordinals,
                               uint8_t* payload, float* scales, int32_t* expert_idx, int32_t* expert_ordinals,
                               float* weights, uint32_t* destination_masks);
/* Force a protocol failure from the host.  fault: 1 withhold counts_ready,
 * 2 withhold counts_consumed, 3 withhold the last payload ACK, 4 publish a
 * wrong payload sequence, 5 send a unique-row ordinal beyond the announced
 * count, 6 send an expert ordinal beyond the announced count, 7 name a payload
 * slot beyond the ring in the descriptor (4-7 on the last row of every channel).  Applies to rank `rank` for the next started epochs;
 * fault 0 clears. */
int pcie_ep_peers_inject_fault(pcie_ep_runtime* runtime, int32_t rank, int32_t fault);

/* Host implementations the emulator uses, exposed so CPU tests can check them
 * against the oracle without a GPU. */
int pcie_ep_host_quantize_fp8(const void* x_bf16, uint8_t* codes, float* scales, int32_t tokens, int32_t hidden);
int pcie_ep_host_dequantize_fp8(const uint8_t* codes, const float* scales, void* out_bf16, int32_t tokens, int32_t hidden);
/* Route plan of one source on the host: mask [T], rank_ordinals [T,P],
 * expert_indices [T,K], expert_ordinals [T,K], counts [P+E]; returns 0, or 2
 * (the device error code) for invalid routing. */
int pcie_ep_host_source_layout(const int64_t* topk_idx, int32_t tokens, int32_t topk, int32_t num_ranks, int32_t num_experts,
                               uint32_t* mask, int32_t* rank_ordinals, int32_t* expert_indices, int32_t* expert_ordinals,
                               int32_t* counts);

#ifdef __cplusplus
}
#endif
#endif /* PCIE_EP_AMD_H */

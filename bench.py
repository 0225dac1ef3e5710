"""Benchmark of the host-staged dispatch on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tokens 8192] [--wire bf16|fp8] [--routing uniform|hotspot]

One step is one full dispatch of the receiver's share: the GPU is logical rank
0 of 8; its own T tokens go through the real TX path into the pinned host ring,
the 7 other sources are staged by host threads in the same rings and are read
once over PCIe and expanded into expert-major rows in HBM.  Inputs of the GPU's
own source are resident in HBM before the timed region; remote payloads are
resident in pinned host memory, which is where this transport has them by
definition (the host threads do not rewrite unchanged rows between the timed
steps: ``config.peer_restage`` is false; the ``restaged`` record repeats the
measurement with every slot rewritten and every sent row read back per step).

Prints ONE JSON line.  Top level: the headline workload (dispatch time and PCIe
payload rate against the measured pinned-copy peak, T=8192, H=7168, top-8, BF16
wire) with ``roofline`` (stand-alone expand kernel against HBM), ``pcie`` (the
transport kernel against the pinned hipMemcpy peak of the same run) and
``cpu_baseline`` (layout + expand in PyTorch on the host cores).  The default run
adds one compact record per further workload of the metric — ``fp8`` (FP8 wire,
heavy-tailed inputs), ``hotspot_top4``, ``t4096``, ``eager_small_t``
(T in 16..2048) and ``graph_replay_us`` (cached layout + hipGraph replay) —
each timed the same way and each with a ``parity`` flag from an untimed
dispatch checked bit for bit against the oracle.
"""

from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for entry in (ROOT, ROOT / "pcie-ep_amd", ROOT / "tests"):
    if str(entry) not in sys.path:
        sys.path.insert(0, str(entry))

WORLD, EXPERTS, HIDDEN = 8, 256, 7168
HBM_PEAK_GBPS = 8000.0
COPY_BYTES = 1 << 30  # calibration copy: 1 GiB read + 1 GiB written
HOST_COPY_BYTES = 1 << 29  # kernel-driven pinned copy: 512 MiB each way
BIT_EXACT = "bit-exact vs oracle"
SPLIT_LAUNCH = False  # --split-launch: the prologue as a kernel of its own in front of the transport kernel


def log(*items) -> None:
    print(*items, file=sys.stderr, flush=True)


def build_inputs(tokens: int, topk: int, routing: str, heavy_tail: bool):
    from helpers import baseline_inputs

    return baseline_inputs(tokens, topk, routing, heavy_tail, WORLD, EXPERTS, HIDDEN)


def make_buffer(tokens, topk, wire, channels, fuse, timeout_ms=30000, graph=False, peer_threads=None):
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    config = HostStagedConfig(channels=channels, stage=7 if wire == "fp8" else 6, wire_dtype="fp8_e4m3" if wire == "fp8" else "bf16",
                              fuse_receive_expand=fuse, receive_expand_mode="pipelined" if fuse else "scalar", timeout_ms=timeout_ms,
                              enable_graph=graph)
    return HostStagedEPBuffer(num_max_tokens_per_rank=tokens, hidden=HIDDEN, num_topk=topk, num_experts=EXPERTS, config=config,
                              num_ranks=WORLD, rank=0, split_launch=SPLIT_LAUNCH, peer_threads=peer_threads)


def set_peers(buffer, inputs):
    for source in range(1, WORLD):
        buffer.peers.set_source(source, *inputs[source])


def cpu_baseline(inputs, payload_bytes, budget_s=20.0, fp8=False):
    """Oracle-side layout+expand in PyTorch on the host cores (reported only)."""
    import torch

    from oracle import cpu_baseline as baseline

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    all_x, all_idx, all_w = zip(*inputs)
    sample_tokens = all_x[0].shape[0]
    sample = "full workload"
    started = time.perf_counter()
    out = baseline.layout_and_expand(all_x, all_idx, all_w, 0, EXPERTS, 1, fp8)
    first = time.perf_counter() - started
    if first > budget_s / 4:  # bound the CPU work: time a prefix of every source instead
        sample_tokens = max(256, int(sample_tokens * (budget_s / 8) / first))
        sample = f"first {sample_tokens} tokens of every source"
        all_x, all_idx, all_w = ([t[:sample_tokens] for t in group] for group in (all_x, all_idx, all_w))
        out = baseline.layout_and_expand(all_x, all_idx, all_w, 0, EXPERTS, 1, fp8)
    times = []
    deadline = time.perf_counter() + budget_s
    for _ in range(5):
        started = time.perf_counter()
        out = baseline.layout_and_expand(all_x, all_idx, all_w, 0, EXPERTS, 1, fp8)
        times.append(time.perf_counter() - started)
        if time.perf_counter() > deadline:
            break
    mean = sum(times) / len(times)
    idx0 = all_idx[0]
    remote = (idx0 // (EXPERTS // WORLD) != 0) & (idx0 >= 0)
    own_remote_tokens = int(remote.any(dim=1).sum())
    moved = (own_remote_tokens + out["remote_unique"]) * payload_bytes
    return {
        "value": moved / mean / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port", "sample": sample,
        "us": mean * 1e6, "min_us": min(times) * 1e6, "runs": len(times),
        "expand_GBps": ((out["remote_unique"] + out["local_unique"]) + out["expanded_count"]) * HIDDEN * 2 / mean / 1e9,
    }


def percentiles(values):
    ordered = sorted(values)
    pick = lambda q: ordered[min(len(ordered) - 1, int(round(q * (len(ordered) - 1))))]
    return [pick(0.5), pick(0.95)]


def source_stamp() -> str:
    """Hash of the kernel sources the library was built from (csrc/*.hip, *.h,
    *.cpp): every counter summary under profiles/ names the stamp of the sources it
    was measured on, and a counted figure is only reported beside a live
    measurement while the two agree."""
    import hashlib

    digest = hashlib.sha256()
    for path in sorted((ROOT / "pcie-ep_amd" / "csrc").iterdir()):
        if path.suffix in (".hip", ".h", ".cpp"):
            digest.update(path.name.encode())
            digest.update(path.read_bytes())
    return digest.hexdigest()[:16]


def stamped(summary: Path) -> bool:
    """Whether a counter summary was measured on the sources of this build."""
    for line in summary.read_text().splitlines():
        if line.startswith("sources:"):
            return line.split(":", 1)[1].strip().split()[0] == source_stamp()
    return False


def counted_traffic(tokens, topk, routing, wire):
    """HBM bytes per launch of the expand kernel as counted by rocprofv3 (FETCH_SIZE
    + WRITE_SIZE, scaled by the calibration copy), from the committed counter
    summary of exactly this workload; None when there is none."""
    summary = ROOT / "profiles" / f"expand_kernel_T{tokens}_top{topk}_{routing}_counters.txt"
    if wire != "bf16" or not summary.exists() or not stamped(summary):
        return None
    for line in summary.read_text().splitlines():
        if line.startswith("hbm_traffic_bytes_per_launch"):
            return int(line.split("=")[1].strip())
    return None


def counted_host_traffic(tokens, topk, routing, wire):
    """Host-link bytes per launch of the transport kernel as counted by the L2's
    IO request counters (rocprofv3 --pmc, scaled by the kernel-driven pinned
    copy), from the committed counter summary of exactly this workload."""
    summary = ROOT / "profiles" / f"transport_kernel_T{tokens}_top{topk}_{routing}_{wire}_counters.txt"
    found = {"read": None, "write": None}
    if summary.exists() and stamped(summary):
        for line in summary.read_text().splitlines():
            for direction in found:
                if line.startswith(f"host_{direction}_traffic_bytes_per_launch"):
                    found[direction] = int(line.split("=")[1].strip())
    return found


def measure_expand(inputs, tokens, topk, channels, repeats=20):
    """Stand-alone expand kernel (unique rows -> expert-major rows) against HBM."""
    import torch

    from helpers import verify_dispatch

    buffer = make_buffer(tokens, topk, "bf16", channels, fuse=False)
    try:
        set_peers(buffer, inputs)
        buffer.peers.start(1)
        x, idx, weights = (item.cuda() for item in inputs[0])
        result = buffer.dispatch(x, idx, weights, do_expand=True)
        torch.cuda.synchronize()
        buffer.peers.wait(120_000)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, topk, True, 1, False)
        handle = result[3]
        unique, expanded = int(handle.unique_count.cpu()), int(handle.expanded_count.cpu())
        pool = next(pool for pool in buffer.runtime._pools if not pool.idle())
        plan = handle._layout
        # HIP events on the launch stream around `batch` back-to-back launches:
        # the per-launch mean then carries no event or launch-gap overhead and is
        # comparable with the profiler's kernel durations.
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        batch = 10
        for _ in range(3):
            buffer.runtime.expand_unique(pool.tensors, plan, 1, False)
        torch.cuda.synchronize()
        durations = []
        for _ in range(max(1, repeats // batch) + 1):
            begin.record()
            for _ in range(batch):
                buffer.runtime.expand_unique(pool.tensors, plan, 1, False)
            end.record()
            end.synchronize()
            durations.append(begin.elapsed_time(end) / batch)
        mean_ms = sum(durations) / len(durations)
        algorithmic = (unique + expanded) * HIDDEN * 2 + expanded * 36
        del result, handle
        # The same traffic shape with no metadata and no dependent loads (one row
        # read, one written, the same share of rows written twice), by write order:
        # what HBM gives a write-heavy row scatter on this part.
        from pcie_ep import _native

        ceilings = {}
        extra = max(0, min(1024, round((expanded / max(unique, 1) - 1.0) * 1024)))
        for name, pattern in (("linear", 0), ("expert_streams", 1), ("hashed", 2), ("read_only", 3), ("write_only", 4)):
            rate = _native.C.c_double()
            _native.check(_native.library().pcie_ep_measure_row_scatter(0, unique, HIDDEN * 2, extra, pattern, EXPERTS // WORLD, 5, _native.C.byref(rate)),
                          invalid=RuntimeError)
            ceilings[name] = rate.value
        return {
            "shape_ceiling_GBps": ceilings,
            "bound": "hbm", "kernel": "expand_pieces_kernel", "achieved": algorithmic / mean_ms / 1e6, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": algorithmic / mean_ms / 1e6 / HBM_PEAK_GBPS, "traffic": None, "algorithmic_bytes": algorithmic,
            "avg_us": mean_ms * 1e3, "min_us": min(durations) * 1e3, "unique_rows": unique, "expanded_rows": expanded,
        }
    finally:
        buffer.close()


def run_workload(inputs, tokens, topk, wire, channels, steps, warmup, peaks, verify=True, restage=False):
    """`steps` eager dispatches submitted back to back (wall clock per step), a second
    pass with HIP events around every kernel, and one untimed dispatch checked
    against the oracle.  Returns the measurements of this workload."""
    import torch

    from helpers import verify_dispatch

    # Restaging, the host threads move as many bytes as the GPU: every peer's source and receiver get a thread each.
    buffer = make_buffer(tokens, topk, wire, channels, fuse=True, peer_threads=2 * (WORLD - 1) if restage else None)
    try:
        sizes = buffer.runtime.sizes
        payload_bytes, meta_bytes = int(sizes.payload_bytes), int(sizes.meta_bytes)
        set_peers(buffer, inputs)
        x, idx, weights = (item.cuda() for item in inputs[0])
        sync_steps = steps if tokens <= 512 else 0
        stage_started = time.perf_counter()
        buffer.peers.start(warmup + 3 * steps + sync_steps + (1 if verify else 0), restage=restage, read_rows=restage)
        buffer.peers.wait_staged(120_000)
        # The emulator on its own: the first epoch is staged while the GPU is idle.
        stage_seconds = time.perf_counter() - stage_started
        # The interpreter's cyclic collector stays out of the measured passes, as under
        # `timeit`: a full collection of this process's heap takes 40 ms, some 700
        # small dispatches, and would land inside one of them.
        gc.collect()
        gc.disable()
        for _ in range(warmup):
            result = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True)
            del result
        torch.cuda.synchronize()
        # Timed region: exactly `steps` dispatches submitted back to back, as a
        # steady caller would (nothing is read back, the CPU never waits inside).
        started = time.perf_counter()
        for _ in range(steps):
            result = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True)
            del result
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - started) / steps * 1e3

        # The reference harness's figure (benchmarks/benchmark.py:165-198): an event pair
        # around every whole dispatch, on the stream the dispatch runs on.
        comm = buffer.get_comm_stream()
        pairs = []
        for _ in range(steps):
            before, after = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            before.record(comm)
            result = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True)
            after.record(comm)
            pairs.append((before, after))
            del result
        torch.cuda.synchronize()
        event_us = [before.elapsed_time(after) * 1e3 for before, after in pairs]
        # The default, synchronous mode (the caller's stream waits for every result) at
        # the sizes where the submission cost shows.
        sync_us = None
        if sync_steps:
            started = time.perf_counter()
            for _ in range(sync_steps):
                result = buffer.dispatch(x, idx, weights, do_expand=True)
                del result
            torch.cuda.synchronize()
            sync_us = (time.perf_counter() - started) / sync_steps * 1e6

        # Per-kernel durations: a second pass with HIP events recorded on the launch
        # stream around every kernel (reading them waits for that dispatch, so this
        # pass is not the one that is timed as a whole).
        buffer.runtime.set_kernel_timing(True)
        kernel_ms = {"prologue": [], "transport": []}
        inside_ns = []
        for _ in range(steps):
            result = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True)
            stamps = result[3].transport_timestamps_ns
            times = buffer.runtime.kernel_times_ms()
            for name in kernel_ms:
                kernel_ms[name].append(times[name])
            inside_ns.append(stamps.clone())
            del result, stamps
        torch.cuda.synchronize()
        buffer.runtime.set_kernel_timing(False)
        inside_ns = [item.cpu().tolist() for item in inside_ns]

        # One more, checked bit for bit against the oracle (untimed).
        parity = "skipped"
        result = None
        if verify:
            result = buffer.dispatch(x, idx, weights, do_expand=True)
            torch.cuda.synchronize()
        buffer.peers.wait(120_000)
        if result is not None:
            summary = verify_dispatch(result, inputs, 0, WORLD, EXPERTS, topk, True, 1, False, fp8_wire=wire == "fp8")
            parity = BIT_EXACT
            stats, unique, expanded = summary["stats"], summary["unique"], summary["expanded"]
        else:
            probe = buffer._last_handle
            stats = probe.stats.cpu().tolist()
            unique, expanded = int(probe.unique_count.cpu()), int(probe.expanded_count.cpu())
        del result
    finally:
        gc.enable()
        buffer.close()

    mean = lambda values: sum(values) / len(values)
    own_writes, remote_reads, descriptors = int(stats[0]), int(stats[1]), int(stats[7])
    transport_ms = mean(kernel_ms["transport"])
    # Per remote row read: payload + slot metadata + one 16-byte descriptor entry;
    # per own token written: payload + slot metadata, one 16-byte descriptor entry
    # per destination; per remote row: an 8-byte payload ACK, and an 8-byte credit
    # for every polled run of up to eight entries.
    read_bytes = remote_reads * (payload_bytes + meta_bytes + 16)
    write_bytes = own_writes * (payload_bytes + meta_bytes) + descriptors * 16 + remote_reads * 9
    h2d, d2h, kernel_read, kernel_write = peaks
    pcie = {
        "bound": "pcie", "kernel": "transport_kernel", "avg_us": transport_ms * 1e3, "min_us": min(kernel_ms["transport"]) * 1e3,
        "inside_kernel_us": mean([(end - begin) / 1e3 for begin, end in inside_ns]),
        "read_GBps": read_bytes / (transport_ms * 1e-3) / 1e9, "write_GBps": write_bytes / (transport_ms * 1e-3) / 1e9,
        "read_payload_GBps": remote_reads * payload_bytes / (transport_ms * 1e-3) / 1e9,
        "peak_h2d_GBps": h2d, "peak_d2h_GBps": d2h, "kernel_copy_read_GBps": kernel_read, "kernel_copy_write_GBps": kernel_write,
        "frac": read_bytes / (transport_ms * 1e-3) / 1e9 / h2d,
        "algorithmic_read_bytes": read_bytes, "algorithmic_write_bytes": write_bytes,
    }
    event_stats = {"mean": mean(event_us), "p50": percentiles(event_us)[0], "p95": percentiles(event_us)[1]}
    return {
        "dispatch_event_us": event_stats, "dispatch_sync_us": sync_us,
        "emulator_stage_GBps": remote_reads * (payload_bytes + meta_bytes) / stage_seconds / 1e9 if restage else None,
        "ms_per_step": ms_per_step, "kernel_ms": kernel_ms, "pcie": pcie, "parity": parity, "payload_bytes": payload_bytes,
        "value": (own_writes + remote_reads) * payload_bytes / (ms_per_step * 1e-3) / 1e9,
        "rows": {"own_published": own_writes, "remote_unique": remote_reads, "local_unique": unique - remote_reads, "expanded": expanded},
    }


def compact(run, tokens, topk):
    """The sub-record of one further workload."""
    mean = lambda values: sum(values) / len(values)
    return {
        "dispatch_us": run["ms_per_step"] * 1e3, "transport_us": mean(run["kernel_ms"]["transport"]) * 1e3,
        "prologue_us": mean(run["kernel_ms"]["prologue"]) * 1e3, "payload_GBps": run["value"],
        "dispatch_event_us": run["dispatch_event_us"], "dispatch_sync_us": run["dispatch_sync_us"],
        "pcie": run["pcie"]["frac"], "read_GBps": run["pcie"]["read_GBps"], "rows": run["rows"], "parity": run["parity"],
        "logical_GBps": tokens * topk * HIDDEN * 2 / (run["ms_per_step"] * 1e-3) / 1e9,
    }


def graph_replay_sweep(topk, channels, sizes=(16, 128, 512, 2048, 8192), replays=20, inputs_by_size=None):
    """Cached layout + hipGraph replay: the plan is built by one eager dispatch,
    the dispatch is captured with that plan, `replays` GPU-only replays are
    timed back to back (mean microseconds per replay, by size), and one more,
    untimed, is checked against the oracle."""
    import torch

    from helpers import verify_dispatch

    out = {}
    requested = replays
    for tokens in sizes:
        # The shortest replay needs more of them between the synchronisations that bracket the timed region (at
        # larger sizes more than a few dozen launches of one instantiated graph in flight make hipGraphLaunch block).
        replays = max(requested, 100) if tokens <= 16 else requested
        inputs = (inputs_by_size or {}).get(tokens) or build_inputs(tokens, topk, "uniform", False)
        with make_buffer(tokens, topk, "bf16", channels, fuse=True, graph=True) as buffer:
            set_peers(buffer, inputs)
            x, idx, weights = (item.cuda() for item in inputs[0])
            buffer.peers.start(1 + 3 + replays + 1)
            result = buffer.dispatch(x, idx, weights, do_expand=True)
            cache = buffer.cache_layout(result[3])
            del result
            graph = buffer.capture_dispatch(x, topk_weights=weights, handle=cache, do_expand=True)
            gc.collect()
            gc.disable()  # as in run_workload
            try:
                for _ in range(3):
                    graph.replay(async_with_compute_stream=True)
                torch.cuda.synchronize()
                started = time.perf_counter()
                for _ in range(replays):
                    graph.replay(async_with_compute_stream=True)
                torch.cuda.synchronize()
                replay_us = (time.perf_counter() - started) / replays * 1e6
            finally:
                gc.enable()
            result = graph.replay()
            torch.cuda.synchronize()
            buffer.peers.wait(120_000)
            verify_dispatch(result, inputs, 0, WORLD, EXPERTS, topk, True, 1, False)
            del result
            out[str(tokens)] = {"replay_us": replay_us, "replays": replays, "parity": BIT_EXACT}
        log(f"[bench] graph replay T={tokens}: {replay_us:.1f} us")
    return out


def role_timeline(sizes, wire, channels, repeats=15):
    """Per-role timeline of the dispatch (profiling build of the library): for every
    size, `repeats` dispatches submitted one at a time, each read back; the median of
    every event, in microseconds after the prologue's entry."""
    import statistics

    import torch

    from pcie_ep import profiling

    out = {}
    for tokens in sizes:
        inputs = build_inputs(tokens, 8, "uniform", wire == "fp8")
        buffer = make_buffer(tokens, 8, wire, channels, fuse=True)
        try:
            set_peers(buffer, inputs)
            x, idx, weights = (item.cuda() for item in inputs[0])
            buffer.peers.start(5 + repeats)
            buffer.peers.wait_staged(120_000)
            samples = []
            for step in range(5 + repeats):
                result = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True)
                torch.cuda.synchronize()
                if step >= 5:
                    samples.append(profiling.timeline(profiling.read(buffer.runtime)))
                del result
            buffer.peers.wait(120_000)
        finally:
            buffer.close()
        out[str(tokens)] = {name: round(statistics.median(sample[name] for sample in samples), 2) for name in samples[0]}
        log(f"[bench] role timeline T={tokens}: last role exit {out[str(tokens)]['transport.last_role_exit']} us after the prologue's entry")
    return out


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=5)
    parser.add_argument("--tokens", type=int, default=8192)
    parser.add_argument("--wire", choices=("bf16", "fp8"), default="bf16")
    parser.add_argument("--routing", choices=("uniform", "hotspot"), default="uniform")
    parser.add_argument("--channels", type=int, default=32)
    parser.add_argument("--skip-cpu-baseline", action="store_true")
    parser.add_argument("--skip-expand", action="store_true")
    parser.add_argument("--skip-verify", action="store_true")
    parser.add_argument("--only-headline", action="store_true",
                        help="time only the workload named by --tokens/--wire/--routing (no fp8 / hotspot / T=4096 / small-T / "
                             "graph-replay / restaged sub-records); what the profiler runs use")
    parser.add_argument("--expand-only", action="store_true",
                        help="run only the calibration copy kernel and the stand-alone expand kernel (short; for counter collection)")
    parser.add_argument("--source-stamp", action="store_true", help="print the hash of the kernel sources (the stamp of a profile summary) and exit")
    parser.add_argument("--split-launch", action="store_true",
                        help="run the prologue as a kernel of its own in front of the transport kernel (default: one launch per dispatch "
                             "wherever the prologue fits into the transport launch)")
    parser.add_argument("--role-timeline", type=str, default="",
                        help="comma-separated token counts: print the per-role timeline of the dispatch at those sizes and exit "
                             "(needs the profiling build: python pcie-ep_amd/build.py --profiling)")
    args = parser.parse_args()
    global SPLIT_LAUNCH
    SPLIT_LAUNCH = args.split_launch
    if args.source_stamp:
        print(source_stamp())
        return 0
    if args.role_timeline:
        os.environ["PCIE_EP_PROFILING"] = "1"
    if args.gpus != 1:
        print(f"bench.py measures one GPU's share of the dispatch; --gpus {args.gpus} is not supported "
              "(this build uses no second GPU, no collective and no rank code)", file=sys.stderr)
        return 2

    import torch

    from pcie_ep import _native

    torch.cuda.set_device(0)
    if args.role_timeline:
        sizes = [int(item) for item in args.role_timeline.split(",")]
        print(json.dumps({"role_timeline_us": role_timeline(sizes, args.wire, args.channels), "wire": args.wire,
                          "note": "median of 15 dispatches, microseconds after the prologue leader's entry; profiling build"}), flush=True)
        return 0
    topk = 4 if args.routing == "hotspot" else 8
    tokens = args.tokens
    log(f"[bench] building inputs: T={tokens} H={HIDDEN} top-{topk} {args.routing} {args.wire} wire")
    inputs = build_inputs(tokens, topk, args.routing, heavy_tail=args.wire == "fp8")

    h2d, d2h = _native.C.c_double(), _native.C.c_double()
    _native.check(_native.library().pcie_ep_measure_pinned_copy(0, 1 << 30, 5, _native.C.byref(h2d), _native.C.byref(d2h)), invalid=RuntimeError)
    log(f"[bench] pinned hipMemcpy peak: H2D {h2d.value:.2f} GB/s, D2H {d2h.value:.2f} GB/s")

    kernel_read, kernel_write = _native.C.c_double(), _native.C.c_double()
    _native.check(_native.library().pcie_ep_measure_kernel_host_copy(0, HOST_COPY_BYTES, 3, 96, _native.C.byref(kernel_read),
                                                                    _native.C.byref(kernel_write)), invalid=RuntimeError)
    log(f"[bench] kernel-driven pinned copy of {HOST_COPY_BYTES} bytes, 96 wavefronts: read {kernel_read.value:.2f} GB/s, "
        f"write {kernel_write.value:.2f} GB/s")
    copy_rate = _native.C.c_double()
    _native.check(_native.library().pcie_ep_measure_device_copy(0, COPY_BYTES, 5, _native.C.byref(copy_rate)), invalid=RuntimeError)
    log(f"[bench] plain device copy of {COPY_BYTES} bytes: {copy_rate.value:.0f} GB/s read+write")
    if args.expand_only:
        record = measure_expand(inputs, tokens, topk, args.channels, repeats=5)
        record["hbm_copy_GBps"] = copy_rate.value
        print(json.dumps({"roofline": record}), flush=True)
        return 0
    peaks = (h2d.value, d2h.value, kernel_read.value, kernel_write.value)

    log("[bench] headline workload")
    run = run_workload(inputs, tokens, topk, args.wire, args.channels, args.steps, args.warmup, peaks, verify=not args.skip_verify)
    mean = lambda values: sum(values) / len(values)
    ms_per_step, kernel_ms, pcie = run["ms_per_step"], run["kernel_ms"], run["pcie"]
    traffic = counted_host_traffic(tokens, topk, args.routing, args.wire)
    pcie["traffic_read"], pcie["traffic_write"] = traffic["read"], traffic["write"]
    if traffic["read"] is None:
        pcie["traffic_note"] = "no counter summary under profiles/ carries the stamp of these kernel sources (" + source_stamp() + ")"
    record = {
        "metric": "dispatch PCIe payload GB/s ((U+F_r)*B/t) and us per dispatch, receiver rank 0 of 8",
        "value": run["value"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.wire == "bf16" else "fp8_e4m3 wire / bf16",
        "data": "synthetic",
        "sources": source_stamp(),
        "config": {
            "workload": f"T={tokens}/source x 8 logical ranks, h{HIDDEN}, top-{topk} {args.routing}, {EXPERTS} experts (32 local), "
                        f"{args.wire} wire, C{args.channels}, Q=L=256, expand on, own TX + 7 host-staged sources",
            "tokens_per_rank": tokens, "hidden": HIDDEN, "topk": topk, "experts": EXPERTS, "channels": args.channels, "wire": args.wire,
            "peer_restage": False, "launches_per_dispatch": 2 if SPLIT_LAUNCH else 1,
        },
        "dispatch_us": ms_per_step * 1e3, "dispatch_event_us": run["dispatch_event_us"], "dispatch_sync_us": run["dispatch_sync_us"],
        "dispatch_gpu_us": (mean(kernel_ms["transport"]) + mean(kernel_ms["prologue"])) * 1e3,
        "kernel_us": {name: mean(values) * 1e3 for name, values in kernel_ms.items()},
        "dispatch_gpu_us_p50_p95": percentiles([1e3 * sum(step) for step in zip(*kernel_ms.values())]),
        "pcie_pct_of_peak": 100.0 * pcie["frac"],
        "logical_GBps": tokens * topk * HIDDEN * 2 / (ms_per_step * 1e-3) / 1e9,
        "rows": run["rows"],
        "parity": run["parity"],
        "pcie": pcie,
    }
    if not args.skip_expand:
        log("[bench] measuring the stand-alone expand kernel")
        record["roofline"] = measure_expand(inputs, tokens, topk, args.channels)
        record["roofline"]["hbm_copy_GBps"] = copy_rate.value
        record["roofline"]["traffic"] = counted_traffic(tokens, topk, args.routing, args.wire)
        if record["roofline"]["traffic"] is None:
            record["roofline"]["traffic_note"] = "no counter summary under profiles/ carries the stamp of these kernel sources (" + source_stamp() + ")"
    else:
        record["roofline"] = None
    if not args.skip_cpu_baseline:
        log("[bench] timing the CPU baseline on the host cores")
        record["cpu_baseline"] = cpu_baseline(inputs, run["payload_bytes"], fp8=args.wire == "fp8")
    else:
        record["cpu_baseline"] = None

    if not args.only_headline:
        steps, warmup = args.steps, args.warmup
        # The same workload with the host threads rewriting every slot and reading
        # every sent row in every step: host-memory traffic concurrent with the
        # GPU's.  Seven host threads cannot stage 0.5 GB per step as fast as the GPU
        # reads it, so this figure is bounded by the emulator, not by the link.
        log("[bench] headline workload, peers restaging every step")
        restaged = run_workload(inputs, tokens, topk, args.wire, args.channels, max(3, steps // 4), 2, peaks, verify=False, restage=True)
        record["restaged"] = {"dispatch_us": restaged["ms_per_step"] * 1e3, "transport_us": mean(restaged["kernel_ms"]["transport"]) * 1e3,
                              "pcie": restaged["pcie"]["frac"], "read_GBps": restaged["pcie"]["read_GBps"], "peer_restage": True,
                              "emulator_stage_GBps": restaged["emulator_stage_GBps"],
                              "note": "every source slot rewritten and every sent row read by the host threads per step; "
                                      "emulator_stage_GBps is their staging rate for the first epoch, with the GPU idle"}
        uniform_8192 = inputs if (tokens, args.routing, args.wire) == (8192, "uniform", "bf16") else None
        del inputs
        log("[bench] fp8 wire, heavy-tailed inputs, T=8192 top-8")
        record["fp8"] = compact(run_workload(build_inputs(8192, 8, "uniform", True), 8192, 8, "fp8", args.channels, steps, warmup, peaks), 8192, 8)
        log("[bench] hotspot top-4, T=8192")
        record["hotspot_top4"] = compact(run_workload(build_inputs(8192, 4, "hotspot", False), 8192, 4, "bf16", args.channels, steps, warmup, peaks), 8192, 4)
        log("[bench] uniform top-8, T=4096")
        record["t4096"] = compact(run_workload(build_inputs(4096, 8, "uniform", False), 4096, 8, "bf16", args.channels, steps, warmup, peaks), 4096, 8)
        small = {}
        small_inputs = {}
        for size in (16, 128, 512, 2048):
            small_inputs[size] = build_inputs(size, 8, "uniform", False)
            # A short dispatch needs more of them between the two synchronisations that bracket the timed region:
            # twenty of 55 us are 1.1 ms, of which the closing synchronisation alone is 3 %.
            many = max(steps, 200) if size <= 512 else steps
            small[str(size)] = compact(run_workload(small_inputs[size], size, 8, "bf16", args.channels, many, warmup, peaks), size, 8)
            small[str(size)]["steps"] = many
            log(f"[bench] eager T={size}: {small[str(size)]['dispatch_us']:.1f} us per dispatch")
        record["eager_small_t"] = small
        if uniform_8192 is not None:
            small_inputs[8192] = uniform_8192
        record["graph_replay_us"] = graph_replay_sweep(8, args.channels, replays=steps, inputs_by_size=small_inputs)
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

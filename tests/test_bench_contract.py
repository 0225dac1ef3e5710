"""The benchmark's command-line contract: one JSON line with the agreed keys on a
GPU, and a clear refusal of more than one GPU (this build uses no second GPU)."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def test_more_than_one_gpu_is_refused_with_a_message():
    outcome = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert outcome.returncode != 0
    assert "--gpus 2 is not supported" in outcome.stderr and not outcome.stdout.strip()


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    command = [sys.executable, str(ROOT / "bench.py"), "--tokens", "256", "--steps", "3", "--warmup", "1", "--only-headline"]
    print("case: " + " ".join(command[1:]), flush=True)
    outcome = subprocess.run(command, capture_output=True, text=True, timeout=300)
    assert outcome.returncode == 0, outcome.stderr[-2000:]
    lines = [line for line in outcome.stdout.splitlines() if line.strip()]
    assert len(lines) == 1, lines
    record = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline", "pcie"):
        assert key in record, key
    assert record["n_gpus"] == 1 and record["steps"] == 3 and record["warmup"] == 1 and record["vs_baseline"] is None
    assert record["higher_is_better"] is True and record["data"] == "synthetic" and "workload" in record["config"]
    assert record["parity"] == "bit-exact vs oracle" and record["value"] > 0
    roofline = record["roofline"]
    assert roofline["bound"] == "hbm" and roofline["peak"] == 8000.0 and roofline["unit"] == "GB/s"
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-9
    baseline = record["cpu_baseline"]
    assert baseline["kind"] == "port" and baseline["cores"] >= 1 and baseline["value"] > 0 and baseline["sample"]
    # The reference harness's own measure (an event pair around each whole dispatch) and the default synchronous mode.
    events = record["dispatch_event_us"]
    assert 0 < events["p50"] <= events["p95"] and events["mean"] > 0
    assert record["dispatch_sync_us"] > 0  # reported up to 512 tokens, where the submission cost shows
    # A counted figure is reported only with a summary measured on these kernel sources; otherwise null, with a note.
    assert len(record["sources"]) == 16
    assert "traffic" in roofline and (roofline["traffic"] is not None or "traffic_note" in roofline)
    assert record["pcie"]["traffic_read"] is not None or "traffic_note" in record["pcie"]


def test_counter_summaries_are_stamped_with_the_sources_they_were_measured_on():
    """Every counted figure bench.py may quote comes from a summary that names the
    hash of the kernel sources it was measured on and the command that made it."""
    sys.path.insert(0, str(ROOT))
    import bench

    stamp = bench.source_stamp()
    assert len(stamp) == 16 and stamp == bench.source_stamp()
    for summary in sorted((ROOT / "profiles").glob("*.txt")):
        text = summary.read_text()
        assert any(line.startswith("sources:") for line in text.splitlines()), summary.name
        assert any(line.startswith("command") for line in text.splitlines()), summary.name


"""The hand-off everything else rests on, alone: a payload in pinned host memory
published by a sequence word, between the GPU and a CPU thread, in both
directions, and between two kernels on two streams, by one wavefront and by a workgroup, with the last thread delayed
on either side (the reference's experiment: tests/MAPPED_LITMUS.md, 1 M rounds of
14 336 bytes, `--delay 1000 --writer-delay 1000`).  Every round the consumer
compares every word with what that round must hold, so a payload word that
arrives after its sequence word, or a slot reused before its reader was done,
fails the round."""

from __future__ import annotations

import pytest

pytestmark = pytest.mark.gpu

MODES = {"gpu-wave-to-cpu": 0, "gpu-workgroup-to-cpu": 1, "cpu-to-gpu-wave": 2, "cpu-to-gpu-workgroup": 3,
         # both ends kernels, on two streams, the slot in host memory between them (the reference's experiment proper)
         "gpu-wave-to-gpu-wave": 4, "gpu-workgroup-to-gpu-workgroup": 5}


@pytest.mark.parametrize("name", list(MODES))
def test_publication_litmus(name):
    from pcie_ep import litmus

    for payload_bytes, writer_delay_ns, reader_delay_ns, iterations in ((14336, 0, 0, 200_000), (14336, 1000, 1000, 60_000),
                                                                       (7168 + 192, 300, 0, 60_000), (2048, 0, 700, 60_000), (16, 0, 0, 60_000)):
        print(f"litmus {name}: {payload_bytes} B, writer delay {writer_delay_ns} ns, reader delay {reader_delay_ns} ns, {iterations} rounds", flush=True)
        result = litmus.run(MODES[name], iterations, payload_bytes, writer_delay_ns, reader_delay_ns, timeout_ms=10_000)
        assert result["gpu"]["code"] == 0 and result["host"]["code"] == 0, result
        assert result["completed"] == iterations, result
        print(f"  {result['seconds'] / iterations * 1e6:.2f} us per round", flush=True)


@pytest.mark.parametrize("name", list(MODES))
def test_publication_litmus_while_the_link_is_busy(name):
    """The same with both directions of the host link saturated by copy kernels, as
    during a dispatch: small control stores and loads then wait tens of
    microseconds behind row traffic and take other paths through the fabric."""
    from pcie_ep import litmus

    with litmus.link_traffic():
        for payload_bytes, writer_delay_ns, reader_delay_ns, iterations in ((14336, 0, 0, 100_000), (14336, 1000, 1000, 50_000), (2048, 0, 0, 50_000)):
            print(f"litmus under load {name}: {payload_bytes} B, delays {writer_delay_ns}/{reader_delay_ns} ns, {iterations} rounds", flush=True)
            result = litmus.run(MODES[name], iterations, payload_bytes, writer_delay_ns, reader_delay_ns, timeout_ms=10_000)
            assert result["gpu"]["code"] == 0 and result["host"]["code"] == 0, result
            assert result["completed"] == iterations, result


@pytest.mark.parametrize("modes", [(0, 1), (4, 5)], ids=["gpu-to-cpu", "gpu-to-gpu"])
def test_negative_control_publishing_before_the_stores_are_acknowledged_fails(modes):
    """The experiment can fail: a producer that stores the sequence word without
    waiting for its payload stores is caught by the consumer (the CPU thread, or the consumer kernel) with a stale payload
    word once the link carries other traffic (seen after 5 to 32 000 rounds).  The
    kernel ends normally - its peer raises the abort word it polls."""
    from pcie_ep import litmus

    caught = []
    with litmus.link_traffic():
        for mode in modes + modes:
            for delays in ((0, 0), (1000, 0)):
                result = litmus.run(mode | litmus.PUBLISH_EARLY, 400_000 if mode < 4 else 60_000, 14336, delays[0], delays[1], timeout_ms=10_000)
                print(f"negative control mode {mode} delays {delays}: {result}", flush=True)
                # The consumer finds the stale word (code 4), the producer is then told to stop (code 3); between two
                # kernels the consumer's verdict is the "gpu" entry and the producer's the "host" entry.
                consumer, producer = (result["gpu"], result["host"]) if mode >= 4 else (result["host"], result["gpu"])
                assert producer["code"] in (0, 3) and consumer["code"] in (0, 4), result
                if consumer["code"] == 4:
                    caught.append(consumer["iteration"])
            if len(caught) >= 2:
                break
    if not caught:
        # Whether unacknowledged stores overtake each other depends on the path between
        # this GPU and host memory; a box on which they never do tells nothing either way.
        pytest.skip("publishing early was not caught on this box: no evidence from the negative control here (between two kernels of ONE GPU the "
                    "consumer's reads follow the producer's writes over the same link, which orders them; the CPU sees the writes as they land)")
    print(f"negative control caught after {caught} rounds", flush=True)


def test_litmus_rejects_bad_arguments():
    from pcie_ep import litmus

    for arguments in ((6, 10, 14336), (0, 0, 14336), (0, 10, 8), (0, 10, 24), (2 | 16, 10, 14336)):
        with pytest.raises(ValueError):
            litmus.run(*arguments)

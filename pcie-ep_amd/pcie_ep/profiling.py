"""Per-role timing records of a dispatch (profiling builds of the library only).

Counterpart of the reference's ``handle.profiling`` tensor and its schema
(docs/pcie-ep/profiling-instrumentation.md:40-92): one record of 32 int64 per
role wavefront, written once when the role ends.  Build the variant with
``python pcie-ep_amd/build.py --profiling`` and select it with
``PCIE_EP_PROFILING=1`` before importing ``pcie_ep``.

Rows: TX control ``[0, C)``, RX control ``[C, 2C)``, payload wavefronts
``[2C, 2C + W)``, prologue leader ``[2C + W]``, epoch begin ``[2C + W + 1]``, producer of the
receive prefixes ``[2C + W + 2]`` (the last two hold records only where those are
roles of their own; ``read`` folds their stamps into the leader's and RX control 0's).  Stamps (``*_ns``) are
nanoseconds of the device wall clock, sums are accumulated nanoseconds; a zero
stamp means the event did not happen.  Intervals of different roles overlap.
"""

from __future__ import annotations

import ctypes as C
from typing import Dict

import numpy as np

from . import _native

COMMON = ("enter_ns", "exit_ns", "total_ns", "items")
CONTROL = COMMON + ("first_ticket_ns", "last_ticket_ns", "workers_done_ns", "drained_ns", "finished_ns", "polls", "poll_misses",
                    "poll_sum", "health_scans", "health_sum", "counts_known_ns", "spare", "prefix_enter_ns",
                    "prefix_counts_ready_ns", "prefix_mailbox_ns", "prefix_published_ns")
WORKER = COMMON + ("first_claim_ns", "last_row_ns", "tx_rows", "rx_rows", "sampled_tx_rows", "sampled_rx_rows", "ticket_wait_sum",
                   "idle_sum", "tx_flow_wait_sum", "tx_copy_sum", "rx_request_sum", "rx_prefix_wait_sum", "rx_scatter_sum", "gate_open_ns",
                   "first_look_ns", "first_tagged_ns", "first_entry_ns", "first_request_ns", "first_data_ns")
PROLOGUE = COMMON + ("layout_ns", "totals_ns", "verdict_ns", "mailbox_free_ns", "mailbox_acked_ns", "counts_ready_ns",
                     "begun_ns", "routes_ns", "masks_ns", "chunk_totals_ns", "plan_ready_ns")


def read(runtime) -> Dict[str, np.ndarray]:
    """Records of the runtime's last dispatch (waits for the device), split by role."""
    lib = _native.library()
    rows, fields, channels, wavefronts = (C.c_int32() for _ in range(4))
    _native.check(lib.pcie_ep_profile_shape(runtime.handle, C.byref(rows), C.byref(fields), C.byref(channels), C.byref(wavefronts)),
                  invalid=RuntimeError)
    if rows.value == 0:
        raise RuntimeError("the loaded library has no profiling records: build with --profiling and set PCIE_EP_PROFILING=1")
    table = np.zeros((rows.value, fields.value), dtype=np.int64)
    _native.check(lib.pcie_ep_profile_read(runtime.handle, table.ctypes.data_as(C.POINTER(C.c_int64))), invalid=RuntimeError)
    c, w = channels.value, wavefronts.value
    prologue = table[2 * c + w].copy()
    begin = table[2 * c + w + 1]
    # The epoch begin keeps a record of its own where it is a workgroup of its own
    # (prologue inside the transport launch); its stamps are folded into the leader's.
    if begin[0]:
        for name in ("begun_ns", "verdict_ns", "mailbox_free_ns"):
            prologue[PROLOGUE.index(name)] = begin[PROLOGUE.index(name)]
    # Likewise the producer of the receive prefixes: its stamps are folded into RX control 0's.
    rx_control = table[c : 2 * c].copy()
    producer = table[2 * c + w + 2]
    if producer[0]:
        for name in ("prefix_enter_ns", "prefix_counts_ready_ns", "prefix_mailbox_ns", "prefix_published_ns"):
            rx_control[0, CONTROL.index(name)] = producer[CONTROL.index(name)]
    return {"tx_control": table[:c], "rx_control": rx_control, "workers": table[2 * c : 2 * c + w], "prologue": prologue,
            "epoch_begin": begin, "prefix_producer": producer}


def _col(rows: np.ndarray, names, name: str) -> np.ndarray:
    return rows[..., names.index(name)]


def timeline(records: Dict[str, np.ndarray]) -> Dict[str, float]:
    """Key events of one dispatch in microseconds after the prologue's entry
    (min over roles for 'first' events, max for 'last' ones)."""
    pro, txc, rxc, wrk = records["prologue"], records["tx_control"], records["rx_control"], records["workers"]
    zero = int(_col(pro, PROLOGUE, "enter_ns"))

    def first(values) -> float:
        values = np.asarray(values).reshape(-1)
        values = values[values > 0]
        return float("nan") if values.size == 0 else (int(values.min()) - zero) / 1e3

    def last(values) -> float:
        values = np.asarray(values).reshape(-1)
        values = values[values > 0]
        return float("nan") if values.size == 0 else (int(values.max()) - zero) / 1e3

    def per(total, count) -> float:
        count = int(np.sum(count))
        return float("nan") if count == 0 else float(np.sum(total)) / count / 1e3

    def median(values) -> float:
        values = np.asarray(values).reshape(-1)
        values = values[values > 0]
        return float("nan") if values.size == 0 else (float(np.median(values)) - zero) / 1e3

    out = {f"prologue.{name[:-3]}": first(_col(pro, PROLOGUE, name)) for name in PROLOGUE[4:] + ("exit_ns",)}
    active = wrk[_col(wrk, WORKER, "items") > 0]
    # Wavefronts whose first row was a received one, claimed before any row had come in.
    receivers = wrk[(_col(wrk, WORKER, "first_entry_ns") > 0) & (_col(wrk, WORKER, "first_entry_ns") <= _col(wrk, WORKER, "first_request_ns"))]
    out.update({
        "transport.first_role_enter": first(np.concatenate([_col(txc, CONTROL, "enter_ns"), _col(rxc, CONTROL, "enter_ns"), _col(wrk, WORKER, "enter_ns")])),
        "prefix.enter": first(_col(rxc, CONTROL, "prefix_enter_ns")), "prefix.counts_ready_seen": first(_col(rxc, CONTROL, "prefix_counts_ready_ns")),
        "prefix.mailboxes_returned": first(_col(rxc, CONTROL, "prefix_mailbox_ns")), "prefix.published": first(_col(rxc, CONTROL, "prefix_published_ns")),
        "rx.first_gate_open": first(_col(wrk, WORKER, "gate_open_ns")), "rx.first_ticket": first(_col(rxc, CONTROL, "first_ticket_ns")),
        "rx.last_ticket": last(_col(rxc, CONTROL, "last_ticket_ns")), "rx.counts_known_first": first(_col(rxc, CONTROL, "counts_known_ns")),
        "rx.rows_scattered_last": last(_col(rxc, CONTROL, "workers_done_ns")), "rx.finished_last": last(_col(rxc, CONTROL, "finished_ns")),
        "rx.descriptor_poll_us": per(_col(rxc, CONTROL, "poll_sum"), _col(rxc, CONTROL, "polls")),
        "rx.polls": float(np.sum(_col(rxc, CONTROL, "polls"))), "rx.poll_misses": float(np.sum(_col(rxc, CONTROL, "poll_misses"))),
        "tx.first_ticket": first(_col(txc, CONTROL, "first_ticket_ns")), "tx.last_ticket": last(_col(txc, CONTROL, "last_ticket_ns")),
        "tx.rows_published_last": last(_col(txc, CONTROL, "workers_done_ns")), "tx.drained_last": last(_col(txc, CONTROL, "drained_ns")),
        "tx.finished_last": last(_col(txc, CONTROL, "finished_ns")), "tx.drain_poll_us": per(_col(txc, CONTROL, "poll_sum"), _col(txc, CONTROL, "polls")),
        "tx.drain_polls": float(np.sum(_col(txc, CONTROL, "polls"))), "tx.drain_misses": float(np.sum(_col(txc, CONTROL, "poll_misses"))),
        # The way of a payload wavefront's first row (median over the wavefronts whose first row was a received one).
        **{f"first_row.{name}": median(_col(receivers, WORKER, field)) for name, field in (
            ("look", "first_look_ns"), ("claim", "first_claim_ns"), ("tag_seen", "first_tagged_ns"), ("entry_read", "first_entry_ns"),
            ("gate_passed", "gate_open_ns"), ("requested", "first_request_ns"), ("metadata_back", "first_data_ns"))},
        "workers.first_claim": first(_col(wrk, WORKER, "first_claim_ns")), "workers.last_row_end": last(_col(wrk, WORKER, "last_row_ns")),
        "workers.active": float(active.shape[0]),
        "workers.ticket_wait_us": per(_col(wrk, WORKER, "ticket_wait_sum"), _col(wrk, WORKER, "items")),
        "workers.rx_request_to_data_us": per(_col(wrk, WORKER, "rx_request_sum"), _col(wrk, WORKER, "sampled_rx_rows")),
        "workers.rx_request_to_stores_us": per(_col(wrk, WORKER, "rx_scatter_sum"), _col(wrk, WORKER, "sampled_rx_rows")),
        "workers.rx_prefix_wait_us": per(_col(wrk, WORKER, "rx_prefix_wait_sum"), _col(wrk, WORKER, "sampled_rx_rows")),
        "workers.tx_flow_wait_us": per(_col(wrk, WORKER, "tx_flow_wait_sum"), _col(wrk, WORKER, "sampled_tx_rows")),
        "workers.tx_copy_to_ack_us": per(_col(wrk, WORKER, "tx_copy_sum"), _col(wrk, WORKER, "sampled_tx_rows")),
        "workers.idle_us_mean": per(_col(wrk, WORKER, "idle_sum"), np.array([max(1, wrk.shape[0])])),
        "transport.last_role_exit": last(np.concatenate([_col(txc, CONTROL, "exit_ns"), _col(rxc, CONTROL, "exit_ns"), _col(wrk, WORKER, "exit_ns")])),
    })
    return out

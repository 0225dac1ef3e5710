"""CPU-only checks of the C ABI: the library loads, exports exactly what the
header declares, the ctypes mirror has the C layout, and the host-side
arithmetic the library exposes agrees with the oracle.  Nothing here touches a
GPU (no dispatch is launched).
"""

from __future__ import annotations

import ctypes as C
import re
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import dispatch_oracle as oracle
from oracle import fp8_oracle
from pcie_ep import _native

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "pcie_ep_amd.h"


def declared_functions() -> list:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(pcie_ep_[a-z0-9_]+)\s*\(", text)))


def make_config(**overrides) -> _native.Config:
    values = dict(num_ranks=8, local_rank=0, max_tokens=8192, hidden=7168, topk=8, num_experts=256, channels=32, payload_slots=256,
                  descriptor_slots=256, wire_fp8=0, timeout_ms=30000, fuse_receive_expand=1, tx_waves=0, rx_waves=0, peer_threads=0,
                  staging_numa_node=-1, device=0, worker_groups=0)
    values.update(overrides)
    return _native.Config(**values)


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 30
    library = C.CDLL(str(_native.LIBRARY_PATH))
    missing = [name for name in names if not hasattr(library, name)]
    assert not missing, f"declared in the header but not exported: {missing}"
    # ... and the ctypes binding covers the same set, no more, no fewer.
    assert sorted(_native.EXPORTED_SYMBOLS) == names


def test_abi_version_matches_header():
    version = int(re.search(r"#define PCIE_EP_ABI_VERSION (\d+)", HEADER.read_text()).group(1))
    assert _native.library().pcie_ep_abi_version() == version


def test_ctypes_structs_have_the_c_layout(tmp_path):
    """Compile the header as plain C and compare sizeof / offsetof with ctypes."""
    probes = {
        "pcie_ep_config": (_native.Config, ["num_ranks", "worker_groups", "receive_expand_mode", "reserved", "rank_numa_nodes", "relay_cpus", "relay_delay_ns"]),
        "pcie_ep_sizes": (_native.Sizes, ["unique_rows", "local_experts", "transport_workgroups", "reserved"]),
        "pcie_ep_dispatch_args": (_native.DispatchArgs, ["x", "num_tokens", "plan", "unique_payload", "errors", "prefix_tx_timestamps_ns",
                                                        "expanded_capacity_rows"]),
    }
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void) {"]
    for struct, (_, members) in probes.items():
        lines.append(f'printf("{struct} %zu\\n", sizeof({struct}));')
        for member in members:
            lines.append(f'printf("{struct}.{member} %zu\\n", offsetof({struct}, {member}));')
    lines += ["return 0;", "}"]
    source = tmp_path / "probe.c"
    source.write_text("\n".join(lines))
    binary = tmp_path / "probe"
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", str(source), "-o", str(binary)], check=True)
    reported = dict(line.split() for line in subprocess.run([str(binary)], check=True, capture_output=True, text=True).stdout.splitlines())
    for struct, (mirror, members) in probes.items():
        assert int(reported[struct]) == C.sizeof(mirror), struct
        for member in members:
            assert int(reported[f"{struct}.{member}"]) == getattr(mirror, member).offset, f"{struct}.{member}"


@pytest.mark.parametrize("ranks,tokens,hidden,topk,experts,fp8", [
    (8, 8192, 7168, 8, 256, 0), (8, 8192, 7168, 8, 256, 1), (8, 64, 512, 2, 16, 0), (2, 16, 100, 3, 6, 0), (16, 4096, 7168, 32, 4096, 1),
    (1, 128, 256, 4, 8, 0),
])
def test_query_sizes_matches_the_capacity_formulas(ranks, tokens, hidden, topk, experts, fp8):
    sizes = _native.Sizes()
    config = make_config(num_ranks=ranks, max_tokens=tokens, hidden=hidden, topk=topk, num_experts=experts, wire_fp8=fp8)
    assert _native.library().pcie_ep_query_sizes(C.byref(config), C.byref(sizes)) == 0, _native.last_error()
    unique, expanded = oracle.capacities(ranks, tokens, topk, experts)
    assert (sizes.unique_rows, sizes.expanded_rows) == (unique, expanded)
    assert sizes.local_experts == experts // ranks
    assert sizes.payload_bytes == hidden * (1 if fp8 else 2)
    assert sizes.meta_bytes >= 96 + 12 * topk and sizes.meta_bytes % 16 == 0
    assert sizes.slot_stride % 4096 == 0 and sizes.slot_stride >= sizes.payload_bytes + sizes.meta_bytes
    assert sizes.mailbox_dwords == 1 + experts // ranks + 32
    # Slots dominate the segment: C * Q slots plus signals and descriptors.
    assert sizes.segment_bytes >= 32 * 256 * sizes.slot_stride and sizes.segment_bytes % 4096 == 0
    assert sizes.plan_bytes >= tokens * (4 + 4 * ranks + 8 * topk)


def test_expanded_capacity_known_value():
    # 8 ranks x 8192 tokens, top-8, 32 local experts: 65 536 * 8 + 32 * 255 rows
    # (the figure quoted for one result pool of the reference at this size).
    sizes = _native.Sizes()
    config = make_config()
    assert _native.library().pcie_ep_query_sizes(C.byref(config), C.byref(sizes)) == 0
    assert sizes.expanded_rows == 532_448 and sizes.unique_rows == 65_536


@pytest.mark.parametrize("overrides,fragment", [
    (dict(num_ranks=0), "unsupported advanced dimensions"),
    (dict(num_ranks=17), "unsupported advanced dimensions"),
    (dict(topk=33), "unsupported advanced dimensions"),
    (dict(num_experts=250), "unsupported advanced dimensions"),
    (dict(num_experts=8192), "unsupported advanced dimensions"),
    (dict(local_rank=8), "unsupported advanced dimensions"),
    (dict(channels=0), "channels must be 1..32"),
    (dict(channels=33), "channels must be 1..32"),
    (dict(payload_slots=0), "invalid advanced capacity or timeout"),
    (dict(timeout_ms=0), "invalid advanced capacity or timeout"),
    (dict(tx_waves=9), "tx_waves"),
    (dict(worker_groups=100000), "worker_groups"),
])
def test_query_sizes_rejects_bad_configs(overrides, fragment):
    sizes = _native.Sizes()
    config = make_config(**overrides)
    assert _native.library().pcie_ep_query_sizes(C.byref(config), C.byref(sizes)) == _native.E_INVALID
    assert fragment in _native.last_error()
    with pytest.raises(ValueError):
        _native.check(_native.E_INVALID)


def test_null_arguments_are_rejected_not_dereferenced():
    library = _native.library()
    assert library.pcie_ep_query_sizes(None, None) == _native.E_INVALID
    assert library.pcie_ep_runtime_create(None, None) == _native.E_INVALID
    assert library.pcie_ep_runtime_destroy(None) == 0


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the failure mode of a box without a GPU")
def test_runtime_create_fails_loudly_without_a_gpu():
    runtime = C.c_void_p()
    config = make_config(max_tokens=64, hidden=512, topk=2, num_experts=16)
    status = _native.library().pcie_ep_runtime_create(C.byref(config), C.byref(runtime))
    assert status == _native.E_HIP and not runtime.value
    assert "needs a GPU" in _native.last_error()


def random_routes(generator: torch.Generator, tokens: int, topk: int, experts: int, unused: float = 0.0) -> np.ndarray:
    idx = torch.rand(tokens, experts, generator=generator).topk(topk, dim=1).indices.to(torch.int64)
    if unused:
        idx[torch.rand(tokens, topk, generator=generator) < unused] = -1
    return idx.numpy()


@pytest.mark.parametrize("tokens,topk,ranks,experts,unused", [
    (64, 2, 8, 16, 0.0), (1000, 8, 8, 256, 0.0), (777, 4, 4, 64, 0.3), (1, 1, 1, 1, 0.0), (0, 8, 8, 256, 0.0), (300, 32, 16, 4096, 0.1),
])
def test_host_source_layout_matches_the_oracle(tokens, topk, ranks, experts, unused):
    generator = torch.Generator().manual_seed(tokens * 31 + topk)
    idx = np.ascontiguousarray(random_routes(generator, tokens, topk, experts, unused).reshape(tokens, topk))
    mask = np.zeros(tokens, np.uint32)
    rank_ordinals = np.zeros((tokens, ranks), np.int32)
    expert_indices = np.zeros((tokens, topk), np.int32)
    expert_ordinals = np.zeros((tokens, topk), np.int32)
    counts = np.zeros(ranks + experts, np.int32)
    pointer = lambda array: array.ctypes.data_as(C.c_void_p)
    status = _native.library().pcie_ep_host_source_layout(pointer(idx), tokens, topk, ranks, experts, pointer(mask), pointer(rank_ordinals),
                                                          pointer(expert_indices), pointer(expert_ordinals), pointer(counts))
    expected = oracle.source_layout(idx, ranks, experts)
    assert status == expected.error == 0
    np.testing.assert_array_equal(mask.astype(np.uint64), expected.destination_mask)
    np.testing.assert_array_equal(rank_ordinals, expected.rank_ordinals)
    np.testing.assert_array_equal(expert_indices, expected.expert_indices)
    np.testing.assert_array_equal(expert_ordinals, expected.expert_ordinals)
    np.testing.assert_array_equal(counts, expected.counts)


@pytest.mark.parametrize("bad", ["duplicate", "too_large", "below_minus_one"])
def test_host_source_layout_reports_invalid_routing(bad):
    idx = random_routes(torch.Generator().manual_seed(5), 32, 4, 64).copy()
    if bad == "duplicate":
        idx[7, 3] = idx[7, 0]
    elif bad == "too_large":
        idx[7, 3] = 64
    else:
        idx[7, 3] = -2
    outputs = [np.zeros(32, np.uint32), np.zeros((32, 8), np.int32), np.zeros((32, 4), np.int32), np.zeros((32, 4), np.int32),
               np.zeros(8 + 64, np.int32)]
    status = _native.library().pcie_ep_host_source_layout(idx.ctypes.data_as(C.c_void_p), 32, 4, 8, 64,
                                                          *[item.ctypes.data_as(C.c_void_p) for item in outputs])
    assert status == oracle.ERROR_INVALID_ROUTING == oracle.source_layout(idx, 8, 64).error


@pytest.mark.parametrize("tokens,hidden", [(64, 512), (33, 7168), (5, 100), (1, 1), (16, 7)])
def test_host_fp8_codec_matches_the_oracle_bytes(tokens, hidden):
    generator = torch.Generator().manual_seed(hidden)
    x = torch.randn(tokens, hidden, generator=generator)
    x[:, :: max(1, hidden // 7)] *= 50.0  # heavy-tailed channels
    if tokens > 2:
        x[1].zero_()  # an all-zero row takes the scale floor
        x[2] *= 1e-30
    x = x.bfloat16().contiguous()
    codes = np.zeros((tokens, hidden), np.uint8)
    scales = np.zeros(tokens, np.float32)
    library = _native.library()
    assert library.pcie_ep_host_quantize_fp8(C.c_void_p(x.data_ptr()), codes.ctypes.data_as(C.c_void_p), scales.ctypes.data_as(C.c_void_p),
                                             tokens, hidden) == 0
    expected_codes, expected_scales = fp8_oracle.quantize(x)
    np.testing.assert_array_equal(codes, expected_codes.view(torch.uint8).numpy())
    np.testing.assert_array_equal(scales, expected_scales.numpy().reshape(-1))
    restored = torch.empty_like(x)
    assert library.pcie_ep_host_dequantize_fp8(codes.ctypes.data_as(C.c_void_p), scales.ctypes.data_as(C.c_void_p), C.c_void_p(restored.data_ptr()),
                                               tokens, hidden) == 0
    expected_restored = fp8_oracle.dequantize(expected_codes, expected_scales)
    assert torch.equal(restored.view(torch.int16), expected_restored.view(torch.int16))


def test_missing_library_raises_instead_of_falling_back(monkeypatch, tmp_path):
    monkeypatch.setattr(_native, "_library", None)
    monkeypatch.setattr(_native, "LIBRARY_PATH", tmp_path / "libpcie_ep_amd.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _native.library()


def test_product_never_imports_the_oracle():
    offenders = []
    for path in (ROOT / "pcie-ep_amd").rglob("*"):
        if path.suffix in (".py", ".hip", ".cpp", ".h") and "build" not in path.parts[len(ROOT.parts):-1]:
            text = path.read_text()
            if re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M) or "oracle/" in text:
                offenders.append(str(path.relative_to(ROOT)))
    assert not offenders, offenders

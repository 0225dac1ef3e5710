"""Build the gfx950 shared library in-tree.

    python pcie-ep_amd/build.py            # compile every source, link the .so
    python pcie-ep_amd/build.py --if-missing
    python pcie-ep_amd/build.py --profiling   # additionally libpcie_ep_amd_profiling.so (per-role timing records)

hipcc cross-compiles for gfx950 without a GPU.  The library lands in
``pcie-ep_amd/pcie_ep/lib/libpcie_ep_amd.so`` so it travels with the tree.
"""

from __future__ import annotations

import argparse
import concurrent.futures
import shutil
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
OUT_DIR = HERE / "pcie_ep" / "lib"
LIBRARY = OUT_DIR / "libpcie_ep_amd.so"
PROFILING_LIBRARY = OUT_DIR / "libpcie_ep_amd_profiling.so"
CLIENT = OUT_DIR / "abi_client"
OBJ_DIR = HERE / "build"

HIP_SOURCES = ["prologue_kernel.hip", "transport_kernel.hip", "expand_kernels.hip", "litmus.hip", "runtime.hip"]
CXX_SOURCES = ["peers.cpp", "relay.cpp"]

COMMON = ["-O3", "-std=c++20", "-fPIC", "-Wall", "-Wno-unused-function", "-pthread"]
# Packed FP32 instructions are disabled for all device code of this build.
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(command: list[str]) -> None:
    result = subprocess.run(command, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    stderr = "\n".join(line for line in result.stderr.splitlines() if noise not in line)
    if result.returncode != 0:
        raise RuntimeError(f"{' '.join(command)}\n{result.stdout}\n{stderr}")
    if stderr.strip():
        print(stderr, file=sys.stderr)


def _compile(name: str, profiling: bool = False) -> Path:
    source = CSRC / name
    target = OBJ_DIR / (name + (".profiling.o" if profiling else ".o"))
    command = ["hipcc", *COMMON]
    if profiling:
        command.append("-DPCIE_EP_ENABLE_PROFILING=1")
    if name.endswith(".hip"):
        command += DEVICE
    command += ["-c", str(source), "-o", str(target)]
    _run(command)
    return target


def _link(objects: list, library: Path) -> None:
    _run(["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-pthread", *map(str, objects), "-o", str(library)])


def build(force: bool = True, profiling: bool = False) -> Path:
    """Compile and link the library; with ``profiling`` also the variant whose
    kernels keep per-role timing records (same sources, -DPCIE_EP_ENABLE_PROFILING=1)."""
    if not force and LIBRARY.exists() and (not profiling or PROFILING_LIBRARY.exists()):
        return LIBRARY
    if shutil.which("hipcc") is None:
        raise RuntimeError("hipcc not found: the HIP extension cannot be built")
    OBJ_DIR.mkdir(exist_ok=True)
    OUT_DIR.mkdir(exist_ok=True)
    sources = HIP_SOURCES + CXX_SOURCES
    with concurrent.futures.ThreadPoolExecutor(max_workers=7) as pool:
        plain = [pool.submit(_compile, name) for name in sources]
        timed = [pool.submit(_compile, name, True) for name in HIP_SOURCES] if profiling else []
        objects = [job.result() for job in plain]
        timed_objects = [job.result() for job in timed]
    _link(objects, LIBRARY)
    if profiling:
        # The host-only sources do not depend on the switch.
        _link(timed_objects + objects[len(HIP_SOURCES):], PROFILING_LIBRARY)
    build_client()
    return LIBRARY


def build_client() -> Path:
    """The torch-free C++ client of the C ABI (tests/abi_client.cpp): plain g++,
    the public header, the HIP runtime API and the library, nothing else."""
    rocm = Path(shutil.which("hipcc")).resolve().parents[1]
    _run(["g++", "-O2", "-std=c++17", "-Wall", "-D__HIP_PLATFORM_AMD__", f"-I{rocm / 'include'}", f"-I{HERE.parent / 'include'}",
          str(HERE.parent / "tests" / "abi_client.cpp"), f"-L{OUT_DIR}", "-lpcie_ep_amd", f"-L{rocm / 'lib'}", "-lamdhip64",
          "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{rocm / 'lib'}", "-o", str(CLIENT)])
    return CLIENT


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("--if-missing", action="store_true")
    parser.add_argument("--profiling", action="store_true")
    arguments = parser.parse_args()
    print(build(force=not arguments.if_missing, profiling=arguments.profiling))

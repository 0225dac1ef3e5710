"""Extract golden vectors from DATA files the reference holds.

Run once in the authoring container (the reference checkout is not present on
the GPU box):  python tests/golden/make_fixtures.py [/root/reference]

Nothing from the reference is imported or executed; only its JSON/NPZ data
files are read (``numpy.load`` with pickling disabled).  Outputs, all in this
directory:

* ``hotspot_20_80_routes.npz`` — byte copy of the reference's frozen hotspot
  top-4 routes (benchmarks/data/top4_skew/hotspot_20_80_routes.npz): indices
  int64 [8,8192,4], weights float32 [8,8192,4].
* ``hotspot_20_80_stats.json`` — for every published T: expert_counts[256],
  rank_expanded_branches[8], rank_unique_received_tokens[8],
  source_destination_unique_tokens[8][8], route_volume and the per-rank
  SHA-256 of route/weight bytes (benchmarks/data/top4_skew/hotspot_20_80_routes.json).
* ``uniform_top8_volumes.json`` — for every published T of the uniform top-8
  generator: per-rank SHA-256 of the route and weight bytes and the U/F/M
  route volume (benchmarks/data/nccl_shm_routes.json).
"""

from __future__ import annotations

import hashlib
import json
import shutil
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent


def main(reference: Path) -> None:
    data = reference / "benchmarks" / "data"
    npz = data / "top4_skew" / "hotspot_20_80_routes.npz"
    manifest = json.loads((data / "top4_skew" / "hotspot_20_80_routes.json").read_text())
    digest = hashlib.sha256(npz.read_bytes()).hexdigest()
    if digest != manifest["tensors_sha256"]:
        raise SystemExit("hotspot route file does not match its manifest digest")
    shutil.copyfile(npz, HERE / "hotspot_20_80_routes.npz")
    arrays = np.load(npz, allow_pickle=False)
    assert arrays["indices"].shape == (8, 8192, 4) and arrays["weights"].shape == (8, 8192, 4)
    hotspot = {
        "source": "benchmarks/data/top4_skew/hotspot_20_80_routes.json",
        "tensors_sha256": manifest["tensors_sha256"],
        "world_size": manifest["world_size"],
        "experts": manifest["experts"],
        "topk": manifest["topk"],
        "design_hot_expert_ids": manifest["probability_model"]["design_hot_expert_ids"],
        "routes": [],
    }
    for entry in manifest["routes"]:
        stats = entry["statistics"]
        hotspot["routes"].append(
            {
                "tokens_per_gpu": entry["tokens_per_gpu"],
                "per_rank": entry["per_rank"],
                "route_volume": entry["route_volume"],
                "expert_counts": stats["expert_counts"],
                "rank_expanded_branches": stats["rank_expanded_branches"],
                "rank_unique_received_tokens": stats["rank_unique_received_tokens"],
                "source_destination_unique_tokens": stats["source_destination_unique_tokens"],
            }
        )
    (HERE / "hotspot_20_80_stats.json").write_text(json.dumps(hotspot, separators=(",", ":")) + "\n")

    uniform = json.loads((data / "nccl_shm_routes.json").read_text())
    volumes = {
        "source": "benchmarks/data/nccl_shm_routes.json",
        "world_size": uniform["world_size"],
        "experts": uniform["experts"],
        "topk": uniform["topk"],
        "seed": uniform["seed"],
        "routes": [
            {
                "tokens_per_gpu": entry["tokens_per_gpu"],
                "per_rank": entry["per_rank"],
                "route_volume": entry["route_volume"],
            }
            for entry in uniform["routes"]
        ],
    }
    (HERE / "uniform_top8_volumes.json").write_text(json.dumps(volumes, separators=(",", ":")) + "\n")


if __name__ == "__main__":
    main(Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference"))

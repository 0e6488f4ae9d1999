"""Benchmark of the Map step (BASELINE configuration 2) on one MI355X.

A step is one kernel-map build from UNSORTED unique voxels to finished
per-offset (in_idx, out_idx) lists: coordinate sort -> 3x3x3 query -> sizes ->
pair lists, all through the C ABI of libminuet_hip.so.  Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0


def map_step(_C, coords_dev, offsets):
    _, sorted_dev, bounds = _C.sort_coordinates(coords_dev, return_bounds=True)
    built = _C.kernel_map_build(sorted_dev, sorted_dev, offsets, None, None, reorder=False,
                                want_masks=False, want_lists=True, source_bounds=bounds,
                                target_bounds=bounds)
    return sorted_dev, built


def cpu_baseline(coords, offsets, budget_s=12.0):
    """The plain-C restatement of the reference algorithm (oracle/oracle_c.c) on
    the host cores, same cloud, for about `budget_s` seconds."""
    import c_oracle
    c_oracle.map_step(coords, offsets)            # warm-up (page faults, thread pool)
    times = []
    start = time.perf_counter()
    while time.perf_counter() - start < budget_s and len(times) < 200:
        t0 = time.perf_counter()
        c_oracle.map_step(coords, offsets)
        times.append(time.perf_counter() - t0)
    return {"value": round(1e3 * float(np.median(times)), 3), "unit": "ms", "cores": c_oracle.num_threads(),
            "kind": "port",
            "sample": f"{len(times)} full Map steps (sort, query, sizes, pair lists) of the same "
                      f"{coords.shape[0]}-voxel cloud; median"}


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=1000)
    parser.add_argument("--warmup", type=int, default=100)
    parser.add_argument("--scale", type=float, default=1.0, help="voxel-count scale of the workload")
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this run has a single MI355X and the "
              "path needs no exchange between GPUs; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import minuet_oracle as orc
    from minuet_amd.nn.functional import _C
    from minuet_amd.synthetic import make_cloud

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda:0")
    cloud = make_cloud(2, scale=args.scale)
    coords = cloud["coords"]
    offsets = orc.generate_kernel_offsets(3, 3, 1, 1)
    offsets32 = offsets.astype(np.int32)
    coords_dev = torch.from_numpy(coords).to(device)
    n = coords.shape[0]

    # bring the GPU out of its idle power state before anything is measured
    spin_until = time.perf_counter() + 1.5
    while time.perf_counter() < spin_until:
        map_step(_C, coords_dev, offsets)
    for _ in range(max(1, args.warmup)):
        sorted_dev, built = map_step(_C, coords_dev, offsets)
    torch.cuda.synchronize()
    nnz = int(built["sizes_host"].sum())

    # parity of what is being timed (bit-exact), once
    order = orc.arg_sort_coordinates(coords)
    ref_sorted = coords[order]
    assert np.array_equal(sorted_dev.cpu().numpy(), ref_sorted)
    import c_oracle
    ref_map = c_oracle.query(ref_sorted, ref_sorted, offsets32)
    ein, eout = c_oracle.pair_lists(ref_map)
    assert np.array_equal(built["in_idx"].cpu().numpy(), ein)
    assert np.array_equal(built["out_idx"].cpu().numpy(), eout)

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        map_step(_C, coords_dev, offsets)
    torch.cuda.synchronize()
    wall_ms = 1e3 * (time.perf_counter() - t0) / args.steps

    # per-stage device time from the library's own stream events
    _C.profile_enable(True)
    stage = {}
    reps = max(10, min(args.steps, 50))
    for _ in range(reps):
        map_step(_C, coords_dev, offsets)
        for name, ms in _C.profile_read():
            stage.setdefault(name, []).append(ms)
    _C.profile_enable(False)
    stage_ms = {k: float(np.median(v)) for k, v in stage.items()}
    device_ms = sum(v for k, v in stage_ms.items() if not k.startswith("enter:"))

    bytes_map = 12 * n + 12 * n + 4 * n + 8 * nnz + 4 * offsets.shape[0]
    bytes_query = 12 * n + 8 * nnz
    query_ms = stage_ms.get("query", float("nan"))
    achieved = bytes_query / (query_ms * 1e-3) / 1e9 if query_ms == query_ms and query_ms > 0 else None
    result = {
        "metric": "Map-step ms + SC layer Mvoxels/s + sparse UNet fwd latency (1 GPU)",
        "value": round(wall_ms, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int64",
        "data": "synthetic",
        "config": {"workload": "config 2: Map step, 3x3x3 submanifold kernel map (27 offsets) from "
                               "unsorted unique voxels to per-offset (in,out) int32 lists",
                   "voxels": n, "nnz": nnz, "generator": cloud["note"], "seed": 1002,
                   "bounding_box": [coords.min(0).tolist(), coords.max(0).tolist()],
                   "mvoxels_per_s": round(n / wall_ms / 1e3, 2)},
        "roofline": {"bound": "hbm", "kernel": "query_kernel",
                     "achieved": None if achieved is None else round(achieved, 2),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": None if achieved is None else round(achieved / HBM_PEAK_GBS, 5),
                     "traffic": None,
                     "algorithmic_bytes": bytes_query,
                     "avg_launch_ms": None if achieved is None else round(query_ms, 5),
                     "map_step": {"algorithmic_bytes": bytes_map,
                                  "device_ms": round(device_ms, 4),
                                  "achieved": round(bytes_map / (wall_ms * 1e-3) / 1e9, 2),
                                  "frac": round(bytes_map / (wall_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 5),
                                  "stage_ms": {k: round(v, 5) for k, v in stage_ms.items()}}},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(coords, offsets32)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()

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


def _time_ms(fn, warmup, reps):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return 1e3 * (time.perf_counter() - t0) / reps


def extras(device):
    """The other two parts of the metric, measured briefly: layer throughput
    (configurations 1 and 3) and sparse UNet forward latency (configuration 4,
    kernel-map cache reset before every forward)."""
    import torch
    import minuet_amd as minuet
    from minuet_amd.nn.functional import _C
    from minuet_amd.synthetic import make_cloud
    from minuet_amd.unet import SparseUNet

    out = {}
    with torch.no_grad():
        # configuration 1: submanifold 3x3x3, 32 -> 32, fp32
        c1 = torch.from_numpy(make_cloud(1)["coords"]).to(device)
        _, s1 = _C.sort_coordinates(c1)
        conv = minuet.nn.SparseConv3d(32, 32, 3, dtype=torch.float32, device=device)
        cache = minuet.nn.KernelMapCache(3, torch.int32, device)
        conv.set_kernel_map_cache(cache)
        conv.tunable_config.update(gather_tile_size=0, scatter_tile_size=0)
        x = minuet.SparseTensor(torch.randn(s1.shape[0], 32, device=device), s1)
        warm = _time_ms(lambda: conv(x), 20, 200)

        def cold1():
            cache.reset()
            conv(x)
        cold = _time_ms(cold1, 20, 200)
        out["config1_layer_fp32"] = {"voxels": int(s1.shape[0]), "ms_map_cached": round(warm, 4),
                                     "ms_map_included": round(cold, 4),
                                     "mvoxels_per_s_map_cached": round(s1.shape[0] / warm / 1e3, 1)}
        # configuration 3: stride-2 down conv 64 -> 128 then transposed 128 -> 64, fp16
        c3 = torch.from_numpy(make_cloud(3)["coords"]).to(device)
        _, s3 = _C.sort_coordinates(c3)
        down = minuet.nn.SparseConv3d(64, 128, 2, stride=2, dtype=torch.float16, device=device)
        up = minuet.nn.SparseConv(3, 128, 64, 2, stride=2, transposed=True, dtype=torch.float16, device=device)
        cache3 = minuet.nn.KernelMapCache(3, torch.int32, device)
        for m in (down, up):
            m.set_kernel_map_cache(cache3)
            m.tunable_config.update(gather_tile_size=0, scatter_tile_size=0)
        x3 = minuet.SparseTensor(torch.randn(s3.shape[0], 64, device=device).half(), s3)
        pair = _time_ms(lambda: up(down(x3)), 20, 200)
        out["config3_down_up_fp16"] = {"voxels": int(s3.shape[0]), "ms_map_cached": round(pair, 4),
                                       "mvoxels_per_s_map_cached": round(s3.shape[0] / pair / 1e3, 1)}
        # configuration 4: sparse UNet forward, fp16, batch of two scans
        cloud = make_cloud(4)
        c4 = torch.from_numpy(cloud["coords"]).to(device)
        bd = torch.from_numpy(cloud["batch_dims"]).to(device)
        _, s4 = _C.sort_coordinates(c4, bd)
        net = SparseUNet(4, 32, dtype=torch.float16, device=device).eval()
        cache4 = minuet.nn.KernelMapCache(3, torch.int32, device)
        minuet.set_kernel_map_cache(net, cache4)
        for m in net.modules():
            if isinstance(m, minuet.nn.SparseConv):
                m.tunable_config.update(gather_tile_size=0, scatter_tile_size=0)
        x4 = minuet.SparseTensor(torch.randn(s4.shape[0], 4, device=device).half(), s4, batch_dims=bd)

        def forward():
            cache4.reset()
            net(x4)
        lat = _time_ms(forward, 5, 30)
        out["config4_unet_fp16"] = {"voxels": int(s4.shape[0]), "batch": 2,
                                    "forward_ms_cold_cache": round(lat, 3)}
    return out


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=1000)
    parser.add_argument("--warmup", type=int, default=100)
    parser.add_argument("--scale", type=float, default=1.0, help="voxel-count scale of the workload")
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    parser.add_argument("--no-extras", action="store_true",
                        help="skip the layer-throughput and UNet-latency side measurements")
    parser.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                        help="also run one plain device copy of this many MiB (a known-size "
                             "reference for scaling profiler byte counters)")
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

    if args.copy_calibration > 0:
        src = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

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
    if not args.no_extras:
        result["extra"] = extras(device)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(coords, offsets32)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()

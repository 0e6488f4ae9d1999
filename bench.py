"""Benchmark of the Map step (BASELINE configuration 2) on one MI355X.

A step is one kernel-map build from UNSORTED unique voxels to finished
per-offset (in_idx, out_idx) lists: coordinate sort -> 3x3x3 query -> sizes ->
pair lists, all through the C ABI of libminuet_hip.so.  Prints one JSON line:
the Map step is `value`; `extra` holds the other parts of the metric (layer
throughput of configurations 1, 3 and 5, sparse UNet forward latency of
configuration 4) and the Gather / grouped GEMM / Scatter kernels one by one
with their algorithmic bytes and flops.
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
MAP_PROFILE = os.path.join(ROOT, "profiles", "map_step_config2_200k_voxels.md")


def kernel_sources_digest():
    """Digest of the HIP sources the library is built from: a profile summary
    records the one it was taken with, so a reader can tell whether counters
    quoted from it belong to the code that is running."""
    import glob
    import hashlib
    digest = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(ROOT, "minuet_amd", "csrc", "*"))):
        digest.update(os.path.basename(path).encode())
        digest.update(open(path, "rb").read())
    return digest.hexdigest()[:16]


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` on this workload at scale 1, from the
    committed rocprofv3 summary (FETCH_SIZE + WRITE_SIZE, each scaled by what
    the counter reads for a plain device copy of known size), and where the
    figure comes from: the counters need a profiler run of their own, so they
    are those of the summary's run, with its date and the digest of the kernel
    sources it profiled beside the digest of the sources at hand.  (None, ...)
    when the summary does not list the kernel."""
    import re
    source = {"file": os.path.relpath(MAP_PROFILE, ROOT), "sources_now": kernel_sources_digest()}
    try:
        text = open(MAP_PROFILE).read()
    except OSError:
        return None, source
    for key in ("date", "sources"):
        found = re.search(rf"^{key}:\s*(\S+)", text, flags=re.M)
        source[f"profile_{key}"] = found.group(1) if found else None
    source["same_sources"] = source.get("profile_sources") == source["sources_now"]
    match = re.search(r"traffic_bytes:\s*(\{.*?\})", text)
    if not match:
        return None, source
    return json.loads(match.group(1)).get(kernel), source


def device_record(_C):
    """What the box is: compute units and clocks as the runtime reports them, and
    the memory ceilings measured here and now with one plain streaming kernel
    each over 512 MiB (copy = bytes read + bytes written per second)."""
    facts = _C.device_facts()
    nbytes = 512 << 20
    ceilings = {}
    for kind, moved in (("copy", 2 * nbytes), ("read", nbytes), ("write", nbytes)):
        ms = min(_C.time_memory(kind, nbytes, repeats=10) for _ in range(3))
        ceilings[kind + "_GBs"] = round(moved / (ms * 1e-3) / 1e9, 1)
    facts["measured_hbm_ceiling"] = dict(ceilings, bytes_per_pass=nbytes,
                                         note="plain 16-byte streaming kernels, 10 back-to-back passes, best of 3")
    facts["vendor_hbm_peak_GBs"] = HBM_PEAK_GBS
    return facts


def map_step(_C, coords_dev, offsets, want_coordinates=False):
    """One Map step: unsorted voxels -> sorted voxels -> per-offset pair lists in
    the order KernelMapCache keeps them (rows by ascending size), one library call."""
    built = _C.sorted_kernel_map_lists(coords_dev, offsets, reorder=True, result_only=True)
    return built["coordinates"] if want_coordinates else None, built


def check_parity(coords, offsets, sorted_dev, built):
    """The timed call's results against the CPU restatement of the reference
    algorithm, bit for bit (sorted voxels, both pair lists).  The only place of
    the measured path that touches the oracle: as the checker."""
    import c_oracle
    import minuet_oracle as orc
    order = orc.arg_sort_coordinates(coords)
    ref_sorted = coords[order]
    assert np.array_equal(sorted_dev.cpu().numpy(), ref_sorted)
    ref_map = c_oracle.query(ref_sorted, ref_sorted, offsets.astype(np.int32))
    ein, eout, _ = orc.kernel_map_pair_lists(ref_map[orc.stable_size_order(orc.compute_kernel_map_sizes(ref_map))])
    assert np.array_equal(built["in_idx"].cpu().numpy(), ein)
    assert np.array_equal(built["out_idx"].cpu().numpy(), eout)


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _median_ms(fn, budget_s, most):
    fn()                                          # warm-up (page faults, thread pool)
    times = []
    start = time.perf_counter()
    while time.perf_counter() - start < budget_s and len(times) < most:
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return 1e3 * float(np.median(times)), len(times)


def cpu_baseline(coords, offsets, budget_s=10.0):
    """The plain-C restatement of the reference algorithm (oracle/oracle_c.c) on
    the host cores: the Map step of the same cloud for about `budget_s` seconds,
    then the layer of configuration 1 (3x3x3, 32 -> 32 channels, fp32: gather,
    per-offset GEMM, scatter, with its kernel map built beforehand)."""
    import c_oracle
    import minuet_oracle as orc
    from minuet_amd.synthetic import make_cloud
    map_ms, map_runs = _median_ms(lambda: c_oracle.map_step(coords, offsets), budget_s, 200)
    c1 = make_cloud(1)["coords"]
    _, s1 = c_oracle.arg_sort(c1)
    dense = c_oracle.query(s1, s1, offsets)
    sizes = c_oracle.sizes(dense)
    order = orc.stable_size_order(sizes)
    sm, tm = c_oracle.masks(dense, s1.shape[0], order)
    rng = np.random.default_rng(1001)
    feats = rng.normal(size=(s1.shape[0], 32)).astype(np.float32)
    weights = (rng.normal(size=(27, 32, 32)) / np.sqrt(27 * 32)).astype(np.float32)
    layer_ms, layer_runs = _median_ms(
        lambda: c_oracle.conv_forward(feats, weights, sm, tm, order, sizes[order]), 5.0, 200)
    return {"value": round(map_ms, 3), "unit": "ms", "cores": c_oracle.num_threads(),
            "kind": "port", "cpu_model": cpu_model(), "host_cpus": os.cpu_count(),
            "sample": f"{map_runs} full Map steps (sort, query, sizes, pair lists) of the same "
                      f"{coords.shape[0]}-voxel cloud; median",
            "config1_layer_fp32": {"ms": round(layer_ms, 3), "voxels": int(s1.shape[0]),
                                   "mvoxels_per_s": round(s1.shape[0] / layer_ms / 1e3, 2),
                                   "sample": f"{layer_runs} forward passes of the configuration-1 layer "
                                             f"(gather, 27 GEMMs, scatter; kernel map cached); median"}}


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


def _time_stats(fn, warmup, reps):
    """Wall mean over `reps` back-to-back calls plus the distribution of the
    per-call time between stream events (the events sit on torch's current
    stream, the one the library is given)."""
    import torch
    mean = _time_ms(fn, warmup, reps)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    marks[0].record()
    for i in range(reps):
        fn()
        marks[i + 1].record()
    torch.cuda.synchronize()
    each = np.array([marks[i].elapsed_time(marks[i + 1]) for i in range(reps)])
    return {"ms_mean": round(mean, 4), "ms_median": round(float(np.median(each)), 4),
            "ms_p10": round(float(np.percentile(each, 10)), 4),
            "ms_p90": round(float(np.percentile(each, 90)), 4), "iterations": reps}


MFMA_PEAK_TFLOPS = {"fp16": 2500.0, "bf16": 2500.0, "fp32": 157.3}


def layer_stages(device, config, channels, kernel_size, dtype_name, tune=False):
    """Gather, grouped GEMM and Scatter timed one by one through the library's
    stage timers (the reference's cuda_time_* interface), then the whole layer
    through both dataflows, with the algorithmic bytes / flops of each."""
    import torch
    import minuet_amd as minuet
    from minuet_amd.nn import functional as F
    from minuet_amd.nn.functional import _C
    from minuet_amd.synthetic import make_cloud

    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}[dtype_name]
    esize = torch.empty(0, dtype=dtype).element_size()
    coords = torch.from_numpy(make_cloud(config)["coords"]).to(device)
    _, sorted_dev = _C.sort_coordinates(coords)
    conv = minuet.nn.SparseConv3d(channels, channels, kernel_size, dtype=dtype, device=device)
    cache = minuet.nn.KernelMapCache(3, torch.int32, device)
    conv.set_kernel_map_cache(cache)
    x = minuet.SparseTensor(torch.randn(sorted_dev.shape[0], channels, device=device).to(dtype), sorted_dev)
    with torch.no_grad():
        conv.tunable_config["dataflow"] = "gather_gemm_scatter"     # builds the rank tables
        conv(x)
        kernel_map = next(iter(cache._kernel_maps_cache.values()))
        source_masks, target_masks, order, sizes = kernel_map
        host_sizes = np.asarray(kernel_map.sizes_host, dtype=np.int64)
        voxels = int(sorted_dev.shape[0])
        nnz = int(host_sizes.sum())
        moved = nnz - voxels                       # the centre offset takes the shortcut
        args = dict(weights=conv.kernel, source_masks=source_masks, target_masks=target_masks,
                    kernel_map_sizes=sizes, allow_shortcut_matmul=True, threshold=-1)
        med = lambda timer, **kw: float(np.median([timer(**args, **kw) for _ in range(15)]))
        gather_ms = med(F.cuda_time_gather, tile_size=0)
        scatter_ms = med(F.cuda_time_scatter, tile_size=0)
        gemm_ms = med(F.cuda_time_gemm)
        # second clock: 20 launches back to back between the two events, time of
        # one (no launch gap inside the interval: what a kernel trace shows per launch)
        _C.timer_repeats(20)
        try:
            gather_b2b = med(F.cuda_time_gather, tile_size=0)
            scatter_b2b = med(F.cuda_time_scatter, tile_size=0)
            gemm_b2b = med(F.cuda_time_gemm)
        finally:
            _C.timer_repeats(1)
        bytes_gather = voxels * channels * esize + moved * channels * esize + 4 * moved
        bytes_scatter = moved * channels * esize + voxels * channels * esize + 4 * moved
        flops = 2.0 * nnz * channels * channels
        out = {"voxels": voxels, "nnz": nnz, "channels": channels, "dtype": dtype_name,
               "offsets": int(host_sizes.shape[0])}

        def hbm(nbytes, ms, ms_b2b=None):
            gbs = nbytes / (ms * 1e-3) / 1e9
            rec = {"ms": round(ms, 4), "algorithmic_bytes": int(nbytes), "achieved_GBs": round(gbs, 1),
                   "frac_of_8TBs": round(gbs / HBM_PEAK_GBS, 4)}
            if ms_b2b is not None:
                rec.update(ms_back_to_back=round(ms_b2b, 4),
                           frac_of_8TBs_back_to_back=round(nbytes / (ms_b2b * 1e-3) / 1e9 / HBM_PEAK_GBS, 4))
            return rec
        out["clocks"] = ("ms: one launch between two stream events (the reference's cuda_time_* protocol, "
                         "launch gap included); ms_back_to_back: 20 launches between the events, time of one")
        out["gather_kernel"] = hbm(bytes_gather, gather_ms, gather_b2b)
        out["scatter_kernel"] = hbm(bytes_scatter, scatter_ms, scatter_b2b)
        tflops = flops / (gemm_ms * 1e-3) / 1e12
        out["grouped_gemm_kernel"] = {"ms": round(gemm_ms, 4), "ms_back_to_back": round(gemm_b2b, 4),
                                      "flops": flops, "achieved_TFLOPs": round(tflops, 1),
                                      "frac_of_mfma_peak": round(tflops / MFMA_PEAK_TFLOPS[dtype_name], 4),
                                      "frac_of_mfma_peak_back_to_back": round(
                                          flops / (gemm_b2b * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS[dtype_name], 4),
                                      # rows in and out of the buffers: what bounds it at small widths
                                      **{"hbm_" + k: v for k, v in hbm(2 * nnz * channels * esize, gemm_ms).items()
                                         if k != "ms"}}
        for flow in ("gather_gemm_scatter", "list_driven", "implicit", "offset_groups"):
            if flow == "implicit" and not _C.implicit_forward_supported(channels, channels, dtype):
                continue
            if flow == "offset_groups" and not (conv.kernel.shape[0] == 27 and _C.offset_groups_forward_supported(
                    channels, channels, dtype)):
                continue
            conv.tunable_config["dataflow"] = flow
            if flow == "list_driven":
                # its Scatter alone, from the library's stage marks: target-major row lists,
                # every hit's product row read once (the centre offset's too), no rank table
                for _ in range(5):
                    conv(x)
                _C.profile_enable(True)
                marks = []
                for _ in range(15):
                    conv(x)
                    marks += [ms for name, ms in _C.profile_read() if name == "scatter"]
                _C.profile_enable(False)
                if marks:
                    rows_bytes = nnz * channels * esize + voxels * channels * esize + 4 * (voxels + 1)
                    out["scatter_rows_kernel"] = hbm(rows_bytes, float(np.median(marks)))
            stats = _time_stats(lambda: conv(x), 10, 50)
            stats["mvoxels_per_s"] = round(voxels / stats["ms_mean"] / 1e3, 1)
            stats["achieved_TFLOPs"] = round(flops / (stats["ms_mean"] * 1e-3) / 1e12, 1)
            out["layer_" + flow] = stats
        if tune:
            # the layer's own autotuner (padding threshold, gather / scatter tile, dataflow)
            # on this workload, then the layer as tuned
            conv.tunable_config.update(dataflow="auto", threshold=-1, gather_tile_size=0, scatter_tile_size=0)
            t0 = time.perf_counter()
            minuet.autotune(conv, cache, [x])
            seconds = time.perf_counter() - t0
            cache.reset()
            tuned = dict(conv.tunable_config)
            stats = _time_stats(lambda: conv(x), 10, 50)
            stats["mvoxels_per_s"] = round(voxels / stats["ms_mean"] / 1e3, 1)
            # rows of the GEMM buffers under the padding plans the threshold chooses between
            # (padded rows are laid out, never computed: the kernel's tiles stop at each group's size)
            sizes_list = [int(v) for v in host_sizes[:-1]]          # the centre offset takes the shortcut
            plans = {}
            for name, threshold in (("none (-1)", -1), ("0.5", 0.5), ("one bucket (None)", None)):
                buckets = _C.generate_padding_buckets(sizes_list, threshold)
                rows = _C.cumsum_kernel_padded_sizes(sizes_list, buckets)[-1]
                plans[name] = {"buckets": len(buckets) - 1, "buffer_rows": int(rows),
                               "padding_waste": round(rows / max(1, sum(sizes_list)) - 1.0, 4)}
            out["autotune"] = {"seconds": round(seconds, 2), "tuned_config": tuned, "layer_as_tuned": stats,
                               "padding_plans": plans, "group_sizes_min_median_max": [
                                   int(host_sizes.min()), int(np.median(host_sizes)), int(host_sizes.max())]}
    return out


def extras(device, with_config5, section="all"):
    """The other two parts of the metric: layer throughput (configurations 1, 3
    and 5, kernel map cached and included) and sparse UNet forward latency
    (configuration 4, kernel-map cache reset before every forward); plus the
    Gather / GEMM / Scatter kernels one by one on the configuration-2 cloud."""
    import torch
    import minuet_amd as minuet
    from minuet_amd.nn.functional import _C
    from minuet_amd.synthetic import make_cloud
    from minuet_amd.unet import SparseUNet

    out = {}
    if section == "layer-kernels":
        return {"config2_layer_kernels_fp16_c64": layer_stages(device, 2, 64, 3, "fp16")}
    if section == "config5":
        return {"config5_layer_bf16_c64_k5": layer_stages(device, 5, 64, 5, "bf16", tune=True)}
    with torch.no_grad():
        # The configuration-2 cloud through the cache a NETWORK uses: what a layer pays
        # for its map on an unsorted cloud.  A single-kernel layer asks for the dense
        # map [27, N] alone; a Gather-GEMM-Scatter layer for dense map, both rank
        # tables, sizes, order and the pair lists.  (The headline times the lists-only
        # build, which is the output configuration 2 names.)
        c2 = torch.from_numpy(make_cloud(2)["coords"]).to(device)
        cache2 = minuet.nn.KernelMapCache(3, torch.int32, device)

        def through_cache(tables):
            def run():
                cache2.reset()
                _, s2 = _C.sort_coordinates(c2)
                if tables:
                    cache2.get_kernel_map(s2, 1, None, s2, 1, None, 3, 1)
                else:
                    cache2.get_dense_kernel_map(s2, 1, None, s2, 1, None, 3, 1)
            return run
        out["config2_map_through_kernel_map_cache"] = {
            "voxels": int(c2.shape[0]),
            "sort+dense_map (single-kernel layers)": _time_stats(through_cache(False), 10, 100),
            "sort+dense_map+rank_tables+lists (gather-GEMM-scatter layers)": _time_stats(through_cache(True), 10, 100)}
        cache2.reset()
        del c2, cache2
        # configuration 1: submanifold 3x3x3, 32 -> 32, fp32
        c1 = torch.from_numpy(make_cloud(1)["coords"]).to(device)
        _, s1 = _C.sort_coordinates(c1)
        conv = minuet.nn.SparseConv3d(32, 32, 3, dtype=torch.float32, device=device)
        cache = minuet.nn.KernelMapCache(3, torch.int32, device)
        conv.set_kernel_map_cache(cache)
        x = minuet.SparseTensor(torch.randn(s1.shape[0], 32, device=device), s1)
        warm = _time_stats(lambda: conv(x), 20, 200)

        def cold1():
            cache.reset()
            conv(x)
        cold = _time_stats(cold1, 20, 200)
        out["config1_layer_fp32"] = {"voxels": int(s1.shape[0]), "map_cached": warm, "map_included": cold,
                                     "mvoxels_per_s_map_cached": round(s1.shape[0] / warm["ms_mean"] / 1e3, 1),
                                     "mvoxels_per_s_map_included": round(s1.shape[0] / cold["ms_mean"] / 1e3, 1)}
        # configuration 3: stride-2 down conv 64 -> 128 then transposed 128 -> 64, fp16
        c3 = torch.from_numpy(make_cloud(3)["coords"]).to(device)
        _, s3 = _C.sort_coordinates(c3)
        down = minuet.nn.SparseConv3d(64, 128, 2, stride=2, dtype=torch.float16, device=device)
        up = minuet.nn.SparseConv(3, 128, 64, 2, stride=2, transposed=True, dtype=torch.float16, device=device)
        cache3 = minuet.nn.KernelMapCache(3, torch.int32, device)
        for m in (down, up):
            m.set_kernel_map_cache(cache3)
        x3 = minuet.SparseTensor(torch.randn(s3.shape[0], 64, device=device).half(), s3)
        pair = _time_stats(lambda: up(down(x3)), 20, 200)

        def cold3():
            cache3.reset()
            up(down(x3))
        pair_cold = _time_stats(cold3, 10, 100)
        out["config3_down_up_fp16"] = {"voxels": int(s3.shape[0]), "map_cached": pair, "map_included": pair_cold,
                                       "mvoxels_per_s_map_cached": round(s3.shape[0] / pair["ms_mean"] / 1e3, 1)}
        # configuration 4: sparse UNet forward, fp16, batch of two scans
        cloud = make_cloud(4)
        c4 = torch.from_numpy(cloud["coords"]).to(device)
        bd = torch.from_numpy(cloud["batch_dims"]).to(device)
        _, s4 = _C.sort_coordinates(c4, bd)
        net = SparseUNet(4, 32, dtype=torch.float16, device=device).eval()
        cache4 = minuet.nn.KernelMapCache(3, torch.int32, device)
        minuet.set_kernel_map_cache(net, cache4)
        x4 = minuet.SparseTensor(torch.randn(s4.shape[0], 4, device=device).half(), s4, batch_dims=bd)

        def forward():
            cache4.reset()
            net(x4)
        lat = _time_stats(forward, 5, 50)
        kept = _time_stats(lambda: net(x4), 5, 50)
        # the same pass with cached maps, replayed as one HIP graph
        try:
            graphed = minuet.capture_forward(lambda: net(x4))
            replayed = _time_stats(graphed.replay, 5, 50)
            del graphed
        except Exception as error:          # reported, never fatal for the headline
            replayed = {"error": str(error)[:200]}
        # cold passes again with the cache's look-ahead: from the second pass on the
        # worker thread builds levels and maps beside the layers (same results)
        ahead4 = minuet.nn.KernelMapCache(3, torch.int32, device, lookahead=True)
        minuet.set_kernel_map_cache(net, ahead4)

        passes = [0]

        def forward_ahead():
            ahead4.reset()
            net(x4)
            passes[0] += 1
        try:
            lat_ahead = _time_stats(forward_ahead, 5, 50)
            # the very first pass has no recipe yet and builds everything itself
            lat_ahead["map_builds_taken_from_the_worker_per_pass"] = round(
                ahead4.num_ahead_hits / max(1, passes[0] - 1), 1)
            ahead4.reset()
        except Exception as error:
            lat_ahead = {"error": str(error)[:200]}
        out["config4_unet_fp16"] = {"voxels": int(s4.shape[0]), "batch": 2, "cold_cache": lat,
                                    "cold_cache_lookahead": lat_ahead,
                                    "kernel_maps_cached": kept,
                                    "kernel_maps_cached_graph_replay": replayed,
                                    "forward_ms_cold_cache": lat["ms_median"],
                                    "forward_ms_cold_cache_lookahead": lat_ahead.get("ms_median")}
        del net, cache4, ahead4, x4
    if section == "unet":
        return {"config4_unet_fp16": out["config4_unet_fp16"]}
    out["config2_layer_kernels_fp16_c64"] = layer_stages(device, 2, 64, 3, "fp16")
    if with_config5:
        out["config5_layer_bf16_c64_k5"] = layer_stages(device, 5, 64, 5, "bf16", tune=True)
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
    parser.add_argument("--no-config5", action="store_true",
                        help="skip the 1M-voxel 5x5x5 layer of configuration 5 (half a minute of "
                             "cloud generation)")
    parser.add_argument("--section", default="all",
                        choices=["all", "layer-kernels", "config5", "unet"],
                        help="which of the side measurements to run (profiles isolate one)")
    parser.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                        help="also run one plain device copy of this many MiB (a known-size "
                             "reference for scaling profiler byte counters)")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this run has a single MI355X and the "
              "path needs no exchange between GPUs; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from minuet_amd.nn.functional import _C
    from minuet_amd.synthetic import make_cloud
    from minuet_amd.utils.helpers import generate_kernel_offsets

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda:0")
    cloud = make_cloud(2, scale=args.scale)
    coords = cloud["coords"]
    offsets = np.ascontiguousarray(generate_kernel_offsets(3, 3, 1, 1), dtype=np.int64)
    coords_dev = torch.from_numpy(coords).to(device)
    n = coords.shape[0]

    if args.copy_calibration > 0:
        src = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # parity of what is being timed (bit-exact against the CPU restatement), once,
    # BEFORE the timed region: the check keeps the host busy for a while, and the
    # warm-up has to come right before the steps that are timed
    sorted_dev, built = map_step(_C, coords_dev, offsets, want_coordinates=True)
    torch.cuda.synchronize()
    nnz = int(built["sizes_host"].sum())
    check_parity(coords, offsets, sorted_dev, built)
    device_facts = device_record(_C)

    # bring the GPU out of its idle power state, then the W untimed steps, then
    # exactly K timed steps between two device-wide waits
    spin_until = time.perf_counter() + 1.5
    while time.perf_counter() < spin_until:
        map_step(_C, coords_dev, offsets)
    for _ in range(max(1, args.warmup)):
        map_step(_C, coords_dev, offsets)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        map_step(_C, coords_dev, offsets)
    torch.cuda.synchronize()
    wall_ms = 1e3 * (time.perf_counter() - t0) / args.steps
    # the same step one by one: stream events between the calls, at least 50 of them
    step_stats = _time_stats(lambda: map_step(_C, coords_dev, offsets), 10, max(50, min(args.steps, 500)))
    # how often a step makes the host wait for the device (the library's own tally)
    _C.host_wait_stats(reset=True)
    for _ in range(50):
        map_step(_C, coords_dev, offsets)
    waits, waited_s = _C.host_wait_stats(reset=True)
    step_stats["host_waits_per_step"] = round(waits / 50, 2)
    step_stats["host_wait_ms_per_step"] = round(1e3 * waited_s / 50, 4)

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
    traffic, traffic_source = measured_traffic("query_kernel") if args.scale == 1.0 else (None, None)
    copy_ceiling = device_facts["measured_hbm_ceiling"]["copy_GBs"]
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
                   "mvoxels_per_s": round(n / wall_ms / 1e3, 2),
                   "list_order": "rows by ascending size (what KernelMapCache keeps)"},
        "step_stats": step_stats,
        "roofline": {"bound": "hbm", "kernel": "query_kernel",
                     "achieved": None if achieved is None else round(achieved, 2),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": None if achieved is None else round(achieved / HBM_PEAK_GBS, 5),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "frac_of_measured_copy_ceiling": None if achieved is None else round(achieved / copy_ceiling, 5),
                     "algorithmic_bytes": bytes_query,
                     "avg_launch_ms": None if achieved is None else round(query_ms, 5),
                     "map_step": {"algorithmic_bytes": bytes_map,
                                  "device_ms": round(device_ms, 4),
                                  "achieved": round(bytes_map / (wall_ms * 1e-3) / 1e9, 2),
                                  "frac": round(bytes_map / (wall_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 5),
                                  "stage_ms": {k: round(v, 5) for k, v in stage_ms.items()}}},
    }
    result["device"] = device_facts
    if not args.no_extras:
        result["extra"] = extras(device, not args.no_config5, args.section)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(coords, offsets.astype(np.int32))
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the spatial-search hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--ops all|headline] [--no-cpu]

Prints ONE JSON line.  The headline ("metric"/"value") is BASELINE.json's configs[1]:
furthest point sampling of B=16 clouds of 16384 points down to 4096 samples, in ms per batch
(one step = one pass over the batch, inputs resident in HBM).  The same line carries, under
"ops", the other configurations of BASELINE.json (ball query dense / partial_dense, three_nn,
three_interpolate fwd+bwd, grouping fwd+bwd, Chamfer fwd+bwd), each with its own roofline
figure, and under "cpu_baseline" the reference's CPU implementation timed on this host.

Timing: per-launch durations come from HIP events recorded on the stream the kernels are
launched on (PyTorch's current stream, which is the stream the extension passes to the C
ABI); the headline value is wall-clock time of exactly K steps between two device
synchronisations.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "torch-points-kernels_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

# Published MI355X peaks used for the roofline fractions.
PEAK_HBM_GBS = 8000.0
PEAK_FP32_TFLOPS = 157.3  # published fp32 figure (vector = matrix); it counts every lane-op as an FMA (2 flop)

PROFILES = os.path.join(ROOT, "profiles")
TRAFFIC_FILE = os.path.join(PROFILES, "all_ops_baseline_configs_hbm_traffic.txt")
VALU_FILE = os.path.join(PROFILES, "distance_scans_valu_utilisation.txt")

# Kernels whose HBM traffic adds up to one launch of an operator (names as rocprofv3 prints them).
TRAFFIC_KERNELS = {
    "fps": ["fps_pruned_kernel<16, 1024, 4>"],
    "three_interpolate_fwd": ["gather_fwd_lds_kernel<3, true, int, true>"],
    "three_interpolate_bwd": ["build_lists_kernel<3, true, int>", "gather_bwd_lists_kernel<3, true, 2>"],
    "three_interpolate_bwd_lists": ["gather_bwd_lists_kernel<3, true, 2>"],
    "grouping_bwd_lists": ["gather_bwd_lists_kernel<1, false, 1>"],
    "grouping_fwd": ["gather_fwd_lds_kernel<1, false, long, false>"],
    "grouping_bwd": ["build_lists_kernel<1, false, long>", "gather_bwd_lists_kernel<1, false, 1>"],
    "chamfer_bwd": ["chamfer_bwd_chains_kernel<float>"],
}
# Kernels whose VALU counters describe a distance scan.
VALU_KERNELS = {
    "fps": "fps_pruned_kernel<16, 1024, 4>",
    "ball_query_dense": "ball_query_dense_cells_kernel<false>",
    "ball_query_partial_dense": "ball_query_bins_kernel<false, false>",
    "three_nn": "three_nn_cells_kernel",
    "chamfer_fwd": "chamfer_grid_kernel",
}


def _profile_table(path, columns):
    """Rows 'kernel name  n= k  COUNTER value ...' of a summary under profiles/ -> {kernel: {COUNTER: value}},
    plus the commit the summary says it was measured at."""
    import re

    table, commit = {}, None
    if not os.path.exists(path):
        return table, commit
    for line in open(path):
        m = re.match(r"Measured at commit\s+(\S+)", line)
        if m:
            commit = m.group(1)
        m = re.match(r"(\S.*?)\s+n=\s*(\d+)\s+(.*)$", line)
        if not m:
            continue
        vals = {}
        for name in columns:
            v = re.search(r"\b%s\s+([0-9.eE+-]+)" % re.escape(name), m.group(3))
            if v:
                vals[name] = float(v.group(1))
        if vals:
            table[m.group(1).strip()] = vals
    return table, commit


_TRAFFIC_TABLE = None


def _measured_traffic(key):
    """HBM bytes per launch of operator `key`: 2 x FETCH_SIZE + WRITE_SIZE (KiB, factors from the copy
    kernel of known size in the same runs) summed over the operator's kernels, read from the tracked
    rocprofv3 summary, with the commit it was measured at.  (None, None) when the summary lacks a kernel:
    a renamed or re-shaped kernel thus drops its figure instead of keeping a stale one."""
    global _TRAFFIC_TABLE
    if _TRAFFIC_TABLE is None:
        _TRAFFIC_TABLE = _profile_table(TRAFFIC_FILE, ("FETCH_SIZE", "WRITE_SIZE"))
    table, commit = _TRAFFIC_TABLE
    total = 0.0
    for kernel in TRAFFIC_KERNELS.get(key, []):
        row = table.get(kernel)
        if row is None or "FETCH_SIZE" not in row or "WRITE_SIZE" not in row:
            return None, commit
        total += (2.0 * row["FETCH_SIZE"] + row["WRITE_SIZE"]) * 1024.0
    return (total if key in TRAFFIC_KERNELS else None), commit


_VALU_TABLE = None


def _measured_valu(key):
    global _VALU_TABLE
    if _VALU_TABLE is None:
        _VALU_TABLE = _profile_table(VALU_FILE, ("VALUBusy", "VALUUtilization", "SQ_INSTS_VALU"))
    table, commit = _VALU_TABLE
    row = table.get(VALU_KERNELS.get(key, ""))
    if row is None:
        return None
    return {"valu_busy_pct": row.get("VALUBusy"), "valu_lane_utilisation_pct": row.get("VALUUtilization"),
            "source": "profiles/" + os.path.basename(VALU_FILE), "measured_at_commit": commit}


def _time_gpu(fn, steps, warmup):
    """Returns (wall ms per step, mean HIP-event ms per step)."""
    import torch

    for _ in range(warmup):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    ev = sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / steps
    return wall, ev


def _roof_flops(executed, algorithmic, flops_each, ms, key=None):
    """Roofline object of a distance scan.  `executed` = pair evaluations (or point updates) the kernels
    performed, counted by the counting build of the library in a run outside the timed region;
    `algorithmic` = what a brute-force scan - the reference - performs.  achieved / frac use EXECUTED work,
    so frac <= 1; the algorithmic rate is reported beside it."""
    achieved = executed * flops_each / (ms * 1e-3) / 1e12
    algorithmic_rate = algorithmic * flops_each / (ms * 1e-3) / 1e12
    r = {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
         "frac": achieved / PEAK_FP32_TFLOPS, "traffic": None,
         "executed_pairs": executed, "algorithmic_pairs": algorithmic,
         "algorithmic_rate": algorithmic_rate, "algorithmic_speedup": algorithmic / max(executed, 1),
         "note": "fp32 VALU kernel (inner dimension 3, unfused arithmetic: no MFMA, no FMA, no packed fp32); peak is the "
                 "published fp32 figure, which assumes FMA: without FMA the ceiling is 0.5. achieved = executed pair "
                 "evaluations (counted on device by libtpk_hip_counting.so, one count per lane and distance, padding "
                 "lanes included) x %d flop / kernel time; algorithmic_rate = the pairs a brute-force scan tests "
                 "(what the reference evaluates) x %d flop / the same time; algorithmic_speedup = their ratio" %
                 (flops_each, flops_each)}
    valu = _measured_valu(key) if key else None
    if valu:
        r["valu"] = valu
    return r


PRUNED_NOTE = ("; the kernel orders the clouds along a space filling curve and skips cells that provably hold no "
               "answer; kernel_ms covers the ordering kernel and the search kernel")


def _roof_bytes(nbytes, ms, key):
    achieved = nbytes / (ms * 1e-3) / 1e9
    traffic, commit = _measured_traffic(key)
    r = {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
         "frac": achieved / PEAK_HBM_GBS, "traffic": traffic}
    if traffic is not None:
        r["traffic_source"] = "profiles/" + os.path.basename(TRAFFIC_FILE)
        r["traffic_measured_at_commit"] = commit
    return r


# ---- executed work: the same call made once through the counting build of the library (ctypes on the
# C ABI, PyTorch's current stream), outside every timed region
_COUNTING = None


def _counting_lib():
    global _COUNTING
    if _COUNTING is None:
        import ctypes

        path = os.path.join(ROOT, "torch-points-kernels_amd", "torch_points_kernels", "libtpk_hip_counting.so")
        if not os.path.exists(path):
            sys.exit("bench.py: %s is not built (run torch-points-kernels_amd/build.py)" % path)
        lib = ctypes.CDLL(path)
        for name in ("tpk_fps_workspace_bytes", "tpk_ball_query_partial_workspace_bytes", "tpk_three_nn_workspace_bytes",
                     "tpk_chamfer_fwd_workspace_bytes", "tpk_knn_workspace_bytes",
                     "tpk_ball_query_sorted_dense_workspace_bytes", "tpk_ball_query_sorted_partial_workspace_bytes"):
            getattr(lib, name).restype = ctypes.c_size_t
        _COUNTING = lib
    return _COUNTING


_SHIPPING = None


def _shipping_lib():
    """The shipping library through ctypes: for calls the extension never makes (workspace == NULL, which
    selects the brute-force scans)."""
    global _SHIPPING
    if _SHIPPING is None:
        import ctypes

        _SHIPPING = ctypes.CDLL(os.path.join(ROOT, "torch-points-kernels_amd", "torch_points_kernels", "libtpk_hip.so"))
    return _SHIPPING


def _all_pairs_entry(call, pairs, steps, warmup, valu_kernel):
    """Times call(lib, stream) made without workspace (brute-force scan) and counts its executed pairs."""
    import ctypes

    import torch

    lib = _shipping_lib()

    def run():
        st = call(lib, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert st == 0

    wall, ev = _time_gpu(run, steps, warmup)
    executed = _executed(call)
    roof = _roof_flops(executed, pairs, 8, ev)
    table, commit = _profile_table(VALU_FILE, ("VALUBusy", "VALUUtilization"))
    # the instance a launch picks depends on the sizes: take whichever of the named instances the summary holds
    names = [k for k in ((valu_kernel,) if isinstance(valu_kernel, str) else valu_kernel) if k in table]
    if names:
        valu_kernel = names[0]
        roof["valu"] = {"kernel": valu_kernel, "valu_busy_pct": table[valu_kernel].get("VALUBusy"),
                        "valu_lane_utilisation_pct": table[valu_kernel].get("VALUUtilization"),
                        "source": "profiles/" + os.path.basename(VALU_FILE), "measured_at_commit": commit}
    return {"what": "the same configuration through the C ABI's scan of all pairs (workspace == NULL; three_nn: "
                    "tpk_three_nn_all_pairs_f32): every query scans its whole cloud "
                    "(the kernel the north star describes); same results", "kernel_ms": ev, "wall_ms": wall, "roofline": roof}


COUNT_WORK = True  # --no-count: leave the counting build out (profiler runs: its kernels carry the same names)


def _executed(call):
    """Pair evaluations executed by call(lib, stream) -> status."""
    import ctypes

    import torch

    if not COUNT_WORK:
        return 0
    lib = _counting_lib()
    n = ctypes.c_ulonglong(0)
    assert lib.tpk_work_read_reset(ctypes.byref(n)) == 0
    st = call(lib, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0, "counting call failed with status %d" % st
    assert lib.tpk_work_read_reset(ctypes.byref(n)) == 0
    return int(n.value)


def _autograd_split(forward_recording, backward_from_lists, nbytes, steps, warmup, key):
    """The two halves of a gather's training step as autograd runs them: the forward pass that also inverts the index
    and the backward pass that walks the lists."""
    wall_f, ev_f = _time_gpu(forward_recording, steps, warmup)
    lists = forward_recording()[1]
    wall_b, ev_b = _time_gpu(lambda: backward_from_lists(lists), steps, warmup)
    return {"what": "forward pass with autograd recording (gather, then the lists for the backward pass), then the backward "
                    "pass over those lists", "forward_kernel_ms": ev_f, "forward_wall_ms": wall_f, "backward_kernel_ms": ev_b,
            "backward_wall_ms": wall_b, "backward_roofline": _roof_bytes(nbytes, ev_b, key)}


def _p(t):
    import ctypes

    return ctypes.c_void_p(t.data_ptr())


def _ws(nbytes, dev):
    import torch

    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=dev)


def _cpu_time(fn, repeat=1):
    best = None
    for _ in range(repeat):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None or dt < best else best
    return best


def bench_fps(dev, steps, warmup, with_cpu):
    import ctypes

    import torch

    import torch_points_kernels as tpk
    from tests import workloads as W

    w = W.cfg2_fps()
    xyz = w["xyz"].to(dev)
    npoint = w["npoint"]
    wall, ev = _time_gpu(lambda: tpk.furthest_point_sample(xyz, npoint), steps, warmup)
    updates = W.fps_point_updates()
    out_idx = torch.empty(xyz.shape[0], npoint, dtype=torch.int32, device=dev)
    executed = _executed(lambda lib, st: lib.tpk_fps_f32(xyz.shape[0], xyz.shape[1], npoint, _p(xyz), None,
                                                         ctypes.c_size_t(0), _p(out_idx), st))
    roof = _roof_flops(executed, updates, 10, ev, "fps")
    roof["traffic"], commit = _measured_traffic("fps")
    if roof["traffic"] is not None:
        roof["traffic_source"] = "profiles/" + os.path.basename(TRAFFIC_FILE)
        roof["traffic_measured_at_commit"] = commit
    roof["note"] += "; here a pair = one running minimum updated (10 flop: 8 for the distance, min, max); algorithmic " \
                    "work = every point updated in every round, as the reference does; the kernel skips updates it " \
                    "proves to be no-ops and takes up to 16 samples per round (the points with the largest running minima, as " \
                    "long as none changes the next one's minimum: the same samples in the same order); the rounds " \
                    "of a cloud are sequential and one workgroup owns a cloud: 16 of 256 " \
                    "compute units are occupied by design, executed fraction of those 16 CUs' peak = %.4f, " \
                    "algorithmic %.4f" % (roof["frac"] * 256 / 16, roof["algorithmic_rate"] / PEAK_FP32_TFLOPS * 256 / 16)
    res = {"wall_ms": wall, "kernel_ms": ev, "roofline": roof, "point_updates": updates}
    if with_cpu:
        import oracle

        ref = oracle.ref()
        threads = torch.get_num_threads()
        if ref is not None:
            # the reference's CPU FPS (cpu/src/fps.cpp), started at index 0, full batch
            secs = _cpu_time(lambda: ref.fps(w["xyz"], npoint, False))
            res["cpu_baseline"] = {"value": secs * 1e3, "unit": "ms/batch", "cores": threads, "kind": "reference",
                                   "sample": "the whole configs[1] batch (16 clouds x 16384 points, 4096 samples), "
                                             "reference cpu/src/fps.cpp compiled -O3, ATen ops on %d threads" % threads}
        else:
            clouds = 4
            secs = _cpu_time(lambda: oracle.furthest_point_sample(w["xyz"][:clouds].numpy(), npoint))
            res["cpu_baseline"] = {"value": secs * 1e3 * (16 / clouds), "unit": "ms/batch", "cores": 1, "kind": "port",
                                   "sample": "%d of 16 clouds timed, scaled to the batch; scalar C restatement" % clouds}
    return res


def bench_others(dev, steps, warmup, with_cpu):
    import ctypes

    import torch

    import torch_points_kernels as tpk
    from tests import workloads as W
    from torch_points_kernels._native import native

    nat = native()
    out = {}
    ref = None
    if with_cpu:
        import oracle

        ref = oracle.ref()

    # configs[0]: dense ball query
    w = W.cfg1_ball_query_dense()
    xyz, new_xyz = w["xyz"].to(dev), w["new_xyz"].to(dev)
    wall, ev = _time_gpu(lambda: tpk.ball_query(w["radius"], w["nsample"], xyz, new_xyz, mode="dense"), steps, warmup)
    nq = new_xyz.shape[0] * new_xyz.shape[1]
    pairs = nq * xyz.shape[1]
    bq_idx = torch.empty(new_xyz.shape[0], new_xyz.shape[1], w["nsample"], dtype=torch.int64, device=dev)
    bq_dist = torch.empty(new_xyz.shape[0], new_xyz.shape[1], w["nsample"], device=dev)
    executed = _executed(lambda lib, st: lib.tpk_ball_query_dense_f32(
        xyz.shape[0], xyz.shape[1], new_xyz.shape[1], ctypes.c_float(w["radius"]), w["nsample"], _p(new_xyz), _p(xyz),
        _p(bq_idx), _p(bq_dist), st))
    e = {"workload": "configs[0]: ball_query dense B=8 N=4096 M=1024 r=0.1 nsample=32", "metric": "queries/s",
         "value": nq / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_flops(executed, pairs, 8, ev, "ball_query_dense"), "pairs_upper_bound": pairs}
    e["roofline"]["note"] += ("; every workgroup bins its cloud into cells at least one radius wide and a query tests "
                              "the cells around its ball only")
    if ref is not None:
        secs = _cpu_time(lambda: ref.dense_ball_query(w["new_xyz"], w["xyz"], w["radius"], w["nsample"], 0, False))
        e["cpu_baseline"] = {"value": nq / secs, "unit": "queries/s", "cores": 1, "kind": "reference",
                             "sample": "whole configuration, reference cpu/src (nanoflann kd-tree), 1 thread"}
    out["ball_query_dense"] = e

    # beyond the BASELINE configurations: the same query with sort=True (nearest nsample first), which the
    # reference computes for CPU tensors only
    wall, ev = _time_gpu(lambda: tpk.ball_query(w["radius"], w["nsample"], xyz, new_xyz, mode="dense", sort=True), steps, warmup)
    e = {"workload": "ball_query dense sort=True on configs[0] (B=8 N=4096 M=1024 r=0.1 nsample=32; the reference has this "
                     "mode for CPU tensors only)", "metric": "queries/s", "value": nq / (wall * 1e-3), "kernel_ms": ev,
         "wall_ms": wall, "pairs": pairs, "algorithmic_rate_tflops": pairs * 8 / (ev * 1e-3) / 1e12}
    if ref is not None:
        secs = _cpu_time(lambda: ref.dense_ball_query(w["new_xyz"], w["xyz"], w["radius"], w["nsample"], 0, True))
        e["cpu_baseline"] = {"value": nq / secs, "unit": "queries/s", "cores": 1, "kind": "reference",
                             "sample": "whole configuration, reference cpu/src (nanoflann radius search, sorted), 1 thread"}
    out["ball_query_dense_sorted"] = e

    # configs[3]: partial dense ball query
    w = W.cfg4_ball_query_partial()
    x, y, bx, by = (w[k].to(dev) for k in ("x", "y", "batch_x", "batch_y"))
    wall, ev = _time_gpu(lambda: tpk.ball_query(w["radius"], w["nsample"], x, y, mode="partial_dense", batch_x=bx, batch_y=by),
                         steps, warmup)
    nq = y.shape[0]
    sizes = torch.bincount(w["batch_x"]).tolist()
    qsizes = torch.bincount(w["batch_y"]).tolist()
    pairs = sum(a * b for a, b in zip(sizes, qsizes))
    bq_idx = torch.empty(nq, w["nsample"], dtype=torch.int64, device=dev)
    bq_dist = torch.empty(nq, w["nsample"], device=dev)
    ws_bytes = _counting_lib().tpk_ball_query_partial_workspace_bytes(ctypes.c_int64(x.shape[0]), ctypes.c_int64(nq),
                                                                      w["nsample"])
    ws = _ws(ws_bytes, dev)
    executed = _executed(lambda lib, st: lib.tpk_ball_query_partial_f32(
        ctypes.c_int64(x.shape[0]), ctypes.c_int64(nq), ctypes.c_float(w["radius"]), w["nsample"], _p(x), _p(y), _p(bx),
        _p(by), _p(bq_idx), _p(bq_dist), _p(ws) if ws_bytes else None, ctypes.c_size_t(ws_bytes), st))
    e = {"workload": "configs[3]: ball_query partial_dense clouds 20k/45k/70k/100k, 25% queries, r=0.05 nsample=64",
         "metric": "queries/s", "value": nq / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_flops(executed, pairs, 8, ev, "ball_query_partial_dense"), "pairs_upper_bound": pairs}
    e["roofline"]["note"] += PRUNED_NOTE
    e["all_pairs_kernel"] = _all_pairs_entry(lambda lib, st: lib.tpk_ball_query_partial_f32(
        ctypes.c_int64(x.shape[0]), ctypes.c_int64(nq), ctypes.c_float(w["radius"]), w["nsample"], _p(x), _p(y), _p(bx),
        _p(by), _p(bq_idx), _p(bq_dist), None, ctypes.c_size_t(0), st), pairs, max(3, steps // 4), 1, "ball_query_partial_kernel")
    if ref is not None:
        secs = _cpu_time(lambda: ref.batch_ball_query(w["x"], w["y"], w["batch_x"], w["batch_y"], w["radius"],
                                                      w["nsample"], 0, False))
        e["cpu_baseline"] = {"value": nq / secs, "unit": "queries/s", "cores": 1, "kind": "reference",
                             "sample": "whole configuration, reference cpu/src (nanoflann kd-tree per cloud), 1 thread"}
    out["ball_query_partial_dense"] = e
    wall, ev = _time_gpu(lambda: tpk.ball_query(w["radius"], w["nsample"], x, y, mode="partial_dense", batch_x=bx, batch_y=by,
                                                sort=True), max(3, steps // 4), 1)
    e = {"workload": "ball_query partial_dense sort=True on configs[3] (the reference has this mode for CPU tensors only)",
         "metric": "queries/s", "value": nq / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "pairs": pairs, "algorithmic_rate_tflops": pairs * 8 / (ev * 1e-3) / 1e12,
         "note": "the bin walk of the unsorted packed query with a selection of the nearest in place of its hit list"}
    if ref is not None:
        secs = _cpu_time(lambda: ref.batch_ball_query(w["x"], w["y"], w["batch_x"], w["batch_y"], w["radius"],
                                                      w["nsample"], 0, True))
        e["cpu_baseline"] = {"value": nq / secs, "unit": "queries/s", "cores": 1, "kind": "reference",
                             "sample": "whole configuration, reference cpu/src (nanoflann radius search per cloud, sorted), 1 thread"}
    out["ball_query_partial_dense_sorted"] = e

    # configs[2](a): three_nn + three_interpolate fwd/bwd
    w = W.cfg3a_interpolate()
    unknown, known = w["unknown"].to(dev), w["known"].to(dev)
    wall, ev = _time_gpu(lambda: nat.three_nn(unknown, known), steps, warmup)
    nq = unknown.shape[0] * unknown.shape[1]
    pairs = W.pairs_three_nn()
    nn_d = torch.empty(unknown.shape[0], unknown.shape[1], 3, device=dev)
    nn_i = torch.empty(unknown.shape[0], unknown.shape[1], 3, dtype=torch.int32, device=dev)
    ws_bytes = _counting_lib().tpk_three_nn_workspace_bytes(unknown.shape[0], unknown.shape[1], known.shape[1])
    ws = _ws(ws_bytes, dev)
    executed = _executed(lambda lib, st: lib.tpk_three_nn_f32(
        unknown.shape[0], unknown.shape[1], known.shape[1], _p(unknown), _p(known), _p(nn_d), _p(nn_i),
        _p(ws) if ws_bytes else None, ctypes.c_size_t(ws_bytes), st))
    e = {"workload": "configs[2]a: three_nn unknown (16,16384,3) known (16,4096,3)", "metric": "queries/s",
         "value": nq / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_flops(executed, pairs, 8, ev, "three_nn"), "pairs": pairs}
    e["roofline"]["note"] += ("; every workgroup sorts its known cloud into a grid in LDS and a query looks at the cells "
                              "around it only; kernel_ms also covers the two launches behind it that would answer clouds "
                              "of uneven density (here they return at once)")
    e["all_pairs_kernel"] = _all_pairs_entry(lambda lib, st: lib.tpk_three_nn_all_pairs_f32(
        unknown.shape[0], unknown.shape[1], known.shape[1], _p(unknown), _p(known), _p(nn_d), _p(nn_i), st),
        pairs, max(3, steps // 4), 1, ("three_nn_kernel<1>", "three_nn_kernel<2>", "three_nn_kernel<4>"))
    if ref is not None:
        sub = 4  # clouds
        secs = _cpu_time(lambda: ref.dense_knn(w["known"][:sub], w["unknown"][:sub], 3))
        e["cpu_baseline"] = {"value": (nq * sub / 16) / secs, "unit": "queries/s", "cores": 1, "kind": "reference",
                             "sample": "%d of 16 clouds, reference cpu/src/knn.cpp (nanoflann k=3), 1 thread" % sub}
    out["three_nn"] = e

    # beyond the BASELINE configurations: dense knn (k = 16) on the clouds of configs[2]a; the reference
    # has this operator on the CPU only
    knn_k = 16
    wall, ev = _time_gpu(lambda: nat.dense_knn(known, unknown, knn_k), steps, warmup)
    e = {"workload": "dense knn k=16, queries (16,16384,3), support (16,4096,3) (clouds of configs[2]a; not a BASELINE configuration)",
         "metric": "queries/s", "value": nq / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "pairs": pairs, "algorithmic_rate_tflops": pairs * 8 / (ev * 1e-3) / 1e12}
    if ref is not None:
        sub = 4  # clouds
        secs = _cpu_time(lambda: ref.dense_knn(w["known"][:sub], w["unknown"][:sub], knn_k))
        e["cpu_baseline"] = {"value": (nq * sub / 16) / secs, "unit": "queries/s", "cores": 1, "kind": "reference",
                             "sample": "%d of 16 clouds, reference cpu/src/knn.cpp (nanoflann k=16), 1 thread" % sub}
    out["knn_k16"] = e

    # beyond the BASELINE configurations: region growing on the workload of the reference's
    # benchmark/region_cluster.py; the reference grows the clusters on the host (numba) after copying the
    # neighbour matrix there
    rc = W.region_cluster()
    pos, batch = rc["pos"].to(dev), rc["batch"].to(dev)
    neighbours = tpk.ball_query_partial_dense(rc["radius"], rc["nsample"], pos, pos, batch, batch)[0]
    npts = pos.shape[0]
    nbytes = neighbours.numel() * 8
    grow = {}
    for order, name in ((False, "index"), (True, "reference")):
        wall, ev = _time_gpu(lambda: nat.grow_proximity(neighbours, rc["min_cluster_size"], order), max(3, steps // 4), 1)
        grow[name] = (wall, ev)
    members, starts = nat.grow_proximity(neighbours, rc["min_cluster_size"], False)
    wall, ev = grow["index"]
    e = {"workload": "grow_proximity over the neighbour matrix (300000, 16) of benchmark/region_cluster.py (3 x 100000 uniform "
                     "points, r=0.02, nsample=16, min_cluster_size=32; not a BASELINE configuration); members by index",
         "metric": "points/s", "value": npts / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "members_in_reference_order_wall_ms": grow["reference"][0],
         "clusters": int(starts.numel() - 1), "members": int(members.numel()),
         "largest_cluster": int((starts[1:] - starts[:-1]).max()) if starts.numel() > 1 else 0,
         "roofline": _roof_bytes(nbytes + members.numel() * 8, ev, "grow_proximity"),
         "algorithmic_bytes": nbytes + members.numel() * 8}
    e["roofline"]["note"] = ("algorithmic bytes = the matrix read once + the members written; the call is about 45 short "
                             "kernels and three waits for the stream (data-dependent sweep count and output size), so launch "
                             "and wait time, not bandwidth, decides; kernel_ms is the time between events around the whole call. "
                             "Members in the reference's order need a serial walk per cluster (largest cluster decides)")
    if with_cpu:
        import oracle

        matrix = neighbours.cpu().numpy()
        secs = _cpu_time(lambda: oracle.grow_proximity_core(matrix, rc["min_cluster_size"]))
        e["cpu_baseline"] = {"value": npts / secs, "unit": "points/s", "cores": 1, "kind": "port",
                             "sample": "the whole matrix; C restatement of the reference's numba routine (cluster.py:9-37); the "
                                       "reference also copies the matrix (38 MB) to the host first, not timed here"}
    out["grow_proximity"] = e

    # beyond the BASELINE configurations: instance IoU of 500 proposals of 2000 points against 4 x 50 ground-truth
    # instances (the native call only: the Python front end's per-sample statistics are prepared once)
    ip = W.instance_proposals()
    prop_idx = torch.cat(ip["proposals"]).to(dev)
    prop_off = torch.tensor([0] + [int(p.numel()) for p in ip["proposals"]]).cumsum(0).to(dev)
    gt_dev, batch_dev = ip["gt"].to(dev), ip["batch"].to(dev)
    counts = torch.tensor([int(ip["gt"][ip["batch"] == s_].max()) for s_ in range(4)], device=dev)
    sizes = torch.cat([torch.bincount(ip["gt"][ip["batch"] == s_], minlength=51)[1:51] for s_ in range(4)]).to(dev)
    wall, ev = _time_gpu(lambda: nat.instance_iou_cuda(prop_idx, prop_off, gt_dev, sizes, counts, batch_dev), steps, warmup)
    nbytes = prop_idx.numel() * 16 + 500 * 200 * 4  # an index and a label per proposal point, the output once
    e = {"workload": "instance_iou: 500 proposals x 2000 points, 4 samples x 50 ground-truth instances, 300000 points "
                     "(not a BASELINE configuration)", "metric": "proposals/s", "value": 500 / (wall * 1e-3),
         "kernel_ms": ev, "wall_ms": wall, "roofline": _roof_bytes(nbytes, ev, "instance_iou"), "algorithmic_bytes": nbytes}
    e["roofline"]["note"] = "kernel_ms includes the column sums PyTorch forms to size the output (two small kernels and a read-back)"
    if with_cpu:
        import oracle

        props_np = [p.numpy() for p in ip["proposals"]]
        secs = _cpu_time(lambda: oracle.instance_iou(props_np, ip["gt"].numpy(), ip["batch"].numpy()))
        e["cpu_baseline"] = {"value": 500 / secs, "unit": "proposals/s", "cores": 1, "kind": "port",
                             "sample": "the whole workload; C restatement of the reference's CUDA kernel loops (the reference's "
                                       "CPU path is a numba routine of the same shape)"}
    out["instance_iou"] = e

    # beyond the BASELINE configurations: GRNet's grid operators at its sizes (32 clouds of 2048 points; 64^3 grid;
    # feature map 64 channels x 16^3)
    gg = torch.Generator().manual_seed(11)
    cloud = ((torch.rand(32, 2048, 3, generator=gg) * 2 - 1) * 31.0).to(dev)
    wall, ev = _time_gpu(lambda: nat.gridding(-32.0, 31.0, -32.0, 31.0, -32.0, 31.0, cloud), steps, warmup)
    grid, gw, gi = nat.gridding(-32.0, 31.0, -32.0, 31.0, -32.0, 31.0, cloud)
    npts = 32 * 2048
    nbytes = npts * (12 + 96 + 32) + grid.numel() * 4  # points in; weights and indexes out; the grid written once
    e = {"workload": "gridding forward: 32 clouds x 2048 points into 64^3 grids (not a BASELINE configuration)", "metric": "points/s",
         "value": npts / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall, "roofline": _roof_bytes(nbytes, ev, "gridding_fwd"),
         "algorithmic_bytes": nbytes}
    if with_cpu:
        import oracle

        sub = cloud[:4].cpu().numpy()
        secs = _cpu_time(lambda: oracle.gridding(sub, 32))
        e["cpu_baseline"] = {"value": 4 * 2048 / secs, "unit": "points/s", "cores": 1, "kind": "port",
                             "sample": "4 of 32 clouds; C restatement of the reference's CUDA kernel (the reference has no CPU path)"}
    out["gridding_fwd"] = e
    ggrad = torch.randn(grid.shape, generator=gg).to(dev)
    wall, ev = _time_gpu(lambda: nat.gridding_grad(gw, gi, ggrad), steps, warmup)
    nbytes = npts * (96 + 32 + 32 + 12)  # weights, indexes, 8 gathered gradients per point; 12 bytes out
    out["gridding_bwd"] = {"workload": "gridding backward, same sizes", "metric": "points/s", "value": npts / (wall * 1e-3),
                           "kernel_ms": ev, "wall_ms": wall, "roofline": _roof_bytes(nbytes, ev, "gridding_bwd"),
                           "algorithmic_bytes": nbytes}
    feats = torch.rand(32, 64, 16, 16, 16, generator=gg).to(dev)
    pts16 = (torch.rand(32, 2048, 3, generator=gg) * 15.0).to(dev)
    wall, ev = _time_gpu(lambda: nat.cubic_feature_sampling(16, 1, pts16, feats), steps, warmup)
    pf, pi = nat.cubic_feature_sampling(16, 1, pts16, feats)
    nbytes = pf.numel() * 8 + pi.numel() * 4 + npts * 12  # every sampled feature read and written once
    e = {"workload": "cubic_feature_sampling forward: 32 clouds x 2048 points, 64 channels x 16^3, neighborhood 1 (not a BASELINE "
                     "configuration)", "metric": "GB/s", "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_bytes(nbytes, ev, "cubic_fwd"), "algorithmic_bytes": nbytes}
    if with_cpu:
        import oracle

        secs = _cpu_time(lambda: oracle.cubic_feature_sampling(pts16[:4].cpu().numpy(), feats[:4].cpu().numpy(), 1))
        e["cpu_baseline"] = {"value": nbytes / 8 / secs / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                             "sample": "4 of 32 clouds; C restatement of the reference's CUDA kernel (the reference has no CPU path)"}
    out["cubic_feature_sampling_fwd"] = e
    gpf = torch.randn(pf.shape, generator=gg).to(dev)
    wall, ev = _time_gpu(lambda: nat.cubic_feature_sampling_grad(16, 1, gpf, pi), steps, warmup)
    nbytes = pf.numel() * 4 + pi.numel() * 4 + feats.numel() * 4 + npts * 12
    out["cubic_feature_sampling_bwd"] = {"workload": "cubic_feature_sampling backward, same sizes", "metric": "GB/s",
                                         "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
                                         "roofline": _roof_bytes(nbytes, ev, "cubic_bwd"), "algorithmic_bytes": nbytes}

    dist, idx = tpk.three_nn(unknown, known)
    weight = W.inverse_distance_weights(dist).contiguous()
    feats = w["features"].to(dev)
    gout = w["grad_out"].to(dev)
    m = feats.shape[2]
    nbytes = W.bytes_three_interpolate()
    wall, ev = _time_gpu(lambda: nat.three_interpolate(feats, idx, weight), steps, warmup)
    e = {"workload": "configs[2]a: three_interpolate forward features (16,128,4096) -> (16,128,16384)", "metric": "GB/s",
         "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_bytes(nbytes, ev, "three_interpolate_fwd"), "algorithmic_bytes": nbytes}
    if ref is not None:
        sub = 2
        idx64 = idx[:sub].cpu().long()
        wc = weight[:sub].cpu()
        secs = _cpu_time(lambda: ref.knn_interpolate(w["features"][:sub], idx64, wc))
        e["cpu_baseline"] = {"value": (nbytes * sub / 16) / secs / 1e9, "unit": "GB/s", "cores": 1, "kind": "reference",
                             "sample": "%d of 16 clouds, reference cpu/src/interpolate.cpp scalar loops" % sub}
    out["three_interpolate_fwd"] = e
    wall, ev = _time_gpu(lambda: nat.three_interpolate_grad(gout, idx, weight, m), steps, warmup)
    e = {"workload": "configs[2]a: three_interpolate backward grad (16,128,16384) -> (16,128,4096); the call of the "
                     "reference's interface, which gets (grad_out, idx, weight) and inverts the index itself",
         "metric": "GB/s", "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_bytes(nbytes, ev, "three_interpolate_bwd"), "algorithmic_bytes": nbytes}
    # the same gradient as autograd computes it: the forward pass, knowing that a backward pass follows, also inverts
    # the index, and the backward pass walks the lists
    e["as_autograd_runs_it"] = _autograd_split(
        lambda: nat.three_interpolate_recording(feats, idx, weight),
        lambda lists: nat.three_interpolate_grad_lists(gout, lists, m), nbytes, steps, warmup, "three_interpolate_bwd_lists")
    if ref is not None:
        secs = _cpu_time(lambda: ref.knn_interpolate_grad(w["grad_out"][:sub], idx64, wc, m))
        e["cpu_baseline"] = {"value": (nbytes * sub / 16) / secs / 1e9, "unit": "GB/s", "cores": 1, "kind": "reference",
                             "sample": "%d of 16 clouds, reference cpu/src/interpolate.cpp scalar loops" % sub}
    out["three_interpolate_bwd"] = e
    del feats, gout, dist, idx, weight

    # configs[2](b): grouping fwd/bwd
    w = W.cfg3b_grouping()
    feats, gidx, gout = w["features"].to(dev), w["idx"].to(dev), w["grad_out"].to(dev)
    nbytes = W.bytes_grouping()
    wall, ev = _time_gpu(lambda: nat.grouping_operation(feats, gidx), steps, warmup)
    e = {"workload": "configs[2]b: grouping_operation forward features (16,128,4096) idx (16,1024,32)", "metric": "GB/s",
         "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_bytes(nbytes, ev, "grouping_fwd"), "algorithmic_bytes": nbytes}
    if with_cpu:
        # the reference implementation of this op is torch.gather on a repeated index (CPU tensors)
        def cpu_group():
            all_idx = w["idx"].reshape(16, -1).unsqueeze(1).repeat(1, 128, 1)
            return w["features"].gather(2, all_idx)

        secs = _cpu_time(cpu_group)
        e["cpu_baseline"] = {"value": nbytes / secs / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                             "kind": "reference", "sample": "whole configuration, torch.gather on CPU tensors "
                             "(the reference's implementation, torchpoints.py:129-146)"}
    out["grouping_fwd"] = e
    n = feats.shape[2]
    wall, ev = _time_gpu(lambda: nat.grouping_operation_grad(gout, gidx, n), steps, warmup)
    out["grouping_bwd"] = {"workload": "configs[2]b: grouping_operation backward (the stand-alone call, which inverts the index "
                                       "itself)", "metric": "GB/s",
                           "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
                           "roofline": _roof_bytes(nbytes, ev, "grouping_bwd"), "algorithmic_bytes": nbytes}
    out["grouping_bwd"]["as_autograd_runs_it"] = _autograd_split(
        lambda: nat.grouping_operation_recording(feats, gidx),
        lambda lists: nat.grouping_operation_grad_lists(gout, lists, n), nbytes, steps, warmup, "grouping_bwd_lists")
    del feats, gidx, gout

    # configs[4]: chamfer fwd/bwd
    w = W.cfg5_chamfer()
    a, b = w["xyz1"].to(dev), w["xyz2"].to(dev)
    g1, g2 = w["grad_dist1"].to(dev), w["grad_dist2"].to(dev)
    csteps = max(3, steps // 4)
    wall, ev = _time_gpu(lambda: nat.chamfer_dist(a, b), csteps, min(warmup, 2))
    pairs = W.pairs_chamfer()
    cb, cn, cm = a.shape[0], a.shape[1], b.shape[1]
    cd1, cd2 = torch.empty(cb, cn, device=dev), torch.empty(cb, cm, device=dev)
    ci1 = torch.empty(cb, cn, dtype=torch.int32, device=dev)
    ci2 = torch.empty(cb, cm, dtype=torch.int32, device=dev)
    ws_bytes = _counting_lib().tpk_chamfer_fwd_workspace_bytes(cb, cn, cm)
    ws = _ws(ws_bytes, dev)
    executed = _executed(lambda lib, st: lib.tpk_chamfer_fwd_f32(
        cb, cn, cm, _p(a), _p(b), _p(cd1), _p(cd2), _p(ci1), _p(ci2), _p(ws) if ws_bytes else None,
        ctypes.c_size_t(ws_bytes), st))
    e = {"workload": "configs[4]: Chamfer forward B=32 16384x16384 (both directions)", "metric": "pairs/s",
         "value": pairs / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_flops(executed, pairs, 8, ev, "chamfer_fwd"), "pairs": pairs}
    e["roofline"]["note"] += PRUNED_NOTE
    e["all_pairs_kernel"] = _all_pairs_entry(lambda lib, st: lib.tpk_chamfer_fwd_f32(
        cb, cn, cm, _p(a), _p(b), _p(cd1), _p(cd2), _p(ci1), _p(ci2), None, ctypes.c_size_t(0), st), pairs, 3, 1,
        "chamfer_fwd_kernel<float, 4>")
    if with_cpu:
        import oracle

        sub = 256  # queries per cloud, one cloud pair, one direction
        secs = _cpu_time(lambda: oracle.chamfer_fwd(w["xyz1"][:1, :sub].numpy(), w["xyz2"][:1].numpy()))
        # the timed call evaluates sub*N pairs for direction 1 and N*sub for direction 2
        e["cpu_baseline"] = {"value": 2 * sub * 16384 / secs, "unit": "pairs/s", "cores": 1, "kind": "port",
                             "sample": "the reference has NO CPU Chamfer (chamfer_dist.py:10-11 raises); this is the "
                                       "scalar C restatement on %d x 16384 points of one pair" % sub}
    out["chamfer_fwd"] = e
    d1, d2, i1, i2 = nat.chamfer_dist(a, b)
    nbytes = W.bytes_chamfer_bwd()
    wall, ev = _time_gpu(lambda: nat.chamfer_dist_grad(a, b, i1, i2, g1, g2), steps, warmup)
    out["chamfer_bwd"] = {"workload": "configs[4]: Chamfer backward", "metric": "GB/s",
                          "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
                          "roofline": _roof_bytes(nbytes, ev, "chamfer_bwd"), "algorithmic_bytes": nbytes}
    return out


def headline_object(fps, steps, warmup, device):
    """The full record of a run: the headline keys, the headline's roofline and cpu_baseline objects with their
    prose, and (added by the caller) the per-operator entries under "ops"."""
    full = {
        "metric": "furthest_point_sample ms/batch",
        "value": fps["wall_ms"],
        "unit": "ms/batch",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": fps["wall_ms"],
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: furthest_point_sample B=16 clouds x N=16384 points (8 Gaussian clusters "
                               "sigma=0.05 + 10% uniform), npoint=4096, start index 0, int32 out"},
        "roofline": fps["roofline"],
        "kernel_ms": fps["kernel_ms"],
        "device": device,
    }
    if "cpu_baseline" in fps:
        full["cpu_baseline"] = fps["cpu_baseline"]
    return full


DETAIL_FILE = os.path.join("gpurun_out", "bench_full.json")
LINE_LIMIT = 4096  # bytes of the printed line; whoever runs this script may keep only the end of its output


def _write_detail(full):
    """Writes the full record (every operator with its workload text, notes and sources) next to the other
    results of a GPU run; returns the path relative to the repository, or None when it cannot be written."""
    try:
        os.makedirs(os.path.join(ROOT, os.path.dirname(DETAIL_FILE)), exist_ok=True)
        with open(os.path.join(ROOT, DETAIL_FILE), "w") as f:
            json.dump(full, f, indent=1)
        return DETAIL_FILE
    except OSError:
        return None


def _sig(x, digits=4):
    """Numbers to `digits` significant digits (a printed line, not an archive)."""
    if isinstance(x, float):
        return float("%.*g" % (digits, x))
    return x


def _compact_roofline(r):
    keep = ("bound", "achieved", "peak", "unit", "frac", "traffic", "executed_pairs", "algorithmic_pairs",
            "algorithmic_rate")
    out = {k: _sig(r[k]) for k in keep if k in r}
    if r.get("bound") == "mfma":
        out["bound_detail"] = "fp32 VALU, unfused (no MFMA: inner dimension 3)"
    valu = r.get("valu")
    if valu:
        out["valu"] = {"busy_pct": _sig(valu.get("valu_busy_pct")), "lanes_pct": _sig(valu.get("valu_lane_utilisation_pct"))}
    return out


def _compact_op(e):
    """One operator as a row of the printed table: kernel ms (HIP events), roofline fraction of EXECUTED work
    (or of algorithmic bytes), the algorithmic fraction for the pruned distance scans, measured HBM traffic
    over algorithmic bytes, and the CPU figure in the operator's own unit."""
    row = {"ms": _sig(e.get("kernel_ms"))}
    if "value" in e:
        row["v"] = _sig(e["value"], 3)
        row["unit"] = e.get("metric")
    r = e.get("roofline")
    if r:
        row["bound"] = "valu" if r.get("bound") == "mfma" else r.get("bound")
        row["frac"] = _sig(r.get("frac"), 3)
        if "algorithmic_rate" in r:
            row["alg_frac"] = _sig(r["algorithmic_rate"] / r["peak"], 3)
        if r.get("traffic") and e.get("algorithmic_bytes"):
            row["traffic_x"] = _sig(r["traffic"] / e["algorithmic_bytes"], 3)
    ag = e.get("as_autograd_runs_it")
    if ag:
        row["autograd"] = {"fwd_ms": _sig(ag["forward_kernel_ms"]), "bwd_ms": _sig(ag["backward_kernel_ms"]),
                           "bwd_frac": _sig(ag["backward_roofline"]["frac"], 3)}
    ap = e.get("all_pairs_kernel")
    if ap:
        row["all_pairs"] = {"ms": _sig(ap["kernel_ms"]), "frac": _sig(ap["roofline"]["frac"], 3)}
    c = e.get("cpu_baseline")
    if c:
        row["cpu"] = _sig(c["value"], 3)
        if c["unit"] != e.get("metric"):
            row["cpu_unit"] = c["unit"]
    return row


# Operators of the BASELINE configurations first; the others leave the printed line first when it is too long.
OPS_ORDER = ("ball_query_dense", "ball_query_partial_dense", "three_nn", "three_interpolate_fwd", "three_interpolate_bwd",
             "grouping_fwd", "grouping_bwd", "chamfer_fwd", "chamfer_bwd", "ball_query_dense_sorted",
             "ball_query_partial_dense_sorted", "knn_k16", "grow_proximity", "instance_iou", "gridding_fwd", "gridding_bwd",
             "cubic_feature_sampling_fwd", "cubic_feature_sampling_bwd")


def compact_line(full, detail_file=None, limit=LINE_LIMIT):
    """The ONE line this script prints, at most `limit` bytes: the headline keys, the headline's roofline and
    cpu_baseline without prose, and one short row per operator.  Everything else is in the detail file."""
    line = {k: full[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                 "higher_is_better", "scaling", "vs_baseline", "dtype", "data") if k in full}
    line["value"] = _sig(full["value"], 6)
    line["ms_per_step"] = _sig(full["ms_per_step"], 6)
    line["value_is"] = "wall clock of the timed steps / steps; ops.*.v likewise (wall-based, in ops.*.unit); ops.*.ms = HIP-event time of the operator's kernels"
    line["config"] = {"workload": "configs[1]: furthest_point_sample B=16 N=16384 npoint=4096"}
    line["kernel_ms"] = _sig(full.get("kernel_ms"), 6)
    line["roofline"] = _compact_roofline(full["roofline"])
    c = full.get("cpu_baseline")
    if c:
        line["cpu_baseline"] = {"value": _sig(c["value"]), "unit": c["unit"], "cores": c["cores"], "kind": c["kind"],
                                "sample": c["sample"][:96]}
    if detail_file:
        line["detail"] = detail_file
    ops = full.get("ops") or {}
    names = [n for n in OPS_ORDER if n in ops] + [n for n in ops if n not in OPS_ORDER]
    line["ops"] = {n: _compact_op(ops[n]) for n in names}
    text = json.dumps(line, separators=(",", ":"))
    while len(text) > limit and names:
        line["ops"].pop(names.pop())
        line["ops_dropped"] = line.get("ops_dropped", 0) + 1
        text = json.dumps(line, separators=(",", ":"))
    return text


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ops", choices=["all", "headline"], default="all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-count", action="store_true",
                    help="skip the runs through the counting build of the library (executed work is then reported as 0); "
                         "for profiler runs, whose per-kernel averages those launches would enter")
    args = ap.parse_args()
    global COUNT_WORK
    COUNT_WORK = not args.no_count
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this library runs on ONE GPU (every operator is independent per cloud; nothing is "
                 "exchanged between GPUs), so only --gpus 1 is measured.")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    from torch_points_kernels._native import native

    native()  # fail loudly if the HIP extension is missing

    # One plain device copy of known size, so that a counter run of this script contains a
    # kernel whose HBM traffic is known (calibration of FETCH_SIZE / WRITE_SIZE).
    src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst

    with_cpu = not args.no_cpu
    fps = bench_fps(dev, args.steps, args.warmup, with_cpu)
    full = headline_object(fps, args.steps, args.warmup, torch.cuda.get_device_name(0))
    if args.ops == "all":
        full["ops"] = bench_others(dev, max(5, args.steps), args.warmup, with_cpu)
    detail = _write_detail(full)
    print(compact_line(full, detail))


if __name__ == "__main__":
    main()

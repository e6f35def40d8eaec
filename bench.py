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

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE run + WRITE_SIZE run, each
# scaled by the same counter's reading for a 256 MiB device copy); see profiles/*pmc*.txt.
# None = not measured yet.
MEASURED_TRAFFIC_BYTES = {
    "fps": 4030000,                    # 3.76 MB read (the clouds; set-up passes mostly hit L2) + 0.26 MB written (the indices)
    "three_interpolate_fwd": 174130000,  # = algorithmic bytes: nothing is read twice from HBM
    "three_interpolate_bwd": 308500000,  # list build 57 MB + list walk 252 MB (two column pieces per four rows)
    "grouping_fwd": 352500000,         # rows staged twice (two column halves per row block)
    "grouping_bwd": 407900000,         # list build 27 MB + walk 381 MB (two column pieces per row: outputs written twice)
    "chamfer_bwd": 128000000,          # list build 72.4 MB (padded lists) + list walk 55.6 MB
    "gridding_fwd": 60400000,          # 1.6 MB read + 25.3 MB written + the grid's zero fill 33.5 MB
    "gridding_bwd": 41500000,          # the eight gathered gradients of a point lie in eight lines
    "cubic_fwd": 172800000,            # index kernel 2.9 MB + gather 35.7 MB read (the feature maps once) + 134.2 MB written
    "cubic_bwd": 170800000,            # 136.4 MB read + 33.6 MB written + the zero fill of the points' gradient
    "instance_iou": 13400000,
}


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


def _roof_flops(pairs_or_updates, flops_each, ms):
    achieved = pairs_or_updates * flops_each / (ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / PEAK_FP32_TFLOPS, "traffic": None,
            "note": "fp32 VALU kernel (inner dimension 3, unfused arithmetic: no MFMA, no FMA, no packed "
                    "fp32); peak is the published fp32 figure, which assumes FMA: without FMA the ceiling is 0.5"}


PRUNED_NOTE = ("; algorithmic work = all pairs (8 flop each), which is what the reference evaluates; the kernel "
               "orders both clouds along a space filling curve and skips cells that provably hold no answer, so "
               "the achieved figure is a rate of algorithmic, not executed, flops and may exceed the peak; "
               "kernel_ms covers the ordering kernel and the search kernel")


def _roof_bytes(nbytes, ms, key):
    achieved = nbytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": achieved / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_BYTES.get(key)}


def _cpu_time(fn, repeat=1):
    best = None
    for _ in range(repeat):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None or dt < best else best
    return best


def bench_fps(dev, steps, warmup, with_cpu):
    import torch

    import torch_points_kernels as tpk
    from tests import workloads as W

    w = W.cfg2_fps()
    xyz = w["xyz"].to(dev)
    npoint = w["npoint"]
    wall, ev = _time_gpu(lambda: tpk.furthest_point_sample(xyz, npoint), steps, warmup)
    updates = W.fps_point_updates()
    roof = _roof_flops(updates, 10, ev)
    roof["traffic"] = MEASURED_TRAFFIC_BYTES.get("fps")
    roof["note"] += "; algorithmic work = every point updated in every round (10 flop each), as the reference " \
                    "does; the kernel skips updates it proves to be no-ops, so the achieved figure is a rate of " \
                    "algorithmic, not executed, flops; the rounds of a cloud are sequential and one workgroup " \
                    "owns a cloud: 16 of 256 compute units are occupied by design, fraction of those 16 CUs' " \
                    "peak = %.4f" % (roof["frac"] * 256 / 16)
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
    e = {"workload": "configs[0]: ball_query dense B=8 N=4096 M=1024 r=0.1 nsample=32", "metric": "queries/s",
         "value": nq / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_flops(pairs, 8, ev), "pairs_upper_bound": pairs}
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
         "wall_ms": wall, "roofline": _roof_flops(pairs, 8, ev), "pairs": pairs}
    e["roofline"]["note"] += PRUNED_NOTE
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
    e = {"workload": "configs[3]: ball_query partial_dense clouds 20k/45k/70k/100k, 25% queries, r=0.05 nsample=64",
         "metric": "queries/s", "value": nq / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_flops(pairs, 8, ev), "pairs_upper_bound": pairs}
    e["roofline"]["note"] += PRUNED_NOTE
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
         "roofline": _roof_flops(pairs, 8, ev), "pairs": pairs}
    e["roofline"]["note"] += PRUNED_NOTE + "; the clouds are searched one after the other, after one wait for the stream"
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
    e = {"workload": "configs[2]a: three_nn unknown (16,16384,3) known (16,4096,3)", "metric": "queries/s",
         "value": nq / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall, "roofline": _roof_flops(pairs, 8, ev),
         "pairs": pairs}
    e["roofline"]["note"] += PRUNED_NOTE
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
         "roofline": _roof_flops(pairs, 8, ev), "pairs": pairs}
    e["roofline"]["note"] += PRUNED_NOTE
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
    e = {"workload": "configs[2]a: three_interpolate backward grad (16,128,16384) -> (16,128,4096)", "metric": "GB/s",
         "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
         "roofline": _roof_bytes(nbytes, ev, "three_interpolate_bwd"), "algorithmic_bytes": nbytes}
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
    out["grouping_bwd"] = {"workload": "configs[2]b: grouping_operation backward", "metric": "GB/s",
                           "value": nbytes / (wall * 1e-3) / 1e9, "kernel_ms": ev, "wall_ms": wall,
                           "roofline": _roof_bytes(nbytes, ev, "grouping_bwd"), "algorithmic_bytes": nbytes}
    del feats, gidx, gout

    # configs[4]: chamfer fwd/bwd
    w = W.cfg5_chamfer()
    a, b = w["xyz1"].to(dev), w["xyz2"].to(dev)
    g1, g2 = w["grad_dist1"].to(dev), w["grad_dist2"].to(dev)
    csteps = max(3, steps // 4)
    wall, ev = _time_gpu(lambda: nat.chamfer_dist(a, b), csteps, min(warmup, 2))
    pairs = W.pairs_chamfer()
    e = {"workload": "configs[4]: Chamfer forward B=32 16384x16384 (both directions)", "metric": "pairs/s",
         "value": pairs / (wall * 1e-3), "kernel_ms": ev, "wall_ms": wall, "roofline": _roof_flops(pairs, 8, ev),
         "pairs": pairs}
    e["roofline"]["note"] += PRUNED_NOTE
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ops", choices=["all", "headline"], default="all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    args = ap.parse_args()
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
    line = {
        "metric": "furthest_point_sample ms/batch",
        "value": fps["wall_ms"],
        "unit": "ms/batch",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
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
        "device": torch.cuda.get_device_name(0),
    }
    if "cpu_baseline" in fps:
        line["cpu_baseline"] = fps["cpu_baseline"]
    if args.ops == "all":
        line["ops"] = bench_others(dev, max(5, args.steps), args.warmup, with_cpu)
    print(json.dumps(line))


if __name__ == "__main__":
    main()

"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

numpy front end of ``oracle/tpk_oracle.c`` (the scalar CPU restatement of the
reference kernels' semantics) and a loader for ``oracle/_ref/points_cpu.so`` (the
reference's own ``cpu/src`` compiled where it lies, when that build exists).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The shipped package
(``torch-points-kernels_amd/torch_points_kernels``) never does.
"""
import ctypes
import importlib.machinery
import importlib.util
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtpk_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "points_cpu.so")
_lib = None
_ref = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)


def build(force=False):
    """Compile the C restatement (and, where the reference checkout exists, its CPU module)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "oracle"] + (["-B"] if force else []))
    return _LIB_PATH


def build_ref(jobs=6):
    """Compile the reference's cpu/src into oracle/_ref/ (needs /root/reference)."""
    subprocess.check_call(["make", "-C", _HERE, "-j%d" % jobs, "ref"])
    return _REF_PATH if os.path.exists(_REF_PATH) else None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def have_ref():
    return os.path.exists(_REF_PATH)


def ref():
    """The reference's compiled CPU module (points_cpu), or None when it was not built."""
    global _ref
    if _ref is None and have_ref():
        import torch  # noqa: F401  (the module links against libtorch)

        loader = importlib.machinery.ExtensionFileLoader("points_cpu", _REF_PATH)
        spec = importlib.util.spec_from_loader("points_cpu", loader)
        mod = importlib.util.module_from_spec(spec)
        loader.exec_module(mod)
        _ref = mod
    return _ref


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _p(a, ptype):
    return a.ctypes.data_as(ptype)


def ball_query_dense(radius, nsample, xyz, new_xyz, return_pairs=False):
    """xyz (B,N,3) support, new_xyz (B,M,3) queries -> idx int64 (B,M,ns), dist f32."""
    xyz = _c(xyz, np.float32)
    new_xyz = _c(new_xyz, np.float32)
    b, n, _ = xyz.shape
    m = new_xyz.shape[1]
    idx = np.empty((b, m, nsample), np.int64)
    dist = np.empty((b, m, nsample), np.float32)
    pairs = ctypes.c_int64(0)
    lib().tpk_oracle_ball_query_dense(
        ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(m), ctypes.c_float(radius),
        ctypes.c_int(nsample), _p(new_xyz, _f32p), _p(xyz, _f32p), _p(idx, _i64p),
        _p(dist, _f32p), ctypes.byref(pairs))
    if return_pairs:
        return idx, dist, pairs.value
    return idx, dist


def ball_query_partial_dense(radius, nsample, x, y, batch_x, batch_y, return_pairs=False):
    """x (Nx,3) support, y (Ny,3) queries, sorted int64 batch vectors -> idx (Ny,ns), dist."""
    x = _c(x, np.float32)
    y = _c(y, np.float32)
    batch_x = _c(batch_x, np.int64)
    batch_y = _c(batch_y, np.int64)
    ny = y.shape[0]
    idx = np.empty((ny, nsample), np.int64)
    dist = np.empty((ny, nsample), np.float32)
    pairs = ctypes.c_int64(0)
    f = lib().tpk_oracle_ball_query_partial
    f.restype = ctypes.c_int64
    rc = f(ctypes.c_int64(x.shape[0]), ctypes.c_int64(ny), ctypes.c_float(radius),
           ctypes.c_int(nsample), _p(x, _f32p), _p(y, _f32p), _p(batch_x, _i64p),
           _p(batch_y, _i64p), _p(idx, _i64p), _p(dist, _f32p), ctypes.byref(pairs))
    if rc < 0:
        raise MemoryError("oracle ball_query_partial")
    if return_pairs:
        return idx, dist, pairs.value
    return idx, dist


def ball_query_sorted_dense(radius, nsample, xyz, new_xyz):
    """sort=True, dense layout: xyz (B,n,3) support, new_xyz (B,m,3) queries -> idx int64 (B,m,ns), dist."""
    xyz = _c(xyz, np.float32)
    new_xyz = _c(new_xyz, np.float32)
    b, n, _ = xyz.shape
    m = new_xyz.shape[1]
    idx = np.empty((b, m, nsample), np.int64)
    dist = np.empty((b, m, nsample), np.float32)
    lib().tpk_oracle_ball_query_sorted_dense(ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(m), ctypes.c_float(radius),
                                             ctypes.c_int(nsample), _p(new_xyz, _f32p), _p(xyz, _f32p),
                                             _p(idx, _i64p), _p(dist, _f32p))
    return idx, dist


def ball_query_sorted_partial(radius, nsample, x, y, batch_x, batch_y):
    """sort=True, packed layout: x (Nx,3) support, y (Ny,3) queries, sorted int64 batch vectors."""
    x = _c(x, np.float32)
    y = _c(y, np.float32)
    batch_x = _c(batch_x, np.int64)
    batch_y = _c(batch_y, np.int64)
    ny = y.shape[0]
    idx = np.empty((ny, nsample), np.int64)
    dist = np.empty((ny, nsample), np.float32)
    lib().tpk_oracle_ball_query_sorted_partial(ctypes.c_int64(x.shape[0]), ctypes.c_int64(ny), ctypes.c_float(radius),
                                               ctypes.c_int(nsample), _p(x, _f32p), _p(y, _f32p), _p(batch_x, _i64p),
                                               _p(batch_y, _i64p), _p(idx, _i64p), _p(dist, _f32p))
    return idx, dist


def furthest_point_sample(xyz, npoint):
    xyz = _c(xyz, np.float32)
    b, n, _ = xyz.shape
    out = np.empty((b, npoint), np.int32)
    rc = lib().tpk_oracle_fps(ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(npoint),
                              _p(xyz, _f32p), _p(out, _i32p))
    if rc != 0:
        raise MemoryError("oracle fps")
    return out


def three_nn(unknown, known):
    """-> (dist2 f32 (B,n,3) squared, idx int32 (B,n,3)), as the native entry returns them."""
    unknown = _c(unknown, np.float32)
    known = _c(known, np.float32)
    b, n, _ = unknown.shape
    m = known.shape[1]
    dist2 = np.empty((b, n, 3), np.float32)
    idx = np.empty((b, n, 3), np.int32)
    lib().tpk_oracle_three_nn(ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(m),
                              _p(unknown, _f32p), _p(known, _f32p), _p(dist2, _f32p),
                              _p(idx, _i32p))
    return dist2, idx


def knn(support, query, k):
    """-> (idx int64 (B,m,k), dist2 f32 (B,m,k)), ascending by (distance, index)."""
    support = _c(support, np.float32)
    query = _c(query, np.float32)
    b, n, _ = support.shape
    m = query.shape[1]
    idx = np.empty((b, m, k), np.int64)
    dist2 = np.empty((b, m, k), np.float32)
    lib().tpk_oracle_knn.restype = ctypes.c_int
    rc = lib().tpk_oracle_knn(ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(m), ctypes.c_int(k),
                              _p(support, _f32p), _p(query, _f32p), _p(idx, _i64p), _p(dist2, _f32p))
    if rc != 0:
        raise RuntimeError("Not enough points in support to find %d neighboors" % k)
    return idx, dist2


def grow_proximity_core(neighbours, min_cluster_size):
    """Clusters over a neighbour matrix (n, nsample) int64 -> list of lists, as the numba routine of the
    reference (torch_points_kernels/cluster.py:9-37) returns them."""
    neighbours = _c(neighbours, np.int64)
    n, nsample = neighbours.shape
    members = np.empty(max(n, 1), np.int64)
    starts = np.empty(n + 1, np.int64)
    fn = lib().tpk_oracle_grow_proximity
    fn.restype = ctypes.c_int64
    count = fn(ctypes.c_int64(n), ctypes.c_int(nsample), _p(neighbours, _i64p), ctypes.c_int64(min_cluster_size),
               _p(members, _i64p), _p(starts, _i64p))
    return [members[starts[c]:starts[c + 1]].tolist() for c in range(count)]


def grow_proximity(pos, batch, nsample=16, radius=0.02, min_cluster_size=32):
    """torch_points_kernels/cluster.py:40-45 for tensors on the GPU: neighbours by the packed ball query
    (self query), then the growth above."""
    idx, _ = ball_query_partial_dense(radius, nsample, pos, pos, batch, batch)
    return grow_proximity_core(idx, min_cluster_size)


def region_grow(pos, labels, batch, ignore_labels=(), nsample=16, radius=0.02, min_cluster_size=32):
    """torch_points_kernels/cluster.py:48-109: grow_proximity per label value (ascending), clouds renumbered
    to consecutive values, clusters given as arrays of indices into pos."""
    pos = np.asarray(pos)
    labels = np.asarray(labels)
    batch = np.asarray(batch)
    clusters = []
    ind = np.arange(pos.shape[0])
    for l in np.unique(labels):
        if l in ignore_labels:
            continue
        mask = labels == l
        local = ind[mask]
        _, remapped = np.unique(batch[mask], return_inverse=True)
        for cluster in grow_proximity(pos[mask], remapped.astype(np.int64), nsample, radius, min_cluster_size):
            clusters.append(local[np.asarray(cluster, np.int64)])
    return clusters


def three_interpolate(points, idx, weight):
    points = _c(points, np.float32)
    idx = _c(idx, np.int32)
    weight = _c(weight, np.float32)
    b, c, m = points.shape
    n = idx.shape[1]
    out = np.empty((b, c, n), np.float32)
    lib().tpk_oracle_three_interpolate(ctypes.c_int(b), ctypes.c_int(c), ctypes.c_int(m),
                                       ctypes.c_int(n), _p(points, _f32p), _p(idx, _i32p),
                                       _p(weight, _f32p), _p(out, _f32p))
    return out


def three_interpolate_grad(grad_out, idx, weight, m):
    grad_out = _c(grad_out, np.float32)
    idx = _c(idx, np.int32)
    weight = _c(weight, np.float32)
    b, c, n = grad_out.shape
    out = np.empty((b, c, m), np.float32)
    lib().tpk_oracle_three_interpolate_grad(ctypes.c_int(b), ctypes.c_int(c), ctypes.c_int(n),
                                            ctypes.c_int(m), _p(grad_out, _f32p),
                                            _p(idx, _i32p), _p(weight, _f32p), _p(out, _f32p))
    return out


def grouping_operation(features, idx):
    features = _c(features, np.float32)
    idx = _c(idx, np.int64)
    b, c, n = features.shape
    _, npoint, nsample = idx.shape
    out = np.empty((b, c, npoint, nsample), np.float32)
    lib().tpk_oracle_group(ctypes.c_int(b), ctypes.c_int(c), ctypes.c_int(n),
                           ctypes.c_int64(npoint * nsample), _p(features, _f32p),
                           _p(idx, _i64p), _p(out, _f32p))
    return out


def grouping_operation_grad(grad_out, idx, n):
    grad_out = _c(grad_out, np.float32)
    idx = _c(idx, np.int64)
    b, c, npoint, nsample = grad_out.shape
    out = np.empty((b, c, n), np.float32)
    lib().tpk_oracle_group_grad(ctypes.c_int(b), ctypes.c_int(c), ctypes.c_int(n),
                                ctypes.c_int64(npoint * nsample), _p(grad_out, _f32p),
                                _p(idx, _i64p), _p(out, _f32p))
    return out


def _fp(dtype):
    if dtype == np.float64:
        return np.float64, _f64p, "f64"
    return np.float32, _f32p, "f32"


def chamfer_fwd(xyz1, xyz2):
    """-> dist1 (B,n), dist2 (B,m), idx1 int32 (B,n), idx2 int32 (B,m); dtype follows xyz1."""
    dt, pt, tag = _fp(np.asarray(xyz1).dtype)
    xyz1 = _c(xyz1, dt)
    xyz2 = _c(xyz2, dt)
    b, n, _ = xyz1.shape
    m = xyz2.shape[1]
    dist1 = np.empty((b, n), dt)
    dist2 = np.empty((b, m), dt)
    idx1 = np.empty((b, n), np.int32)
    idx2 = np.empty((b, m), np.int32)
    getattr(lib(), "tpk_oracle_chamfer_fwd_" + tag)(
        ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(m), _p(xyz1, pt), _p(xyz2, pt),
        _p(dist1, pt), _p(dist2, pt), _p(idx1, _i32p), _p(idx2, _i32p))
    return dist1, dist2, idx1, idx2


def chamfer_bwd(xyz1, xyz2, idx1, idx2, grad_dist1, grad_dist2):
    dt, pt, tag = _fp(np.asarray(xyz1).dtype)
    xyz1 = _c(xyz1, dt)
    xyz2 = _c(xyz2, dt)
    idx1 = _c(idx1, np.int32)
    idx2 = _c(idx2, np.int32)
    grad_dist1 = _c(grad_dist1, dt)
    grad_dist2 = _c(grad_dist2, dt)
    b, n, _ = xyz1.shape
    m = xyz2.shape[1]
    g1 = np.empty((b, n, 3), dt)
    g2 = np.empty((b, m, 3), dt)
    getattr(lib(), "tpk_oracle_chamfer_bwd_" + tag)(
        ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(m), _p(xyz1, pt), _p(xyz2, pt),
        _p(idx1, _i32p), _p(idx2, _i32p), _p(grad_dist1, pt), _p(grad_dist2, pt), _p(g1, pt),
        _p(g2, pt))
    return g1, g2


def instance_iou(instance_idx, gt_instances, batch=None):
    """torch_points_kernels/metrics.py:37-104 (front end) + cuda/src/metrics_gpu.cu:9-43: instance_idx is a list of
    index arrays (the proposals), gt_instances the label of every point (0: none), batch the sample of every point.
    -> float32 (proposals, ground-truth instances of all samples)."""
    gt = _c(gt_instances, np.int64)
    batch = np.zeros_like(gt) if batch is None else _c(batch, np.int64)
    sizes, counts = [], []
    for s in range(int(batch[-1]) + 1):
        sample = gt[batch == s]
        count = int(sample.max())
        counts.append(count)
        for k in range(1, count + 1):
            sizes.append(int((sample == k).sum()))
    counts = np.asarray(counts, np.int64)
    sizes = np.asarray(sizes, np.int64)
    offsets = np.concatenate([[0], np.cumsum([len(i) for i in instance_idx])]).astype(np.int64)
    idx = _c(np.concatenate([np.asarray(i, np.int64) for i in instance_idx]), np.int64)
    first = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    total = int(counts.sum())
    out = np.empty((len(instance_idx), total), np.float32)
    lib().tpk_oracle_instance_iou(ctypes.c_int64(total), ctypes.c_int64(len(instance_idx)), _p(counts, _i64p),
                                  _p(idx, _i64p), _p(offsets, _i64p), _p(gt, _i64p), _p(first, _i64p),
                                  _p(batch, _i64p), _p(sizes, _i64p), _p(out, _f32p))
    return out


def _grid_types(a):
    a = np.asarray(a)
    if a.dtype == np.float64:
        return np.float64, ctypes.POINTER(ctypes.c_double), "f64"
    return np.float32, _f32p, "f32"


def gridding(ptcloud, scale):
    """GriddingFunction.forward (torch_points_kernels/gridding.py:9-22): ptcloud (B,n,3) in grid units ->
    (grid (B,(2*scale)^3), grid_pt_weights (B,n,8,3), grid_pt_indexes (B,n,8) int32)."""
    dt, ptr, suf = _grid_types(ptcloud)
    p = _c(ptcloud, dt)
    b, n, _ = p.shape
    side = 2 * scale
    grid = np.empty((b, side ** 3), dt)
    weights = np.empty((b, n, 8, 3), dt)
    indexes = np.empty((b, n, 8), np.int32)
    f = ctypes.c_float
    getattr(lib(), "tpk_oracle_gridding_" + suf)(ctypes.c_int(b), ctypes.c_int(n), f(-scale), f(scale - 1), f(-scale),
                                                  f(scale - 1), f(-scale), f(scale - 1), _p(p, ptr), _p(grid, ptr),
                                                  _p(weights, ptr), _p(indexes, _i32p))
    return grid, weights, indexes


def gridding_grad(grid_pt_weights, grid_pt_indexes, grad_grid):
    dt, ptr, suf = _grid_types(grid_pt_weights)
    w = _c(grid_pt_weights, dt)
    ix = _c(grid_pt_indexes, np.int32)
    g = _c(grad_grid, dt)
    b, n = ix.shape[:2]
    out = np.empty((b, n, 3), dt)
    getattr(lib(), "tpk_oracle_gridding_grad_" + suf)(ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(g.shape[1]),
                                                       _p(w, ptr), _p(ix, _i32p), _p(g, ptr), _p(out, ptr))
    return out


def cubic_feature_sampling(ptcloud, cubic_features, neighborhood_size=1):
    """CubicFeatureSamplingFunction.forward (cubic_feature_sampling.py:9-19): ptcloud (B,n,3) in grid units,
    cubic_features (B,c,m,m,m) -> (point_features (B,n,(2*ns)^3,c), grid_pt_indexes int32)."""
    dt, ptr, suf = _grid_types(ptcloud)
    p = _c(ptcloud, dt)
    feats = _c(cubic_features, dt)
    b, n, _ = p.shape
    c, scale = feats.shape[1], feats.shape[2]
    nv = (2 * neighborhood_size) ** 3
    out = np.empty((b, n, nv, c), dt)
    indexes = np.empty((b, n, nv), np.int32)
    getattr(lib(), "tpk_oracle_cubic_feature_sampling_" + suf)(ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(c),
                                                                ctypes.c_int(scale), ctypes.c_int(neighborhood_size),
                                                                _p(p, ptr), _p(feats, ptr), _p(out, ptr), _p(indexes, _i32p))
    return out, indexes


def cubic_feature_sampling_grad(scale, neighborhood_size, grad_point_features, grid_pt_indexes):
    dt, ptr, suf = _grid_types(grad_point_features)
    g = _c(grad_point_features, dt)
    ix = _c(grid_pt_indexes, np.int32)
    b, n, nv, c = g.shape
    grad_pt = np.empty((b, n, 3), dt)
    grad_feats = np.empty((b, c, scale, scale, scale), dt)
    getattr(lib(), "tpk_oracle_cubic_feature_sampling_grad_" + suf)(ctypes.c_int(b), ctypes.c_int(n), ctypes.c_int(c),
                                                                     ctypes.c_int(scale), ctypes.c_int(neighborhood_size),
                                                                     _p(g, ptr), _p(ix, _i32p), _p(grad_pt, ptr),
                                                                     _p(grad_feats, ptr))
    return grad_pt, grad_feats

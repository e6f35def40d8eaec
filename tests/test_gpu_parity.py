"""Parity of the HIP path with the oracle, on the GPU, through the package's public API
(Python layer -> points_cuda extension -> C ABI -> kernels).

Bar: integer outputs (neighbour / sample / argmin indices, hit counts) bit-exact; ball-query,
three_nn and chamfer distances bit-exact too (same unfused fp32 arithmetic); interpolated
features bit-exact forward; gradients within rtol 1e-5 / atol 1e-6 of the oracle's in-order sums, plus - for
the scatter sums, whose terms the kernels add in another order - two units in the last place of the sum of the
terms' magnitudes (needed by a handful of elements in 10^7: _assert_scatter_sum_close counts them).
"""
import os
import sys

import numpy as np
import pytest
import torch

from tests import workloads as W

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-6


@pytest.fixture(autouse=True)
def _announce(request):
    print("\n[gpu-case] %s" % request.node.nodeid, file=sys.stderr, flush=True)
    yield
    torch.cuda.synchronize()


def _np(t):
    return t.detach().cpu().numpy()


REORDER_ULPS = 2.0  # allowance for a different order of summation, in units of 2^-23 * sum of |terms|
TOLERANCE_LOG = os.path.join("gpurun_out", "gradient_tolerance.jsonl")  # one line per comparison


def _assert_scatter_sum_close(got, want, abs_sum, where=""):
    """Scatter-add results: the kernels add a target's terms in the order of its list (the reference's
    atomics: in no fixed order), the oracle in index order.  Both are fp32 sums of the same terms, so they
    agree to rtol/atol plus a reordering allowance proportional to the sum of the terms' magnitudes, which
    matters only where the terms cancel.  Returns (elements outside the strict bound, worst error in units
    of 2^-23 * sum of |terms| among those) and appends them to the file TOLERANCE_LOG names."""
    import json
    import os

    err = np.abs(got - want)
    strict = ATOL + RTOL * np.abs(want)
    outside = err > strict
    ulp = np.float32(2.0 ** -23) * abs_sum
    worst_ulps = float((err[outside] / np.maximum(ulp[outside], 1e-30)).max()) if outside.any() else 0.0
    record = {"case": where or os.environ.get("PYTEST_CURRENT_TEST", ""), "elements": int(outside.size),
              "outside_strict": int(outside.sum()), "worst_error": float(err.max()),
              "worst_over_strict": float((err / strict).max()), "worst_outside_in_ulps_of_abs_sum": worst_ulps}
    print("[tolerance] %s" % json.dumps(record), file=sys.stderr, flush=True)
    try:
        os.makedirs(os.path.dirname(TOLERANCE_LOG), exist_ok=True)
        with open(TOLERANCE_LOG, "a") as f:
            f.write(json.dumps(record) + "\n")
    except OSError:
        pass
    bad = err > strict + REORDER_ULPS * ulp
    assert not bad.any(), "%d of %d elements differ, worst %g" % (bad.sum(), bad.size, err.max())
    return int(outside.sum()), worst_ulps


def _in_threads(fn, tasks, workers=16):
    """fn(task) for every task on a pool of threads (the oracle's C functions run outside the interpreter
    lock); results in task order."""
    from concurrent.futures import ThreadPoolExecutor

    with ThreadPoolExecutor(max_workers=workers) as pool:
        return list(pool.map(fn, tasks))


def _clustered(g, B, n):
    centres = torch.rand(B, 6, 3, generator=g) * 4.0 - 2.0
    which = torch.randint(0, 6, (B, n), generator=g)
    pts = torch.gather(centres, 1, which.unsqueeze(-1).expand(B, n, 3)) + 0.1 * torch.randn(B, n, 3, generator=g)
    pts[:, : n // 10] = torch.rand(B, n // 10, 3, generator=g) * 6.0 - 3.0
    return pts.contiguous()


# ------------------------------------------------------------------ known answers on the GPU


def test_kat_ball_query_dense(tpk, dev):
    # reference test/test_ballquerry.py:18-23
    a = torch.tensor([[[0, 0, 0], [1, 0, 0], [2, 0, 0]], [[0, 0, 0], [1, 0, 0], [2, 0, 0]]]).float().to(dev)
    b = torch.tensor([[[0, 0, 0]], [[3, 0, 0]]]).float().to(dev)
    idx, dist = tpk.ball_query(1.01, 2, a, b)
    assert idx.dtype == torch.int64 and dist.dtype == torch.float32
    np.testing.assert_array_equal(_np(idx), [[[0, 1]], [[2, 2]]])
    np.testing.assert_array_equal(_np(dist), np.array([[[0, 1]], [[1, -1]]], np.float32))
    # sort=True: reference test/test_ballquerry.py:25-34 (CPU tensors there; its CUDA path raises)
    idx, dist = tpk.ball_query(1.01, 2, a, b, sort=True)
    np.testing.assert_array_equal(_np(idx), [[[0, 1]], [[2, 2]]])
    np.testing.assert_array_equal(_np(dist), np.array([[[0, 1]], [[1, -1]]], np.float32))
    c = torch.tensor([[[0, 0, 0], [1, 0, 0], [1, 1, 0]]]).float().to(dev)
    idx, dist = tpk.ball_query(1.01, 3, c, c, sort=True)
    np.testing.assert_array_equal(_np(idx), [[[0, 1, 0], [1, 0, 2], [2, 1, 2]]])


def test_kat_ball_query_partial(tpk, dev):
    # reference test/test_ballquerry.py:63-78
    x = torch.tensor([[10, 0, 0], [0.1, 0, 0], [0.2, 0, 0], [0.1, 0, 0]]).float().to(dev)
    y = torch.tensor([[0, 0, 0]]).float().to(dev)
    bx = torch.tensor([0, 0, 0, 1]).long().to(dev)
    by = torch.tensor([0]).long().to(dev)
    idx, dist2 = tpk.ball_query(0.2, 4, x, y, mode="PARTIAL_DENSE", batch_x=bx, batch_y=by)
    np.testing.assert_array_equal(_np(idx), [[1, 2, -1, -1]])
    np.testing.assert_array_almost_equal(_np(dist2), np.array([[0.01, 0.04, -1, -1]], np.float32))


def test_kat_fps(tpk, dev):
    # reference test/test_fps.py:13-16
    pts = torch.tensor([[[0, 0, 0], [1, 0, 0], [2, 0, 0]], [[-1, 1, 0], [0, 0, 10], [0, 0, 2]]]).float().to(dev)
    out = tpk.furthest_point_sample(pts, 2)
    assert out.dtype == torch.int32
    np.testing.assert_array_equal(_np(out), [[0, 2], [0, 1]])


def test_kat_three_nn(tpk, dev):
    # reference test/test_knn.py:14-20 (values; the GPU op returns euclidean distances)
    support = torch.tensor([[[0, 0, 0], [1, 0, 0], [2, 0, 0]]]).float().to(dev)
    query = torch.tensor([[[0, 0, 0]] * 3]).float().to(dev)
    dist, idx = tpk.three_nn(query, support)
    assert idx.dtype == torch.int32
    np.testing.assert_array_equal(_np(idx)[0, 0], [0, 1, 2])
    np.testing.assert_array_equal(_np(dist)[0, 0], [0.0, 1.0, 2.0])


def test_kat_grouping(tpk, dev):
    # reference test/test_grouping.py:13-41
    features = torch.tensor(
        [[[0, 10, 0], [1, 11, 0], [2, 12, 0]], [[100, 110, 120], [101, 111, 121], [102, 112, 122]]]
    ).float()
    idx = torch.tensor([[[1, 0], [0, 0]], [[0, 1], [1, 2]]]).long()
    expected = np.array(
        [
            [[[10, 0], [0, 0]], [[11, 1], [1, 1]], [[12, 2], [2, 2]]],
            [[[100, 110], [110, 120]], [[101, 111], [111, 121]], [[102, 112], [112, 122]]],
        ]
    )
    np.testing.assert_array_equal(_np(tpk.grouping_operation(features.to(dev), idx.to(dev))), expected)


def test_kat_chamfer(tpk, dev):
    # reference test/test_chamfer_dist.py:28-39
    from torch_points_kernels.chamfer_dist import chamfer_dist

    xyz1 = torch.tensor([[[0, 0, 0], [1, 1, 1], [2, 0, 1]]]).float().to(dev)
    xyz2 = torch.tensor([[[1, 0, 0], [1, 2, 1]]]).float().to(dev)
    assert abs(chamfer_dist(xyz1, xyz2).item() - 2.333333) < 1e-5
    assert abs(chamfer_dist(xyz1, xyz2, True).item() - 3.0) < 1e-5


# ------------------------------------------------------------------ ball query


@pytest.mark.parametrize(
    "B,N,M,r,ns",
    [
        (2, 100, 37, 0.3, 8),       # less than one tile, ragged query block
        (3, 2049, 65, 0.15, 16),    # one point past a tile boundary
        (2, 5000, 200, 0.08, 32),   # several tiles, some balls empty
        (1, 3000, 40, 0.6, 64),     # most balls overflow nsample (early exit)
        (2, 300, 10, 5.0, 500),     # nsample larger than the cloud
        (1, 64, 5, 0.2, 1),
    ],
)
def test_ball_query_dense_parity(tpk, oracle, dev, B, N, M, r, ns):
    g = torch.Generator().manual_seed(100 + N + M)
    xyz = torch.rand(B, N, 3, generator=g)
    new_xyz = torch.rand(B, M, 3, generator=g)
    idx, dist = tpk.ball_query(r, ns, xyz.to(dev), new_xyz.to(dev), mode="dense")
    want_idx, want_dist = oracle.ball_query_dense(r, ns, xyz.numpy(), new_xyz.numpy())
    np.testing.assert_array_equal(_np(idx), want_idx)
    np.testing.assert_array_equal(_np(dist), want_dist)


def test_ball_query_dense_boundary_and_empty(tpk, oracle, dev):
    # points exactly on the sphere are excluded (strict <); empty support gives zeros / -1
    xyz = torch.tensor([[[0, 0, 0], [0.5, 0, 0], [0.25, 0, 0], [5, 5, 5]]]).float()
    q = torch.tensor([[[1.0, 0, 0], [100, 0, 0], [0, 0, 0]]]).float()
    idx, dist = tpk.ball_query(0.5, 3, xyz.to(dev), q.to(dev))
    wi, wd = oracle.ball_query_dense(0.5, 3, xyz.numpy(), q.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist), wd)
    idx, dist = tpk.ball_query(0.5, 3, torch.zeros(2, 0, 3).to(dev), torch.zeros(2, 4, 3).to(dev))
    assert (idx == 0).all() and (dist == -1).all()


@pytest.mark.parametrize("kind", ["uniform", "clusters", "flat", "one_point", "outlier", "queries_outside", "non_finite", "line",
                                  "offset_3e4", "offset_1e6", "negative"])
@pytest.mark.parametrize("B,N,M,r,ns", [(2, 1024, 100, 0.2, 8), (4, 8192, 300, 0.05, 16), (1, 4096, 1030, 0.1, 100),
                                        (3, 1500, 17, 0.02, 4), (2, 6000, 64, 0.35, 32), (2, 3000, 200, 0.15, 64)])
def test_ball_query_dense_over_cells(tpk, oracle, dev, kind, B, N, M, r, ns):
    # clouds of 512 .. 8192 support points are hung into buckets of cells: shapes of clouds that stress the
    # cells (no extent along an axis, everything in one cell, a far point, queries away from the cloud,
    # coordinates that are not finite or far from the origin), checked against the scan in index order
    g = torch.Generator().manual_seed(7 * N + M)
    xyz = torch.rand(B, N, 3, generator=g)
    new_xyz = xyz[:, torch.randperm(N, generator=g)[:M] % N].clone() + 0.01 * torch.randn(B, M, 3, generator=g)
    if kind == "clusters":
        centres = torch.rand(B, 5, 3, generator=g)
        xyz = centres[:, torch.randint(0, 5, (N,), generator=g)] + 0.03 * torch.randn(B, N, 3, generator=g)
        new_xyz = xyz[:, :M].clone() + 0.005
    elif kind == "flat":
        xyz[..., 2] = 0.25
        new_xyz[..., 2] = 0.25 + 0.5 * r
    elif kind == "one_point":
        xyz[:] = 0.5
        new_xyz[:, ::2] = 0.5
    elif kind == "outlier":
        xyz[:, N // 3] = torch.tensor([400.0, -300.0, 1e6])
    elif kind == "queries_outside":
        new_xyz[:, ::3] += 2.0
        new_xyz[:, 1::3, 0] = -r * 0.5
    elif kind == "non_finite":
        xyz[:, 5, 0] = float("nan")
        xyz[:, 77, 1] = float("inf")
        xyz[:, 300, 2] = -float("inf")
        new_xyz[:, 3, 1] = float("nan")
        new_xyz[:, 4, 2] = float("inf")
    elif kind == "line":
        xyz[..., 1:] = 0.0
        new_xyz[..., 1:] = 0.0
    elif kind.startswith("offset"):
        # coordinates far from the origin: their rounding is no longer small against the radius
        xyz, new_xyz = xyz + float(kind[7:]), new_xyz + float(kind[7:])
    elif kind == "negative":
        xyz, new_xyz = xyz * 3.0 - 2.0, new_xyz * 3.0 - 2.0
    idx, dist = tpk.ball_query(r, ns, xyz.to(dev), new_xyz.contiguous().to(dev), mode="dense")
    want_idx, want_dist = oracle.ball_query_dense(r, ns, xyz.numpy(), new_xyz.numpy())
    np.testing.assert_array_equal(_np(idx), want_idx)
    np.testing.assert_array_equal(_np(dist), want_dist)
    # the nearest first (up to 64 neighbours the same buckets serve this)
    idx, dist = tpk.ball_query(r, ns, xyz.to(dev), new_xyz.contiguous().to(dev), mode="dense", sort=True)
    want_idx, want_dist = oracle.ball_query_sorted_dense(r, ns, xyz.numpy(), new_xyz.contiguous().numpy())
    np.testing.assert_array_equal(_np(idx), want_idx)
    np.testing.assert_array_equal(_np(dist), want_dist)


@pytest.mark.parametrize("kind", ["uniform", "clusters", "flat", "non_finite", "offset_1e4"])
@pytest.mark.parametrize("B,N,M,r,ns", [(2, 8193, 2500, 0.04, 16), (1, 20000, 2100, 0.03, 32), (3, 20000, 700, 0.25, 8),
                                        (1, 100000, 450, 0.015, 64), (1, 100000, 420, 0.2, 20), (2, 12289, 1700, 0.05, 100),
                                        (2, 9000, 50, 0.05, 16)])
def test_ball_query_dense_large_clouds(tpk, oracle, dev, kind, B, N, M, r, ns):
    # clouds above 8192 points do not fit in LDS: the dense layout takes the bin walk of the packed layout under its
    # own rules (strict <, indices inside the cloud, the first hit repeated behind the last); sparse balls (a few
    # points), dense ones (thousands: the walk hands over to the scan in index order) and windows that hold the end
    # of one cloud and the beginning of the next; the last shape has too few pairs to pay for the ordering and keeps
    # the scan of all pairs
    g = torch.Generator().manual_seed(3 * N + M)
    xyz = torch.rand(B, N, 3, generator=g)
    new_xyz = xyz[:, torch.randperm(N, generator=g)[:M]].clone() + 0.003 * torch.randn(B, M, 3, generator=g)
    if kind == "clusters":
        centres = torch.rand(B, 7, 3, generator=g)
        xyz = torch.stack([centres[b, torch.randint(0, 7, (N,), generator=g)] for b in range(B)]) + 0.02 * torch.randn(B, N, 3, generator=g)
        new_xyz = xyz[:, :M].clone() + 0.002
        new_xyz[:, ::5] += 3.0  # queries far from every point
    elif kind == "flat":
        xyz[..., 1] = -0.75
        new_xyz[..., 1] = -0.75 + 0.3 * r
    elif kind == "non_finite":
        xyz[:, 11, 0] = float("nan")
        xyz[:, N // 2, 2] = float("inf")
        new_xyz[:, 2, 1] = float("nan")
        new_xyz[:, 3, 0] = -float("inf")
    elif kind.startswith("offset"):
        xyz, new_xyz = xyz + float(kind[7:]), new_xyz + float(kind[7:])
    idx, dist = tpk.ball_query(r, ns, xyz.to(dev), new_xyz.contiguous().to(dev), mode="dense")
    want_idx, want_dist = oracle.ball_query_dense(r, ns, xyz.numpy(), new_xyz.contiguous().numpy())
    np.testing.assert_array_equal(_np(idx), want_idx)
    np.testing.assert_array_equal(_np(dist), want_dist)


def _packed_case(seed, sizes, qfrac, jitter):
    g = torch.Generator().manual_seed(seed)
    xs, ys, bx, by = [], [], [], []
    for c, n in enumerate(sizes):
        cloud = torch.rand(n, 3, generator=g)
        nq = max(0, int(n * qfrac))
        q = cloud[torch.sort(torch.randperm(n, generator=g)[:nq]).values] + jitter
        xs.append(cloud)
        ys.append(q)
        bx.append(torch.full((n,), c, dtype=torch.long))
        by.append(torch.full((nq,), c, dtype=torch.long))
    return torch.cat(xs), torch.cat(ys), torch.cat(bx), torch.cat(by)


@pytest.mark.parametrize(
    "sizes,qfrac,r,ns",
    [
        ((50, 70, 10), 0.5, 0.3, 8),            # clouds smaller than a query block: blocks straddle clouds
        ((3000, 1, 2100, 4500), 0.25, 0.1, 16),  # a one-point cloud in the middle
        ((2048, 2049), 0.1, 0.2, 64),
        ((700,), 1.0, 0.5, 1000),
    ],
)
def test_ball_query_partial_parity(tpk, oracle, dev, sizes, qfrac, r, ns):
    x, y, bx, by = _packed_case(7 + len(sizes), sizes, qfrac, 0.0)
    idx, dist = tpk.ball_query(r, ns, x.to(dev), y.to(dev), mode="partial_dense", batch_x=bx.to(dev), batch_y=by.to(dev))
    wi, wd = oracle.ball_query_partial_dense(r, ns, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist), wd)


def test_ball_query_partial_missing_and_extra_clouds(tpk, oracle, dev):
    # cloud ids with a gap (0, 2) and queries whose cloud has no support points (id 1, id 3)
    g = torch.Generator().manual_seed(5)
    x = torch.rand(300, 3, generator=g)
    bx = torch.cat([torch.zeros(100), torch.full((200,), 2)]).long()
    y = torch.rand(90, 3, generator=g)
    by = torch.cat([torch.zeros(30), torch.ones(20), torch.full((30,), 2)]).long()
    by = torch.cat([by, torch.full((10,), 3)]).long()
    idx, dist = tpk.ball_query(0.4, 12, x.to(dev), y.to(dev), mode="partial_dense", batch_x=bx.to(dev), batch_y=by.to(dev))
    got_idx, got_dist = _np(idx), _np(dist)
    wi, wd = oracle.ball_query_partial_dense(0.4, 12, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
    # the oracle (like the reference) only walks clouds 0..batch_x[-1]; cloud 3 stays -1
    np.testing.assert_array_equal(got_idx, wi)
    np.testing.assert_array_equal(got_dist, wd)
    assert (got_idx[30:50] == -1).all() and (got_idx[80:] == -1).all()


def test_ball_query_full_config1(tpk, oracle, dev):
    w = W.cfg1_ball_query_dense()
    idx, dist = tpk.ball_query(w["radius"], w["nsample"], w["xyz"].to(dev), w["new_xyz"].to(dev), mode="dense")
    wi, wd = oracle.ball_query_dense(w["radius"], w["nsample"], w["xyz"].numpy(), w["new_xyz"].numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist), wd)
    assert int(idx.min()) >= 0  # reference test/test_ballquerry.py:37-40


def test_ball_query_full_config4(tpk, oracle, dev):
    w = W.cfg4_ball_query_partial()
    x, y, bx, by = (w[k].to(dev) for k in ("x", "y", "batch_x", "batch_y"))
    idx, dist = tpk.ball_query(w["radius"], w["nsample"], x, y, mode="partial_dense", batch_x=bx, batch_y=by)
    assert idx.shape == (y.shape[0], w["nsample"])
    # Size-independent properties over the whole output, evaluated with torch on the GPU:
    valid = idx >= 0
    assert ((dist >= 0) == valid).all()
    cnt = valid.sum(1)
    pos = torch.arange(w["nsample"], device=dev).unsqueeze(0)
    assert (valid == (pos < cnt.unsqueeze(1))).all()          # hits first, -1 padding after
    safe = idx.clamp(min=0)
    assert (bx[safe][valid] == by.unsqueeze(1).expand_as(idx)[valid]).all()  # own cloud only
    d = x[safe] - y.unsqueeze(1)
    d2 = d[..., 0] * d[..., 0] + d[..., 1] * d[..., 1] + d[..., 2] * d[..., 2]
    assert (d2[valid] == dist[valid]).all()                    # stored distance = recomputed
    r2 = torch.tensor(w["radius"], dtype=torch.float32) * torch.tensor(w["radius"], dtype=torch.float32)
    assert (dist[valid] <= r2.item()).all()
    inc = (idx[:, 1:] > idx[:, :-1]) | ~valid[:, 1:]
    assert inc.all()                                           # ascending index order
    # Bit-exact against the oracle on EVERY query (each scans its whole cloud: 4.33 G pairs, split into
    # runs of consecutive queries over the host's threads).
    xs, ys, bxs, bys = w["x"].numpy(), w["y"].numpy(), w["batch_x"].numpy(), w["batch_y"].numpy()
    edges = np.linspace(0, ys.shape[0], 65).astype(np.int64)
    parts = _in_threads(lambda i: oracle.ball_query_partial_dense(
        w["radius"], w["nsample"], xs, ys[edges[i]:edges[i + 1]], bxs, bys[edges[i]:edges[i + 1]]), range(64))
    np.testing.assert_array_equal(_np(idx), np.concatenate([p[0] for p in parts]))
    np.testing.assert_array_equal(_np(dist), np.concatenate([p[1] for p in parts]))


@pytest.mark.parametrize(
    "sizes,qfrac,r,ns",
    [
        ((20000, 30000), 0.25, 0.03, 64),          # sparse neighbourhoods, clouds across window boundaries
        ((9000, 500, 12000), 0.5, 0.06, 8),         # more neighbours than nsample for many queries
        ((16384, 16384), 0.1, 0.05, 1),
        (tuple([50] * 200), 1.0, 0.3, 16),          # many tiny clouds in one window
        (tuple([50] * 200), 0.04, 0.3, 16),         # two queries per cloud: 32 clouds among 64 consecutive queries
        ((40000,), 0.3, 0.012, 32),                 # most balls hold the query point only
        ((90000, 20000), 0.05, 0.04, 32),           # 6 windows x 27 bins: more (window, bin) pairs than lanes
        ((500000, 24288), 0.002, 0.01, 16),         # 64 windows of 8192 rows, 62 of them one cloud's
        ((330000, 200000), 0.002, 0.01, 16),        # more rows than 64 windows of 8192: windows of 16384
    ],
)
def test_ball_query_partial_cell_search_parity(tpk, oracle, dev, sizes, qfrac, r, ns):
    # packed arrays large enough for the search over curve-ordered cells
    x, y, bx, by = _packed_case(11 + len(sizes), sizes, qfrac, 0.0)
    idx, dist = tpk.ball_query(r, ns, x.to(dev), y.to(dev), mode="partial_dense", batch_x=bx.to(dev), batch_y=by.to(dev))
    wi, wd = oracle.ball_query_partial_dense(r, ns, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist), wd)


def test_ball_query_partial_cell_search_edges(tpk, oracle, dev):
    g = torch.Generator().manual_seed(21)
    # points exactly on the sphere count (<=); duplicated support points; a query cloud without support
    lattice_ax = torch.arange(22, dtype=torch.float32) * 0.25
    lattice = torch.stack(torch.meshgrid(lattice_ax, lattice_ax, lattice_ax, indexing="ij"), -1).reshape(-1, 3)
    x = torch.cat([lattice, lattice[:3000], torch.rand(5000, 3, generator=g) * 5.0])
    bx = torch.cat([torch.zeros(lattice.shape[0] + 3000, dtype=torch.long), torch.full((5000,), 2, dtype=torch.long)])
    y = torch.cat([lattice[::7], torch.rand(300, 3, generator=g), torch.rand(400, 3, generator=g) * 5.0])
    by = torch.cat([torch.zeros(lattice[::7].shape[0], dtype=torch.long), torch.ones(300, dtype=torch.long),
                    torch.full((400,), 2, dtype=torch.long)])
    for r, ns in ((0.25, 10), (0.25, 40), (0.5, 16), (0.3, 3)):
        idx, dist = tpk.ball_query(r, ns, x.to(dev), y.to(dev), mode="partial_dense", batch_x=bx.to(dev), batch_y=by.to(dev))
        wi, wd = oracle.ball_query_partial_dense(r, ns, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist), wd)


# ------------------------------------------------------------------ ball query, sort=True


@pytest.mark.parametrize("B,n,m,r,ns", [(2, 40, 30, 0.5, 5), (2, 300, 515, 0.2, 16), (1, 1000, 100, 0.15, 33), (3, 777, 600, 0.1, 8),
                                        (1, 4096, 2500, 0.08, 32), (2, 600, 700, 0.3, 70), (1, 20000, 900, 0.05, 12),
                                        (2, 70, 9, 2.0, 100), (1, 3000, 17000, 0.04, 4), (2, 0, 5, 0.5, 3)])
def test_ball_query_sorted_dense_parity(tpk, oracle, dev, B, n, m, r, ns):
    # n support points, m queries; from 512 points on the search goes over cells, nsample above 32 in rounds
    g = torch.Generator().manual_seed(n + m + ns)
    cases = [(torch.rand(B, n, 3, generator=g), torch.rand(B, m, 3, generator=g))]
    if n >= 10:
        cases.append((_clustered(g, B, n) * 0.3, _clustered(g, B, m) * 0.3))
    for support, query in cases:
        idx, dist = tpk.ball_query(r, ns, support.to(dev), query.to(dev), sort=True)
        wi, wd = oracle.ball_query_sorted_dense(r, ns, support.numpy(), query.numpy())
        assert idx.dtype == torch.int64 and idx.shape == (B, m, ns)
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist), wd)


def test_ball_query_sorted_ties_and_boundary(tpk, oracle, dev):
    # lattice: many equal distances, and points exactly at the radius (d2 == r2 does not count: strict <)
    ax = torch.arange(9, dtype=torch.float32) * 0.25
    lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3).contiguous()
    g = torch.Generator().manual_seed(2)
    base = torch.rand(1, 300, 3, generator=g)
    tripled = torch.cat([base, base.flip(1), base], 1)[:, torch.randperm(900, generator=g)].contiguous()
    for support, query, r, ns in ((lattice, lattice, 0.25, 7), (lattice, lattice, 0.5, 40), (lattice, lattice + 0.125, 0.3, 9),
                                  (tripled, base, 0.2, 10), (tripled, base, 0.05, 3)):
        idx, dist = tpk.ball_query(r, ns, support.to(dev), query.contiguous().to(dev), sort=True)
        wi, wd = oracle.ball_query_sorted_dense(r, ns, support.numpy(), query.numpy())
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist), wd)
    idx, dist = tpk.ball_query(0.25, 7, lattice.to(dev), lattice.to(dev), sort=True)
    assert (_np(dist)[0, :, 0] == 0).all() and (_np(dist)[0, :, 1:] == -1).all()  # only the point itself is inside


@pytest.mark.parametrize("sizes,qfrac,r,ns", [((50, 70, 10), 0.5, 0.3, 8), ((3000, 1, 2100, 4500), 0.25, 0.1, 16),
                                               ((2048, 2049), 0.1, 0.2, 64), ((700,), 1.0, 0.5, 100),
                                               ((20000, 300), 0.05, 0.05, 12),
                                               # balls over most of a cloud (too many bins to walk), more
                                               # neighbours than a wavefront keeps (cloud by cloud), many windows
                                               ((3000, 4000), 0.2, 0.6, 32), ((9000, 5000), 0.1, 0.1, 70),
                                               ((70000,), 0.02, 0.03, 64), (tuple([40] * 150), 0.3, 0.4, 5)])
def test_ball_query_sorted_partial_parity(tpk, oracle, dev, sizes, qfrac, r, ns):
    x, y, bx, by = _packed_case(17 + len(sizes), sizes, qfrac, 0.01)
    idx, dist = tpk.ball_query(r, ns, x.to(dev), y.to(dev), mode="partial_dense", batch_x=bx.to(dev), batch_y=by.to(dev), sort=True)
    wi, wd = oracle.ball_query_sorted_partial(r, ns, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist), wd)


def test_ball_query_sorted_partial_missing_clouds(tpk, oracle, dev):
    # cloud ids with a gap (0, 2), queries whose cloud has no support points (1, 3), a cloud without queries
    g = torch.Generator().manual_seed(6)
    x = torch.rand(500, 3, generator=g)
    bx = torch.cat([torch.zeros(100), torch.full((200,), 2), torch.full((200,), 5)]).long()
    y = torch.rand(90, 3, generator=g)
    by = torch.cat([torch.zeros(30), torch.ones(20), torch.full((30,), 2), torch.full((10,), 3)]).long()
    idx, dist = tpk.ball_query(0.4, 12, x.to(dev), y.to(dev), mode="partial_dense", batch_x=bx.to(dev), batch_y=by.to(dev), sort=True)
    wi, wd = oracle.ball_query_sorted_partial(0.4, 12, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist), wd)
    assert (_np(idx)[30:50] == -1).all() and (_np(idx)[80:] == -1).all()


# ------------------------------------------------------------------ FPS


@pytest.mark.parametrize(
    "B,N,npoint",
    [(2, 3, 3), (3, 100, 40), (2, 512, 100), (2, 513, 513), (2, 1024, 256), (2, 1500, 300), (2, 4096, 512),
     (1, 4097, 90), (1, 7000, 128), (3, 8193, 70), (2, 16384, 200)],
)
def test_fps_parity(tpk, oracle, dev, B, N, npoint):
    g = torch.Generator().manual_seed(N)
    xyz = torch.randn(B, N, 3, generator=g)
    out = tpk.furthest_point_sample(xyz.to(dev), npoint)
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(xyz.numpy(), npoint))


@pytest.mark.parametrize("B,N,npoint", [(2, 20000, 150), (1, 16385, 90), (2, 50001, 300), (1, 163840, 64),
                                        (3, 16385, 60), (3, 30000, 100), (2, 65537, 50), (5, 33333, 40)])
def test_fps_cells_in_memory_parity(tpk, oracle, dev, B, N, npoint):
    # more points than one workgroup keeps in registers: cells of 64 points in memory, of clouds that are brought
    # into a coarse order first, chunk by chunk of 16384 points of the batch (the later shapes: chunks that hold
    # the end of one cloud and the beginning of the next)
    g = torch.Generator().manual_seed(N)
    xyz = _clustered(g, B, N) if N % 2 else torch.rand(B, N, 3, generator=g)
    out = tpk.furthest_point_sample(xyz.to(dev), npoint)
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(xyz.numpy(), npoint))


def test_fps_cells_in_memory_ties(tpk, oracle, dev):
    g = torch.Generator().manual_seed(11)
    ax = torch.arange(30, dtype=torch.float32)
    lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3) + 1.0
    shuffled = lattice[:, torch.randperm(lattice.shape[1], generator=g)]
    for pts in (lattice, shuffled):
        out = tpk.furthest_point_sample(pts.contiguous().to(dev), 300)
        np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(pts.numpy(), 300))
    # every point three times, some points never eligible, 2 clouds, more samples than distinct points
    base = torch.rand(2, 7000, 3, generator=g) * 4.0 - 2.0
    base[:, :37] *= 0.004
    xyz = torch.cat([base, base.flip(1), base], 1)[:, torch.randperm(21000, generator=g)].contiguous()
    out = tpk.furthest_point_sample(xyz.to(dev), 7100)
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(xyz.numpy(), 7100))
    # nothing eligible; a single eligible point
    tiny = torch.full((2, 20000, 3), 0.001)
    assert (tpk.furthest_point_sample(tiny.to(dev), 10) == 0).all()
    tiny[1, 18123] = 1.0
    np.testing.assert_array_equal(_np(tpk.furthest_point_sample(tiny.to(dev), 5)),
                                  oracle.furthest_point_sample(tiny.numpy(), 5))
    # a handful of eligible points: once all are sampled, their minima are all 0 and the tie rule decides
    for first in (0.001, 2.0):
        few = torch.full((2, 20000, 3), 0.001)
        few[:, 0] = first
        few[:, [18123, 77, 4500, 4501, 16000], 0] = torch.tensor([1.0, 3.0, 4.5, 5.0, 9.0])
        np.testing.assert_array_equal(_np(tpk.furthest_point_sample(few.to(dev), 12)), oracle.furthest_point_sample(few.numpy(), 12))


def test_fps_streaming_path_parity(tpk, oracle, dev):
    # more points than the cell kernel keeps summaries for
    g = torch.Generator().manual_seed(77)
    xyz = torch.rand(2, 170000, 3, generator=g)
    out = tpk.furthest_point_sample(xyz.to(dev), 40)
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(xyz.numpy(), 40))


def test_fps_ties_origin_skip_and_exhaustion(tpk, oracle, dev):
    # duplicated points (exact ties in every round), points near the origin (never eligible)
    # and more samples than distinct points: all decided by the tie rule.
    g = torch.Generator().manual_seed(9)
    base = torch.rand(1, 40, 3, generator=g) + 0.5
    xyz = torch.cat([base, base, base.flip(1), torch.full((1, 8, 3), 0.01)], 1)[:, torch.randperm(128, generator=g)]
    for n in (128, 100, 8):
        pts = xyz[:, :n].contiguous()
        out = tpk.furthest_point_sample(pts.to(dev), n)
        np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(pts.numpy(), n))
    # lattice: many exactly equal distances, larger than one reference block
    ax = torch.arange(12, dtype=torch.float32)
    lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3) + 1.0
    out = tpk.furthest_point_sample(lattice.to(dev), 300)
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(lattice.numpy(), 300))
    # lattices of 729 and 2197 points: the cloud sizes of the other register layouts
    for side in (9, 13):
        ax = torch.arange(side, dtype=torch.float32)
        lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3) + 1.0
        out = tpk.furthest_point_sample(lattice.to(dev), 200)
        np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(lattice.numpy(), 200))
    # nothing eligible
    tiny = torch.full((2, 50, 3), 0.001)
    assert (tpk.furthest_point_sample(tiny.to(dev), 10) == 0).all()


def test_fps_ties_large_cloud(tpk, oracle, dev):
    # the same tie cases at cloud sizes served by the kernel that sorts the cloud along a space
    # filling curve (slots no longer in index order: the tie key has to be applied explicitly)
    ax = torch.arange(24, dtype=torch.float32)
    lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3) + 1.0
    g = torch.Generator().manual_seed(5)
    shuffled = lattice[:, torch.randperm(lattice.shape[1], generator=g)]
    for pts in (lattice, shuffled):
        out = tpk.furthest_point_sample(pts.contiguous().to(dev), 400)
        np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(pts.numpy(), 400))
    # every point three times, some points never eligible, 2 clouds
    base = torch.rand(2, 3000, 3, generator=g) * 4.0 - 2.0
    base[:, :37] *= 0.004
    xyz = torch.cat([base, base.flip(1), base], 1)[:, torch.randperm(9000, generator=g)].contiguous()
    out = tpk.furthest_point_sample(xyz.to(dev), 3100)  # more samples than distinct points
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(xyz.numpy(), 3100))
    # nothing eligible
    tiny = torch.full((2, 9000, 3), 0.001)
    assert (tpk.furthest_point_sample(tiny.to(dev), 10) == 0).all()
    # a single eligible point
    tiny[1, 8123] = 1.0
    out = _np(tpk.furthest_point_sample(tiny.to(dev), 5))
    np.testing.assert_array_equal(out, oracle.furthest_point_sample(tiny.numpy(), 5))
    # a handful of eligible points, the first point among them or not: once all are sampled, their minima are
    # all 0 and the tie rule decides among them
    for first in (0.001, 2.0):
        few = torch.full((2, 9000, 3), 0.001)
        few[:, 0] = first
        few[:, [8123, 77, 4500, 4501, 6000], 0] = torch.tensor([1.0, 3.0, 4.5, 5.0, 9.0])
        np.testing.assert_array_equal(_np(tpk.furthest_point_sample(few.to(dev), 12)), oracle.furthest_point_sample(few.numpy(), 12))


@pytest.mark.parametrize("B,N,npoint,kind", [(2, 16384, 2, "uniform"), (1, 12000, 3, "clusters"), (2, 9000, 777, "clusters"),
                                             (1, 16384, 5000, "uniform"), (1, 10000, 10000, "shell"), (3, 8200, 1001, "line"),
                                             (1, 16000, 900, "two_scales"),
                                             # clouds in cells in memory
                                             (2, 16385, 3, "uniform"), (2, 40000, 3001, "uniform"), (1, 30000, 2000, "clusters"),
                                             (1, 20000, 20000, "shell"), (2, 33000, 1500, "line"), (1, 50000, 1200, "two_scales"),
                                             (1, 163840, 700, "uniform"), (2, 24000, 2500, "four_times")])
def test_fps_several_samples_per_round(tpk, oracle, dev, B, N, npoint, kind):
    # clouds of 8193 .. 163840 points take up to 16 samples per round (the points with the largest minima, as long
    # as none changes the next one's minimum): sample counts that end inside a round, every point sampled,
    # clouds whose largest minima lie close together (a line, dense clusters next to a sparse background), every
    # point four times (each round's runner-up is its sample's twin)
    g = torch.Generator().manual_seed(N + npoint)
    xyz = torch.rand(B, N, 3, generator=g) + 0.1
    if kind == "clusters":
        centres = torch.rand(B, 6, 3, generator=g) * 4 + 0.5
        xyz = centres[:, torch.randint(0, 6, (N,), generator=g)] + 0.05 * torch.randn(B, N, 3, generator=g)
    elif kind == "shell":
        p = torch.randn(B, N, 3, generator=g)
        xyz = p / p.norm(dim=2, keepdim=True) * 2.0 + 3.0
    elif kind == "line":
        xyz[..., 1:] = 0.5
    elif kind == "two_scales":
        xyz[:, : N // 2] = xyz[:, : N // 2] * 0.01 + 1.0
        xyz[:, N // 2 :] = xyz[:, N // 2 :] * 20.0
    elif kind == "four_times":
        xyz = xyz[:, : N // 4].repeat(1, 4, 1)[:, torch.randperm(N, generator=g)]
    out = tpk.furthest_point_sample(xyz.contiguous().to(dev), npoint)
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(xyz.contiguous().numpy(), npoint))


@pytest.mark.parametrize("N", [16384, 40000])
def test_fps_lattice_half_random_half(tpk, oracle, dev, N):
    # Half of the cloud lies on a lattice (rounds with equal maxima: one sample each, by the reference's tie rule, and
    # the next rounds go there at once), half is random (rounds of several samples): sampling half of all points
    # alternates between the two kinds of rounds thousands of times, in the register kernel and in the one with cells
    # in memory.
    g = torch.Generator().manual_seed(N)
    side = int(round((N // 2) ** (1.0 / 3.0))) + 1
    axis = torch.arange(side, dtype=torch.float32) * 0.125
    lattice = torch.stack(torch.meshgrid(axis, axis, axis, indexing="ij"), -1).reshape(-1, 3)[: N // 2] + 0.25
    scattered = torch.rand(N - N // 2, 3, generator=g) * (side * 0.125) + 0.25
    scattered[:, 0] += side * 0.125 + 0.3  # beside the lattice, so that both halves keep being sampled
    cloud = torch.cat([lattice, scattered])[torch.randperm(N, generator=g)].unsqueeze(0).contiguous()
    out = tpk.furthest_point_sample(cloud.to(dev), N // 2)
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(cloud.numpy(), N // 2))


def test_fps_full_config2(tpk, oracle, dev):
    w = W.cfg2_fps()
    xyz = w["xyz"].to(dev)
    out = tpk.furthest_point_sample(xyz, w["npoint"])
    out2 = tpk.furthest_point_sample(xyz, w["npoint"])
    assert (out == out2).all()  # deterministic
    np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(w["xyz"].numpy(), w["npoint"]))


# ------------------------------------------------------------------ three_nn / three_interpolate


@pytest.mark.parametrize("B,n,m", [(2, 3, 1), (2, 5, 2), (3, 70, 3), (2, 1000, 1025), (1, 2500, 4096), (4, 513, 300)])
def test_three_nn_parity(tpk, oracle, dev, B, n, m):
    g = torch.Generator().manual_seed(n * 7 + m)
    unknown = torch.randn(B, n, 3, generator=g)
    known = torch.randn(B, m, 3, generator=g)
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    dist2, idx = native.three_nn(unknown.to(dev), known.to(dev))
    wd, wi = oracle.three_nn(unknown.numpy(), known.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist2), wd)
    dist, idx2 = tpk.three_nn(unknown.to(dev), known.to(dev))
    np.testing.assert_array_equal(_np(dist), np.sqrt(wd))


@pytest.mark.parametrize("B,n,m", [(2, 512, 512), (3, 1000, 777), (2, 5000, 515), (1, 16384, 4096), (2, 700, 16384),
                                   (2, 20000, 600), (1, 3000, 40000), (1, 33000, 16385)])
def test_three_nn_cell_search_parity(tpk, oracle, dev, B, n, m):
    # cloud sizes served by the search over curve-ordered cells (512..16384 points each side)
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    g = torch.Generator().manual_seed(n * 3 + m)
    for unknown, known in ((torch.rand(B, n, 3, generator=g), torch.rand(B, m, 3, generator=g)),
                           (_clustered(g, B, n), _clustered(g, B, m))):
        dist2, idx = native.three_nn(unknown.to(dev), known.to(dev))
        wd, wi = oracle.three_nn(unknown.numpy(), known.numpy())
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist2), wd)


def test_three_nn_cell_search_ties(tpk, oracle, dev):
    # equal distances in every triple: tripled known points, lattices, a collapsed cloud
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    g = torch.Generator().manual_seed(4)
    k = torch.rand(1, 400, 3, generator=g)
    tripled = torch.cat([k, k.flip(1), k], 1)[:, torch.randperm(1200, generator=g)]
    ax = torch.arange(10, dtype=torch.float32)
    lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3)
    cases = [(torch.rand(1, 600, 3, generator=g), tripled),
             (lattice + 0.5, lattice[:, torch.randperm(1000, generator=g)]),
             (lattice, lattice),
             (torch.rand(1, 520, 3, generator=g), torch.full((1, 600, 3), 0.5))]
    # the same above 16384 points, where a cloud is ordered in several windows: equal points in
    # different windows, a lattice of 27000 points
    k = torch.rand(1, 7000, 3, generator=g)
    big = torch.cat([k, k.flip(1), k], 1)[:, torch.randperm(21000, generator=g)]
    ax = torch.arange(30, dtype=torch.float32)
    big_lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3)
    cases += [(torch.rand(1, 900, 3, generator=g), big), (big_lattice[:, :17000] + 0.5, big_lattice)]
    for unknown, known in cases:
        unknown, known = unknown.contiguous(), known.contiguous()
        dist2, idx = native.three_nn(unknown.to(dev), known.to(dev))
        wd, wi = oracle.three_nn(unknown.numpy(), known.numpy())
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist2), wd)


@pytest.mark.parametrize("kind", ["uniform", "clusters", "flat", "one_point", "outlier", "queries_outside", "non_finite", "line",
                                  "lattice", "tripled", "offset_1e5", "two_points"])
@pytest.mark.parametrize("B,n,m", [(2, 700, 1024), (1, 5000, 4096), (3, 300, 8192), (300, 40, 1500), (1, 2100, 3000)])
def test_three_nn_grid_in_lds(tpk, oracle, dev, kind, B, n, m):
    # known clouds of 1024 .. 8192 points are sorted into the cells of a grid in LDS, one lane per query: clouds
    # that stress the grid and the widening of the examined block (no extent along an axis, everything in one
    # cell, a far point that makes all cells wide, queries far from the cloud, coordinates that are not finite)
    # and equal distances in every triple (lattices, tripled points), against the scan in index order
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    g = torch.Generator().manual_seed(11 * n + m)
    known = torch.rand(B, m, 3, generator=g)
    unknown = torch.rand(B, n, 3, generator=g)
    if kind == "clusters":
        centres = torch.rand(B, 4, 3, generator=g)
        known = centres[:, torch.randint(0, 4, (m,), generator=g)] + 0.004 * torch.randn(B, m, 3, generator=g)
    elif kind == "flat":
        known[..., 2] = 0.25
    elif kind == "one_point":
        known[:] = 0.5
    elif kind == "outlier":
        known[:, m // 3] = torch.tensor([400.0, -300.0, 1e6])
    elif kind == "queries_outside":
        unknown[:, ::3] += 5.0
        unknown[:, 1::3, 1] = -40.0
    elif kind == "non_finite":
        known[:, 5, 0] = float("nan")
        known[:, 77, 1] = float("inf")
        known[:, 300, 2] = -float("inf")
        unknown[:, 3, 1] = float("nan")
        unknown[:, 4, 2] = float("inf")
    elif kind == "line":
        known[..., 1:] = 0.0
    elif kind == "lattice":
        known = torch.round(known * 12) / 4
        unknown = torch.round(unknown * 12) / 4 + 0.125
    elif kind == "tripled":
        k = known[:, : m // 3]
        known = torch.cat([k, k.flip(1), k, known[:, : m - 3 * (m // 3)]], 1)[:, torch.randperm(m, generator=g)]
    elif kind == "offset_1e5":
        known, unknown = known + 1e5, unknown + 1e5
    elif kind == "two_points":
        known[:, ::2] = 0.25
        known[:, 1::2] = 0.75
    unknown, known = unknown.contiguous(), known.contiguous()
    dist2, idx = native.three_nn(unknown.to(dev), known.to(dev))
    wd, wi = oracle.three_nn(unknown.numpy(), known.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist2), wd)
    # without a workspace the grid has nothing to hand uneven clouds over to and answers them itself
    import ctypes
    import os

    lib = ctypes.CDLL(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "torch-points-kernels_amd",
                                   "torch_points_kernels", "libtpk_hip.so"))
    u, k = unknown.to(dev), known.to(dev)
    dist2.fill_(-1.0)
    idx.fill_(-1)
    st = lib.tpk_three_nn_f32(B, n, m, ctypes.c_void_p(u.data_ptr()), ctypes.c_void_p(k.data_ptr()),
                              ctypes.c_void_p(dist2.data_ptr()), ctypes.c_void_p(idx.data_ptr()), None, ctypes.c_size_t(0),
                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist2), wd)


def test_three_nn_ties(tpk, oracle, dev):
    # duplicated known points: equal distances must keep the lower index first
    g = torch.Generator().manual_seed(3)
    k = torch.rand(1, 300, 3, generator=g)
    known = torch.cat([k, k, k], 1)
    unknown = torch.rand(1, 257, 3, generator=g)
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    dist2, idx = native.three_nn(unknown.to(dev), known.to(dev))
    wd, wi = oracle.three_nn(unknown.numpy(), known.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist2), wd)


def _interp_case(B, C, m, n, seed):
    g = torch.Generator().manual_seed(seed)
    feats = torch.randn(B, C, m, generator=g)
    idx = torch.randint(0, m, (B, n, 3), generator=g, dtype=torch.int32)
    w = torch.rand(B, n, 3, generator=g)
    w = w / w.sum(2, keepdim=True)
    gout = torch.randn(B, C, n, generator=g)
    return feats, idx, w, gout


@pytest.mark.parametrize(
    "B,C,m,n",
    [(2, 5, 40, 70), (3, 30, 100, 500), (2, 19, 4096, 3000), (1, 3, 20000, 1500), (1, 4, 40000, 999)],
)
def test_three_interpolate_parity(tpk, oracle, dev, B, C, m, n):
    # m = 20000 leaves room for one row in LDS, m = 40000 for none (direct path)
    feats, idx, w, gout = _interp_case(B, C, m, n, m + n)
    f = feats.to(dev).requires_grad_(True)
    out = tpk.three_interpolate(f, idx.to(dev), w.to(dev))
    np.testing.assert_array_equal(_np(out), oracle.three_interpolate(feats.numpy(), idx.numpy(), w.numpy()))
    out.backward(gout.to(dev))
    want = oracle.three_interpolate_grad(gout.numpy(), idx.numpy(), w.numpy(), m)
    abs_sum = oracle.three_interpolate_grad(gout.abs().numpy(), idx.numpy(), w.numpy(), m)
    _assert_scatter_sum_close(_np(f.grad), want, abs_sum)


def test_three_interpolate_colliding_indices(tpk, oracle, dev):
    # every column points at the same few rows entries: worst case for the atomic accumulation
    B, C, m, n = 1, 8, 64, 5000
    feats, _, w, gout = _interp_case(B, C, m, n, 4)
    idx = torch.zeros(B, n, 3, dtype=torch.int32)
    idx[..., 1] = 1
    idx[..., 2] = torch.arange(n) % 2
    f = feats.to(dev).requires_grad_(True)
    out = tpk.three_interpolate(f, idx.to(dev), w.to(dev))
    np.testing.assert_array_equal(_np(out), oracle.three_interpolate(feats.numpy(), idx.numpy(), w.numpy()))
    out.backward(gout.to(dev))
    want = oracle.three_interpolate_grad(gout.numpy(), idx.numpy(), w.numpy(), m)
    abs_sum = oracle.three_interpolate_grad(gout.abs().numpy(), idx.numpy(), w.numpy(), m)
    _assert_scatter_sum_close(_np(f.grad), want, abs_sum)  # sums of ~5000 terms each



@pytest.mark.parametrize("n,m,C", [(20001, 130, 3), (16388, 64, 2), (40000, 1000, 5)])
def test_three_interpolate_grad_long_rows(tpk, oracle, dev, n, m, C):
    # rows of grad_out longer than one staged piece (16384 columns): lists per piece, later
    # pieces add to earlier ones; a few targets with very long lists, some with none
    B = 2
    feats, idx, w, gout = _interp_case(B, C, m, n, n + m)
    g = torch.Generator().manual_seed(n)
    heavy = torch.rand(B, n, 3, generator=g) < 0.3
    idx = torch.where(heavy, torch.randint(0, 3, (B, n, 3), generator=g).int(), idx)
    idx[idx == m - 1] = 0  # the last target keeps an empty list
    f = feats.to(dev).requires_grad_(True)
    out = tpk.three_interpolate(f, idx.to(dev), w.to(dev))
    np.testing.assert_array_equal(_np(out), oracle.three_interpolate(feats.numpy(), idx.numpy(), w.numpy()))
    out.backward(gout.to(dev))
    want = oracle.three_interpolate_grad(gout.numpy(), idx.numpy(), w.numpy(), m)
    abs_sum = oracle.three_interpolate_grad(gout.abs().numpy(), idx.numpy(), w.numpy(), m)
    _assert_scatter_sum_close(_np(f.grad), want, abs_sum)
    assert (_np(f.grad)[:, :, m - 1] == 0).all()


def test_interpolate_full_config3a(tpk, oracle, dev):
    w = W.cfg3a_interpolate()
    unknown, known = w["unknown"].to(dev), w["known"].to(dev)
    dist, idx = tpk.three_nn(unknown, known)
    wd2, wi = oracle.three_nn(w["unknown"].numpy(), w["known"].numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist), np.sqrt(wd2))
    weight = W.inverse_distance_weights(dist)
    feats = w["features"].to(dev).requires_grad_(True)
    out = tpk.three_interpolate(feats, idx, weight)
    np.testing.assert_array_equal(_np(out), oracle.three_interpolate(w["features"].numpy(), wi, _np(weight)))
    out.backward(w["grad_out"].to(dev))
    want = oracle.three_interpolate_grad(w["grad_out"].numpy(), wi, _np(weight), known.shape[1])
    abs_sum = oracle.three_interpolate_grad(w["grad_out"].abs().numpy(), wi, _np(weight), known.shape[1])
    outside, _ = _assert_scatter_sum_close(_np(feats.grad), want, abs_sum)
    # measured: 0 of 8 388 608 elements outside rtol 1e-5 / atol 1e-6 (the order of a list varies from run to run)
    assert outside <= 8


def test_backward_over_lists_built_in_the_forward_pass(tpk, oracle, dev):
    """With autograd recording, the forward pass also builds the per-target lists and the
    backward pass only walks them: same gradient as the stand-alone call (which builds them itself), for
    both gathers; one set of lists serves several backward passes; without a gradient nothing is built."""
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    feats, idx, w, gout = _interp_case(3, 21, 700, 5000, 99)
    f, i, wt, go = feats.to(dev), idx.to(dev), w.to(dev), gout.to(dev)
    out, lists = native.three_interpolate_recording(f, i, wt)
    assert lists.numel() > 0 and lists.dtype == torch.uint8
    np.testing.assert_array_equal(_np(out), oracle.three_interpolate(feats.numpy(), idx.numpy(), w.numpy()))
    want = oracle.three_interpolate_grad(gout.numpy(), idx.numpy(), w.numpy(), 700)
    abs_sum = oracle.three_interpolate_grad(gout.abs().numpy(), idx.numpy(), w.numpy(), 700)
    first = native.three_interpolate_grad_lists(go, lists, 700)
    _assert_scatter_sum_close(_np(first), want, abs_sum)
    assert torch.equal(native.three_interpolate_grad_lists(go, lists, 700), first)  # (the walk leaves the lists as they are)
    _assert_scatter_sum_close(_np(native.three_interpolate_grad(go, i, wt, 700)), want, abs_sum)
    fr = f.clone().requires_grad_(True)
    y = tpk.three_interpolate(fr, i, wt)
    y.backward(go, retain_graph=True)
    once = fr.grad.clone()
    y.backward(go)
    _assert_scatter_sum_close(_np(once), want, abs_sum)
    _assert_scatter_sum_close(_np(fr.grad), 2 * want, 2 * abs_sum)
    # on a stream of the caller's own
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fs = f.clone().requires_grad_(True)
        tpk.three_interpolate(fs, i, wt).backward(go)
    torch.cuda.current_stream().wait_stream(side)
    _assert_scatter_sum_close(_np(fs.grad), want, abs_sum)
    # grouping
    g = torch.Generator().manual_seed(5)
    feats = torch.randn(2, 9, 3000, generator=g)
    gidx = torch.randint(0, 3000, (2, 300, 16), generator=g)
    gg = torch.randn(2, 9, 300, 16, generator=g)
    out, lists = native.grouping_operation_recording(feats.to(dev), gidx.to(dev))
    np.testing.assert_array_equal(_np(out), oracle.grouping_operation(feats.numpy(), gidx.numpy()))
    want = oracle.grouping_operation_grad(gg.numpy(), gidx.numpy(), 3000)
    abs_sum = oracle.grouping_operation_grad(gg.abs().numpy(), gidx.numpy(), 3000)
    _assert_scatter_sum_close(_np(native.grouping_operation_grad_lists(gg.to(dev), lists, 3000)), want, abs_sum)
    _assert_scatter_sum_close(_np(native.grouping_operation_grad(gg.to(dev), gidx.to(dev), 3000)), want, abs_sum)
    # shapes the lists do not serve (too many targets for LDS): empty lists, and autograd takes the other backward pass
    feats, idx, w, gout = _interp_case(1, 3, 60000, 900, 7)
    out, lists = native.three_interpolate_recording(feats.to(dev), idx.to(dev), w.to(dev))
    assert lists.numel() == 0
    fb = feats.to(dev).requires_grad_(True)
    tpk.three_interpolate(fb, idx.to(dev), w.to(dev)).backward(gout.to(dev))
    _assert_scatter_sum_close(_np(fb.grad), oracle.three_interpolate_grad(gout.numpy(), idx.numpy(), w.numpy(), 60000),
                              oracle.three_interpolate_grad(gout.abs().numpy(), idx.numpy(), w.numpy(), 60000))


# ------------------------------------------------------------------ grouping


@pytest.mark.parametrize("B,C,N,npoint,nsample", [(2, 3, 10, 4, 2), (2, 17, 1000, 129, 16), (1, 5, 30000, 64, 8), (1, 2, 50000, 40, 4)])
def test_grouping_parity(tpk, oracle, dev, B, C, N, npoint, nsample):
    g = torch.Generator().manual_seed(N + npoint)
    feats = torch.randn(B, C, N, generator=g)
    idx = torch.randint(0, N, (B, npoint, nsample), generator=g)
    gout = torch.randn(B, C, npoint, nsample, generator=g)
    f = feats.to(dev).requires_grad_(True)
    out = tpk.grouping_operation(f, idx.to(dev))
    np.testing.assert_array_equal(_np(out), oracle.grouping_operation(feats.numpy(), idx.numpy()))
    out.backward(gout.to(dev))
    want = oracle.grouping_operation_grad(gout.numpy(), idx.numpy(), N)
    _assert_scatter_sum_close(_np(f.grad), want, oracle.grouping_operation_grad(gout.abs().numpy(), idx.numpy(), N))



@pytest.mark.parametrize("N,npoint,nsample,C", [(1000, 1250, 32, 3), (70, 2049, 8, 2), (5000, 333, 50, 1)])
def test_grouping_grad_long_rows(tpk, oracle, dev, N, npoint, nsample, C):
    # npoint * nsample above one staged piece; clustered indices give long and empty lists
    B = 2
    g = torch.Generator().manual_seed(N + npoint)
    feats = torch.randn(B, C, N, generator=g)
    idx = torch.randint(0, N, (B, npoint, nsample), generator=g)
    idx[:, :, : nsample // 2] = idx[:, :, : nsample // 2] % 5
    gout = torch.randn(B, C, npoint, nsample, generator=g)
    f = feats.to(dev).requires_grad_(True)
    out = tpk.grouping_operation(f, idx.to(dev))
    np.testing.assert_array_equal(_np(out), oracle.grouping_operation(feats.numpy(), idx.numpy()))
    out.backward(gout.to(dev))
    want = oracle.grouping_operation_grad(gout.numpy(), idx.numpy(), N)
    _assert_scatter_sum_close(_np(f.grad), want, oracle.grouping_operation_grad(gout.abs().numpy(), idx.numpy(), N))


def test_grouping_full_config3b(tpk, oracle, dev):
    w = W.cfg3b_grouping()
    f = w["features"].to(dev).requires_grad_(True)
    idx = w["idx"].to(dev)
    out = tpk.grouping_operation(f, idx)
    # the reference implementation itself: torch.gather on the repeated index (torchpoints.py:129-146)
    all_idx = idx.reshape(idx.shape[0], -1).unsqueeze(1).expand(-1, f.shape[1], -1)
    assert (out == f.detach().gather(2, all_idx).reshape(out.shape)).all()
    np.testing.assert_array_equal(_np(out[:2]), oracle.grouping_operation(w["features"][:2].numpy(), w["idx"][:2].numpy()))
    out.backward(w["grad_out"].to(dev))
    want = oracle.grouping_operation_grad(w["grad_out"].numpy(), w["idx"].numpy(), f.shape[2])
    abs_sum = oracle.grouping_operation_grad(w["grad_out"].abs().numpy(), w["idx"].numpy(), f.shape[2])
    outside, _ = _assert_scatter_sum_close(_np(f.grad), want, abs_sum)
    # measured: 1 of 8 388 608 elements outside rtol 1e-5 / atol 1e-6, by less than one unit in the last place of
    # the sum of the terms' magnitudes (a sum of 8 terms that cancel)
    assert outside <= 8


# ------------------------------------------------------------------ knn (general k)


@pytest.mark.parametrize("B,n,m,k", [(1, 3, 1, 3), (2, 40, 70, 5), (2, 300, 515, 16), (1, 1000, 100, 33), (2, 70, 9, 70),
                                     (2, 512, 512, 1), (3, 1000, 777, 8), (1, 4096, 2500, 16), (2, 600, 700, 40),
                                     (1, 20000, 900, 12), (1, 3000, 17000, 4)])
def test_knn_parity(tpk, oracle, dev, B, n, m, k):
    # n support points, m queries; below 512 points all pairs are tested, above the search goes over cells
    g = torch.Generator().manual_seed(n + m + k)
    for support, query in ((torch.rand(B, n, 3, generator=g), torch.rand(B, m, 3, generator=g)),
                           (_clustered(g, B, n), _clustered(g, B, m))):
        idx, dist2 = tpk.knn(support.to(dev), query.to(dev), k)
        wi, wd = oracle.knn(support.numpy(), query.numpy(), k)
        assert idx.dtype == torch.int64 and idx.shape == (B, m, k)
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist2), wd)


def test_knn_ties_and_errors(tpk, oracle, dev):
    # reference test/test_knn.py:14-23
    support = torch.tensor([[[0, 0, 0], [1, 0, 0], [2, 0, 0]]]).float().to(dev)
    query = torch.tensor([[[0, 0, 0]]]).float().to(dev)
    idx, dist = tpk.knn(support, query, 3)
    assert idx.tolist() == [[[0, 1, 2]]] and dist.tolist() == [[[0.0, 1.0, 4.0]]]
    assert tpk.knn(support, query, 2)[0].tolist() == [[[0, 1]]]
    with pytest.raises(RuntimeError):
        tpk.knn(support, query, 5)
    assert tpk.knn(support.cpu(), query.cpu(), 2)[0].tolist() == [[[0, 1]]]  # CPU tensors: the host module
    # equal distances everywhere: tripled points, lattices, a collapsed cloud; small and large clouds
    g = torch.Generator().manual_seed(8)
    base = torch.rand(1, 400, 3, generator=g)
    tripled = torch.cat([base, base.flip(1), base], 1)[:, torch.randperm(1200, generator=g)]
    ax = torch.arange(10, dtype=torch.float32)
    lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3)
    big = torch.rand(1, 6000, 3, generator=g)
    big3 = torch.cat([big, big.flip(1), big], 1)[:, torch.randperm(18000, generator=g)]
    cases = [(tripled, torch.rand(1, 600, 3, generator=g), 7), (lattice, lattice + 0.5, 9), (lattice, lattice, 27),
             (torch.full((1, 600, 3), 0.5), torch.rand(1, 520, 3, generator=g), 40),
             (tripled[:, :300], base[:, :50], 10), (big3, big[:, :700], 5)]
    for support, query, k in cases:
        support, query = support.contiguous(), query.contiguous()
        idx, dist2 = tpk.knn(support.to(dev), query.to(dev), k)
        wi, wd = oracle.knn(support.numpy(), query.numpy(), k)
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist2), wd)


# ------------------------------------------------------------------ region growing


def _blobs(g, clouds, n, spread):
    """Packed clouds of blobs of different density plus scattered points, so that rows of the
    neighbour matrix are cut at nsample in places and clusters of all sizes appear."""
    pos, batch = [], []
    for c in range(clouds):
        centres = torch.rand(12, 3, generator=g)
        which = torch.randint(0, 12, (n,), generator=g)
        scale = spread * (0.3 + torch.rand(12, generator=g))[which].unsqueeze(-1)
        pts = centres[which] + scale * torch.randn(n, 3, generator=g)
        pts[: n // 8] = torch.rand(n // 8, 3, generator=g)
        pos.append(pts[torch.randperm(n, generator=g)])
        batch.append(torch.full((n,), c, dtype=torch.long))
    return torch.cat(pos).contiguous(), torch.cat(batch)


def test_kat_region_grow(tpk, dev):
    # reference test/test_cluster.py:14-44 (positions as floats)
    pos = torch.tensor([[0, 0, 0], [1, 0, 0], [2, 0, 0], [10, 0, 0]] * 2).float().to(dev)
    batch = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1]).to(dev)
    labels = torch.tensor([0, 0, 1, 1, 0, 1, 1, 10]).to(dev)
    from torch_points_kernels.cluster import grow_proximity, region_grow

    for order in ("reference", "index"):
        assert grow_proximity(pos, batch, radius=2, min_cluster_size=1, member_order=order) == [[0, 1, 2], [3], [4, 5, 6], [7]]
        assert grow_proximity(pos, batch, radius=2, min_cluster_size=3, member_order=order) == [[0, 1, 2], [4, 5, 6]]
        assert grow_proximity(pos, batch, radius=2, min_cluster_size=5, member_order=order) == []
        clusters = region_grow(pos, labels, batch, radius=2, min_cluster_size=1, member_order=order)
        assert [c.tolist() for c in clusters] == [[0, 1], [4], [2], [3], [5, 6], [7]]
        assert all(c.is_cuda and c.dtype == torch.int64 for c in clusters)
        clusters = region_grow(pos, labels, batch, ignore_labels=[1, 10], radius=2, min_cluster_size=1, member_order=order)
        assert [c.tolist() for c in clusters] == [[0, 1], [4]]
    assert grow_proximity(pos.cpu(), batch.cpu(), radius=2, min_cluster_size=1) == [[0, 1, 2], [3], [4, 5, 6], [7]]  # host module
    with pytest.raises(ValueError):
        grow_proximity(pos, batch, radius=2, member_order="sorted")


@pytest.mark.parametrize("clouds,n,spread,radius,nsample,min_size",
                         [(1, 300, 0.05, 0.05, 16, 1), (2, 2000, 0.03, 0.02, 16, 32), (3, 9000, 0.03, 0.03, 4, 8),
                          (1, 30000, 0.05, 0.02, 16, 32), (2, 12000, 0.02, 0.05, 70, 2), (1, 5000, 0.1, 0.004, 16, 1),
                          (1, 20000, 0.5, 0.03, 2, 3)])
def test_grow_proximity_parity(tpk, oracle, dev, clouds, n, spread, radius, nsample, min_size):
    from torch_points_kernels.cluster import grow_proximity

    g = torch.Generator().manual_seed(n + nsample)
    pos, batch = _blobs(g, clouds, n, spread)
    want = oracle.grow_proximity(pos.numpy(), batch.numpy(), nsample, radius, min_size)
    assert len(want) > 0
    got = grow_proximity(pos.to(dev), batch.to(dev), nsample, radius, min_size)
    assert got == want  # the reference's lists, member for member
    got = grow_proximity(pos.to(dev), batch.to(dev), nsample, radius, min_size, member_order="index")
    assert got == [sorted(c) for c in want]


def test_region_grow_parity(tpk, oracle, dev):
    from torch_points_kernels.cluster import region_grow

    g = torch.Generator().manual_seed(77)
    pos, batch = _blobs(g, 3, 6000, 0.03)
    labels = torch.randint(0, 4, (pos.shape[0] // 50,), generator=g).repeat_interleave(50) * 3 - 1  # runs of one label
    want = oracle.region_grow(pos.numpy(), labels.numpy(), batch.numpy(), ignore_labels=[2], radius=0.04, min_cluster_size=10)
    got = region_grow(pos.to(dev), labels.to(dev), batch.to(dev), ignore_labels=[2], radius=0.04, min_cluster_size=10)
    assert len(got) == len(want) > 0
    for a, b in zip(got, want):
        np.testing.assert_array_equal(_np(a), b)


def test_grow_proximity_any_matrix(tpk, oracle, dev):
    """Matrices that no ball query produces: rows ending early, entries after a -1 (ignored, the row has ended), chains
    in both directions, points nobody lists, no columns at all."""
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    g = torch.Generator().manual_seed(5)
    cases = []
    for n, ns in ((1, 1), (50, 3), (700, 5), (4000, 2), (3000, 80)):
        rows = torch.stack([torch.randperm(n, generator=g)[: min(ns, n)] for _ in range(n)])  # no repeats in a row
        if rows.shape[1] < ns:
            rows = torch.cat([rows, torch.full((n, ns - rows.shape[1]), -1)], 1)
        cut = torch.randint(0, ns + 1, (n,), generator=g)
        rows[torch.arange(ns).unsqueeze(0) == cut.unsqueeze(1)] = -1  # a -1 somewhere: the row ends there
        rows[torch.rand(n, generator=g) < 0.5, 0] = -1  # empty rows
        cases.append(rows)
    n = 5000
    up = torch.arange(1, n + 1).unsqueeze(1)
    up[-1] = -1
    cases.append(up)  # 0 -> 1 -> 2 ...: one cluster
    cases.append((torch.arange(n) - 1).unsqueeze(1))  # 1 -> 0, 2 -> 1, ...: nobody reaches a later point
    cases.append(torch.zeros(9, 0, dtype=torch.long))
    for rows in cases:
        rows = rows.contiguous()
        for min_size in (1, 2, 40):
            want = oracle.grow_proximity_core(rows.numpy(), min_size)
            for reference_order in (True, False):
                members, starts = native.grow_proximity(rows.to(dev), min_size, reference_order)
                members, starts = members.tolist(), starts.tolist()
                got = [members[a:b] for a, b in zip(starts[:-1], starts[1:])]
                assert got == (want if reference_order else [sorted(c) for c in want])


# ------------------------------------------------------------------ instance IoU


def test_kat_instance_iou(tpk, dev):
    # reference test/test_metrics.py:16-55
    from torch_points_kernels.metrics import instance_iou

    gt = torch.tensor([1, 2, 1, 2, 2, 3, 0]).to(dev)
    ious = instance_iou([torch.tensor([0, 2]).to(dev), torch.tensor([1, 4]).to(dev), torch.tensor([3, 5]).to(dev)], gt)
    torch.testing.assert_close(ious.cpu(), torch.tensor([[1, 0, 0], [0, 2 / 3.0, 0], [0, 1.0 / 4.0, 1.0 / 2.0]]), rtol=1e-4, atol=1e-5)
    batch = torch.tensor([0, 0, 1, 1, 1, 1, 1]).to(dev)
    ious = instance_iou([torch.tensor([0, 1]).to(dev), torch.tensor([3, 4]).to(dev), torch.tensor([5]).to(dev)], gt, batch=batch)
    want = torch.tensor([[0.5, 0.5, 0, 0, 0], [0, 0, 0, 1, 0], [0, 0, 0, 0, 1.0]])
    torch.testing.assert_close(ious.cpu(), want, rtol=1e-4, atol=1e-5)
    host_ious = instance_iou([torch.tensor([0, 2])], gt.cpu())  # CPU tensors: the host module
    assert host_ious.tolist() == [[1.0, 0.0, 0.0]] and not host_ious.is_cuda


@pytest.mark.parametrize("samples,points,instances,proposals,longest", [(1, 1000, 9, 20, 50), (3, 5000, 40, 300, 700),
                                                                         (2, 30000, 300, 64, 9000), (1, 20000, 9000, 5, 4000)])
def test_instance_iou_parity(tpk, oracle, dev, samples, points, instances, proposals, longest):
    # the last case has more instances in a sample than the kernel counts in LDS
    from torch_points_kernels.metrics import instance_iou

    g = torch.Generator().manual_seed(points + proposals)
    batch = torch.sort(torch.randint(0, samples, (points,), generator=g))[0]
    batch[0], batch[-1] = 0, samples - 1
    gt = torch.randint(0, instances + 1, (points,), generator=g)
    gt[torch.rand(points, generator=g) < 0.1] = -100  # the ignore label of the segmentation data sets
    for s in range(samples):
        gt[(batch == s).nonzero()[0]] = instances  # every sample has its last instance
    props = []
    for p in range(proposals):
        size = int(torch.randint(1, longest + 1, (1,), generator=g))
        sample = int(torch.randint(0, samples, (1,), generator=g))
        members = (batch == sample).nonzero().flatten()
        props.append(members[torch.randint(0, members.numel(), (size,), generator=g)])  # repeats allowed
    got = instance_iou([p.to(dev) for p in props], gt.to(dev), batch.to(dev))
    want = oracle.instance_iou([p.numpy() for p in props], gt.numpy(), batch.numpy())
    assert got.dtype == torch.float32 and got.shape == want.shape
    np.testing.assert_array_equal(_np(got), want)  # integer counts and one correctly rounded quotient: bit-exact
    assert (want > 0).any()


# ------------------------------------------------------------------ gridding, cubic feature sampling


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("B,n,scale", [(1, 32, 4), (2, 2048, 32), (3, 700, 8), (1, 1, 2)])
def test_gridding_parity(tpk, oracle, dev, dtype, B, n, scale):
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    g = torch.Generator().manual_seed(n + scale)
    p = ((torch.rand(B, n, 3, generator=g, dtype=torch.float64) * 2 - 1) * scale).to(dtype)  # the last cell's outer vertices fall outside
    p[0, 0] = torch.tensor([1.0, -2.0, 0.0], dtype=dtype)  # integral coordinates
    grid, weights, indexes = native.gridding(-scale, scale - 1, -scale, scale - 1, -scale, scale - 1, p.to(dev))
    wg, ww, wi = oracle.gridding(p.numpy(), scale)
    assert grid.dtype == dtype and indexes.dtype == torch.int32
    np.testing.assert_array_equal(_np(indexes), wi)
    np.testing.assert_array_equal(_np(weights), ww)
    # the grid is a sum in no fixed order (atomics, as in the reference)
    np.testing.assert_allclose(_np(grid), wg, rtol=1e-5 if dtype == torch.float32 else 1e-12, atol=1e-5 if dtype == torch.float32 else 1e-12)
    r = torch.randn(B, (2 * scale) ** 3, generator=g, dtype=torch.float64).to(dtype)
    grad = native.gridding_grad(weights, indexes, r.to(dev))
    np.testing.assert_array_equal(_np(grad), oracle.gridding_grad(ww, wi, r.numpy()))  # one thread's sum in the reference's order


def test_gridding_front_end_and_gradcheck(tpk, oracle, dev):
    from torch_points_kernels.gridding import GriddingFunction, gridding

    # reference test/test_gridding.py:19-29
    # (seeded, and no coordinate within 1e-3 of a grid plane: the finite differences of gradcheck must not
    # step across one, where the weights have a kink)
    g = torch.Generator().manual_seed(31)
    for n, scale in ((32, 4), (64, 8)):
        x = torch.rand(1, n, 3, dtype=torch.float64, generator=g)
        x = torch.where((x - x.round()).abs() < 1e-3, x + 0.01, x).to(dev).requires_grad_()
        assert torch.autograd.gradcheck(GriddingFunction.apply, [x, scale])
    # the front end (gridding.py:34-60): scaled by `scale`, points whose coordinates sum to zero dropped per cloud
    g = torch.Generator().manual_seed(3)
    p = torch.rand(2, 100, 3, generator=g) * 1.8 - 0.9
    p[1, 10:30] = 0
    got = gridding(p.to(dev), 8)
    assert got.shape == (2, 16 ** 3)
    for b in range(2):
        kept = (p[b] * 8)[(p[b] * 8).sum(1) != 0].unsqueeze(0)
        np.testing.assert_allclose(_np(got[b : b + 1]), oracle.gridding(kept.numpy(), 8)[0], rtol=1e-5, atol=1e-5)
    with pytest.raises(ValueError):
        gridding(p[0].to(dev), 8)
    with pytest.raises(NotImplementedError):
        gridding(p, 8)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("B,n,c,scale,ns", [(2, 64, 4, 8, 1), (2, 32, 2, 8, 2), (1, 32, 2, 16, 3), (2, 2048, 64, 16, 1), (1, 300, 7, 4, 2)])
def test_cubic_feature_sampling_parity(tpk, oracle, dev, dtype, B, n, c, scale, ns):
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    g = torch.Generator().manual_seed(n + c + ns)
    p = (torch.rand(B, n, 3, generator=g, dtype=torch.float64) * (scale + 2) - 1).to(dtype)  # some points outside the grid
    p[0, 0] = torch.tensor([2.0, 3.0, 0.0], dtype=dtype)
    feats = torch.rand(B, c, scale, scale, scale, generator=g, dtype=torch.float64).to(dtype)
    out, indexes = native.cubic_feature_sampling(scale, ns, p.to(dev), feats.to(dev))
    wo, wi = oracle.cubic_feature_sampling(p.numpy(), feats.numpy(), ns)
    np.testing.assert_array_equal(_np(indexes), wi)
    np.testing.assert_array_equal(_np(out), wo)
    go = torch.randn(out.shape, generator=g, dtype=torch.float64).to(dtype)
    grad_p, grad_f = native.cubic_feature_sampling_grad(scale, ns, go.to(dev), indexes)
    wp, wf = oracle.cubic_feature_sampling_grad(scale, ns, go.numpy(), wi)
    assert (_np(grad_p) == 0).all() and grad_f.shape == feats.shape
    tol = 1e-4 if dtype == torch.float32 else 1e-11  # sums of up to n * n_vertices terms in no fixed order
    np.testing.assert_allclose(_np(grad_f), wf, rtol=tol, atol=tol)


def test_cubic_feature_sampling_front_end_and_gradcheck(tpk, oracle, dev):
    from torch_points_kernels.cubic_feature_sampling import CubicFeatureSamplingFunction, cubic_feature_sampling

    # reference test/test_cubic_feature_sampling.py:20-56
    # (seeded, and no coordinate within 1e-3 of a grid plane: a finite difference stepping across one changes
    # the sampled vertices, which the analytical gradient - zero in the coordinates - does not follow)
    gen = torch.Generator().manual_seed(32)
    for B, n, c, scale, ns in ((2, 64, 4, 8, 1), (2, 32, 2, 8, 2), (1, 32, 2, 16, 3)):
        p = torch.rand(B, n, 3, dtype=torch.float64, generator=gen) * 2 - 1
        p = torch.where((p - p.round()).abs() < 1e-3, p + 0.01, p).to(dev).requires_grad_()
        feats = torch.rand(B, c, scale, scale, scale, dtype=torch.float64, generator=gen).to(dev).requires_grad_()
        assert torch.autograd.gradcheck(CubicFeatureSamplingFunction.apply, [p, feats, ns])
    # front end (cubic_feature_sampling.py:34-59): coordinates in [-1, 1) mapped to grid units
    g = torch.Generator().manual_seed(4)
    p = torch.rand(2, 50, 3, generator=g) * 2 - 1
    feats = torch.rand(2, 3, 8, 8, 8, generator=g)
    got = cubic_feature_sampling(p.to(dev), feats.to(dev), 2)
    np.testing.assert_array_equal(_np(got), oracle.cubic_feature_sampling((p * 4.0 + 4.0).numpy(), feats.numpy(), 2)[0])
    with pytest.raises(ValueError):
        cubic_feature_sampling(p[0].to(dev), feats.to(dev))


# ------------------------------------------------------------------ committed reference vectors


def test_hip_path_against_committed_reference_vectors(tpk, dev):
    """The reference's own CPU module computed these outputs (tests/golden/make_vectors.py); the HIP path must
    reproduce them bit for bit - no oracle in between."""
    import os

    v = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_cpu_vectors.npz"))
    t = lambda name: torch.from_numpy(v[name]).to(dev)
    idx, dist2 = tpk.knn(t("knn_support"), t("knn_query"), 9)
    np.testing.assert_array_equal(_np(idx), v["knn_idx"])
    np.testing.assert_array_equal(_np(dist2), v["knn_dist2"])
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    dist3, idx3 = native.three_nn(t("knn_query"), t("knn_support"))  # squared distances (the Python layer returns their roots)
    np.testing.assert_array_equal(_np(idx3), v["three_nn_idx"])
    np.testing.assert_array_equal(_np(dist3), v["three_nn_dist2"])
    idx, dist = tpk.ball_query(float(v["ball_sorted_radius"]), 12, t("knn_support"), t("knn_query"), sort=True)
    np.testing.assert_array_equal(_np(idx), v["ball_sorted_idx"])
    np.testing.assert_array_equal(_np(dist), v["ball_sorted_dist"])
    idx, dist = tpk.ball_query(float(v["packed_radius"]), 10, t("packed_x"), t("packed_y"), mode="partial_dense",
                               batch_x=t("packed_batch_x"), batch_y=t("packed_batch_y"), sort=True)
    np.testing.assert_array_equal(_np(idx), v["packed_sorted_idx"])
    np.testing.assert_array_equal(_np(dist), v["packed_sorted_dist"])
    np.testing.assert_array_equal(_np(tpk.furthest_point_sample(t("fps_xyz"), 64)), v["fps_idx"])
    out = tpk.three_interpolate(t("interp_features"), t("interp_idx").int(), t("interp_weight"))
    np.testing.assert_array_equal(_np(out), v["interp_out"])


# ------------------------------------------------------------------ chamfer


@pytest.mark.parametrize("B,n,m", [(1, 3, 2), (2, 300, 515), (2, 1030, 700), (3, 64, 1), (1, 2500, 2047), (2, 1, 9)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_chamfer_parity(tpk, oracle, dev, B, n, m, dtype):
    g = torch.Generator().manual_seed(n + 3 * m)
    a = torch.rand(B, n, 3, generator=g, dtype=dtype)
    b = torch.rand(B, m, 3, generator=g, dtype=dtype)
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    d1, d2, i1, i2 = native.chamfer_dist(a.to(dev), b.to(dev))
    w1, w2, wi1, wi2 = oracle.chamfer_fwd(a.numpy(), b.numpy())
    assert i1.dtype == torch.int32 and d1.dtype == dtype
    np.testing.assert_array_equal(_np(i1), wi1)
    np.testing.assert_array_equal(_np(i2), wi2)
    np.testing.assert_array_equal(_np(d1), w1)
    np.testing.assert_array_equal(_np(d2), w2)
    g1 = torch.randn(B, n, generator=g, dtype=dtype)
    g2 = torch.randn(B, m, generator=g, dtype=dtype)
    ga, gb = native.chamfer_dist_grad(a.to(dev), b.to(dev), i1, i2, g1.to(dev), g2.to(dev))
    wa, wb = oracle.chamfer_bwd(a.numpy(), b.numpy(), wi1, wi2, g1.numpy(), g2.numpy())
    np.testing.assert_allclose(_np(ga), wa, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(_np(gb), wb, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_chamfer_backward_skewed_indices(tpk, dev, dtype):
    # The backward pass keeps, per range of points, the other cloud's points that chose one of them in LDS, with
    # room for the share of the other cloud a range expects and a third more.  Here every point of the second cloud
    # names one of the first 900 points of the first (some of them hundreds of times), so one range meets all 16384
    # and takes the chains of point numbers instead; the first cloud's indices are uniform (entries in LDS); the
    # second pair has them the other way round.  Checked against sums formed in float64, to the stated tolerance
    # plus the reordering allowance.
    B, n, m = 2, 16384, 16384
    g = torch.Generator().manual_seed(9)
    a, b = torch.rand(B, n, 3, generator=g, dtype=dtype), torch.rand(B, m, 3, generator=g, dtype=dtype)
    i1 = torch.randint(0, m, (B, n), generator=g, dtype=torch.int32)
    i2 = (torch.rand(B, m, generator=g) ** 3 * 900).to(torch.int32)
    i1[1], i2[1] = (torch.rand(n, generator=g) ** 3 * 900).to(torch.int32), torch.randint(0, n, (m,), generator=g, dtype=torch.int32)
    g1, g2 = torch.randn(B, n, generator=g, dtype=dtype), torch.randn(B, m, generator=g, dtype=dtype)
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    ga, gb = native.chamfer_dist_grad(a.to(dev), b.to(dev), i1.to(dev), i2.to(dev), g1.to(dev), g2.to(dev))
    an, bn, g1n, g2n = (t.numpy().astype(np.float64) for t in (a, b, g1, g2))
    wa, wb, ma, mb = (np.zeros((B, k, 3)) for k in (n, m, n, m))
    for c in range(B):
        j1, j2 = i1[c].numpy().astype(np.int64), i2[c].numpy().astype(np.int64)
        t1 = 2 * g1n[c][:, None] * (an[c] - bn[c][j1])  # d dist1[i] / d xyz1[i]; its negative goes to xyz2[j1[i]]
        t2 = 2 * g2n[c][:, None] * (bn[c] - an[c][j2])
        wa[c] += t1
        wb[c] += t2
        np.add.at(wb[c], j1, -t1)
        np.add.at(wa[c], j2, -t2)
        ma[c] += np.abs(t1)
        mb[c] += np.abs(t2)
        np.add.at(mb[c], j1, np.abs(t1))
        np.add.at(ma[c], j2, np.abs(t2))
    if dtype == torch.float64:
        np.testing.assert_allclose(_np(ga), wa, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(_np(gb), wb, rtol=1e-12, atol=1e-12)
    else:
        _assert_scatter_sum_close(_np(ga), wa.astype(np.float32), ma.astype(np.float32), "chamfer backward, skewed indices, xyz1")
        _assert_scatter_sum_close(_np(gb), wb.astype(np.float32), mb.astype(np.float32), "chamfer backward, skewed indices, xyz2")


def test_chamfer_ties_take_lowest_index(tpk, oracle, dev):
    a = torch.zeros(1, 300, 3)
    b = torch.full((1, 3000, 3), 5.0)
    b[0, [3, 4, 600, 1100, 2999], 0] = 1.0
    b[0, [3, 4, 600, 1100, 2999], 1:] = 0.0
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    d1, d2, i1, i2 = native.chamfer_dist(a.to(dev), b.to(dev))
    w1, w2, wi1, wi2 = oracle.chamfer_fwd(a.numpy(), b.numpy())
    assert (i1 == 3).all()
    np.testing.assert_array_equal(_np(i1), wi1)
    np.testing.assert_array_equal(_np(i2), wi2)  # every b point ties over all of a: index 0
    np.testing.assert_array_equal(_np(d2), w2)


@pytest.mark.parametrize("B,n,m", [(2, 512, 512), (3, 1000, 777), (2, 4099, 513), (1, 16384, 16384), (2, 9000, 16000),
                                   (2, 20000, 700), (1, 16385, 40001)])
def test_chamfer_cell_search_parity(tpk, oracle, dev, B, n, m):
    # cloud sizes served by the search over curve-ordered cells (float32, 512..16384 points)
    from torch_points_kernels._native import native
    g = torch.Generator().manual_seed(n + m)
    for a, b in ((torch.rand(B, n, 3, generator=g), torch.rand(B, m, 3, generator=g)),
                 (_clustered(g, B, n), _clustered(g, B, m))):
        d1, d2, i1, i2 = native().chamfer_dist(a.to(dev), b.to(dev))
        w1, w2, wi1, wi2 = oracle.chamfer_fwd(a.numpy(), b.numpy())
        np.testing.assert_array_equal(_np(i1), wi1)
        np.testing.assert_array_equal(_np(i2), wi2)
        np.testing.assert_array_equal(_np(d1), w1)
        np.testing.assert_array_equal(_np(d2), w2)


def test_chamfer_cell_search_ties(tpk, oracle, dev):
    # equal distances everywhere: lattices against shifted lattices, every point duplicated,
    # identical clouds, one cloud collapsed to a single location
    from torch_points_kernels._native import native
    g = torch.Generator().manual_seed(3)
    ax = torch.arange(10, dtype=torch.float32)
    lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3)
    shifted = lattice + torch.tensor([0.5, 0.5, 0.0])
    base = torch.rand(1, 700, 3, generator=g)
    doubled = torch.cat([base, base, base.flip(1)], 1)[:, torch.randperm(2100, generator=g)]
    collapsed = torch.full((1, 600, 3), 0.25)
    cases = [(lattice, shifted[:, torch.randperm(1000, generator=g)]),
             (lattice[:, torch.randperm(1000, generator=g)], lattice),
             (doubled, base[:, :640]), (doubled, doubled.flip(1)), (base, collapsed), (collapsed, collapsed)]
    # above 16384 points (clouds ordered in several windows): every point three times, a large lattice
    base = torch.rand(1, 6000, 3, generator=g)
    tripled = torch.cat([base, base, base.flip(1)], 1)[:, torch.randperm(18000, generator=g)]
    ax = torch.arange(27, dtype=torch.float32)
    big_lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3)
    cases += [(tripled, base[:, :5000]), (big_lattice, big_lattice[:, torch.randperm(19683, generator=g)] + 0.5)]
    for a, b in cases:
        a, b = a.contiguous(), b.contiguous()
        d1, d2, i1, i2 = native().chamfer_dist(a.to(dev), b.to(dev))
        w1, w2, wi1, wi2 = oracle.chamfer_fwd(a.numpy(), b.numpy())
        np.testing.assert_array_equal(_np(i1), wi1)
        np.testing.assert_array_equal(_np(i2), wi2)
        np.testing.assert_array_equal(_np(d1), w1)
        np.testing.assert_array_equal(_np(d2), w2)


def test_cell_search_outliers(tpk, oracle, dev):
    # A few far outliers in every group of 64 queries: the cells they keep admitting are served one query at a
    # time (candidates side by side in the lanes) - also where those candidates are duplicated points or a
    # lattice, so that equal distances meet on that path.
    from torch_points_kernels._native import native
    g = torch.Generator().manual_seed(11)
    def with_outliers(cloud, share, spread):
        cloud = cloud.clone()
        pick = torch.rand(cloud.shape[:2], generator=g) < share
        cloud[pick] += spread * torch.randn(int(pick.sum()), 3, generator=g)
        return cloud
    sphere = torch.nn.functional.normalize(torch.randn(2, 6000, 3, generator=g), dim=2)
    base = torch.rand(1, 1500, 3, generator=g)
    doubled = torch.cat([base, base, base.flip(1)], 1)[:, torch.randperm(4500, generator=g)]
    ax = torch.arange(12, dtype=torch.float32) / 12
    lattice = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3)
    cases = [(with_outliers(sphere, 0.05, 0.3), sphere.flip(1)),
             (with_outliers(torch.rand(1, 3000, 3, generator=g), 0.03, 2.0), doubled),
             (with_outliers(lattice, 0.04, 1.5), lattice[:, torch.randperm(1728, generator=g)]),
             (with_outliers(torch.rand(1, 20000, 3, generator=g), 0.02, 1.0), torch.rand(1, 18000, 3, generator=g))]
    for a, b in cases:
        a, b = a.contiguous(), b.contiguous()
        d1, d2, i1, i2 = native().chamfer_dist(a.to(dev), b.to(dev))
        w1, w2, wi1, wi2 = oracle.chamfer_fwd(a.numpy(), b.numpy())
        np.testing.assert_array_equal(_np(i1), wi1)
        np.testing.assert_array_equal(_np(i2), wi2)
        np.testing.assert_array_equal(_np(d1), w1)
        np.testing.assert_array_equal(_np(d2), w2)
        dist2, idx = native().three_nn(a.to(dev), b.to(dev))
        wd, wi = oracle.three_nn(a.numpy(), b.numpy())
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist2), wd)


def test_chamfer_gradcheck_double(tpk, dev):
    # reference test/test_chamfer_dist.py:20-25
    from torch.autograd import gradcheck
    from torch_points_kernels.chamfer_dist import ChamferFunction

    g = torch.Generator().manual_seed(1)
    x = torch.rand(4, 64, 3, generator=g).double().to(dev).requires_grad_(True)
    y = torch.rand(4, 128, 3, generator=g).double().to(dev).requires_grad_(True)
    assert gradcheck(ChamferFunction.apply, [x, y])


def test_chamfer_full_config5(tpk, oracle, dev):
    w = W.cfg5_chamfer()
    a, b = w["xyz1"].to(dev), w["xyz2"].to(dev)
    native = __import__("torch_points_kernels._native", fromlist=["native"]).native()
    d1, d2, i1, i2 = native.chamfer_dist(a, b)
    # (1) stored distance == distance to the reported neighbour, recomputed with separately
    #     rounded torch ops in the reference's operand order
    for da, ia, p, q in ((d1, i1, a, b), (d2, i2, b, a)):
        near = torch.gather(q, 1, ia.long().unsqueeze(-1).expand(-1, -1, 3))
        diff = near - p
        rec = diff[..., 0] * diff[..., 0] + diff[..., 1] * diff[..., 1] + diff[..., 2] * diff[..., 2]
        assert (rec == da).all()
    # (2) bit-exact against the oracle for EVERY point of every cloud, both directions (17.2 G pairs of
    #     brute force, one cloud pair per task over the host's threads)
    an, bn = w["xyz1"].numpy(), w["xyz2"].numpy()
    parts = _in_threads(lambda c: oracle.chamfer_fwd(an[c:c + 1], bn[c:c + 1]), range(an.shape[0]))
    np.testing.assert_array_equal(_np(d1), np.concatenate([p[0] for p in parts]))
    np.testing.assert_array_equal(_np(d2), np.concatenate([p[1] for p in parts]))
    np.testing.assert_array_equal(_np(i1), np.concatenate([p[2] for p in parts]))
    np.testing.assert_array_equal(_np(i2), np.concatenate([p[3] for p in parts]))
    # (3) backward against the oracle on the full size (linear in the number of points)
    ga, gb = native.chamfer_dist_grad(a, b, i1, i2, w["grad_dist1"].to(dev), w["grad_dist2"].to(dev))
    wa, wb = oracle.chamfer_bwd(w["xyz1"].numpy(), w["xyz2"].numpy(), _np(i1), _np(i2),
                                w["grad_dist1"].numpy(), w["grad_dist2"].numpy())
    np.testing.assert_allclose(_np(ga), wa, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(_np(gb), wb, rtol=RTOL, atol=ATOL)
    # (4) determinism of the integer outputs
    _, _, j1, j2 = native.chamfer_dist(a, b)
    assert (j1 == i1).all() and (j2 == i2).all()


# ------------------------------------------------------------------ the C ABI called directly


def test_gridding_last_cell_matches_the_reference_formula_inside_the_grid(tpk, dev):
    """Vertices inside the grid carry the index and weight of the reference's formula (gridding_gpu.cu:17-20, 43-131);
    the vertices of a point in the last cell that lie outside get -1 and deposit nothing, where the reference adds
    their weight to a wrapped cell (y, z) or beyond the cloud's grid (x)."""
    from tests.test_oracle_pinning import check_last_cell_behaviour
    from torch_points_kernels._native import native

    def gridding(points, scale):
        g, w, i = native().gridding(-scale, scale - 1, -scale, scale - 1, -scale, scale - 1, torch.from_numpy(points).to(dev))
        return _np(g), _np(w), _np(i)

    check_last_cell_behaviour(gridding)


def test_c_abi_direct_call(oracle, dev):
    """libtpk_hip.so used without the extension: ctypes + raw device pointers + a stream."""
    import ctypes
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = ctypes.CDLL(os.path.join(root, "torch-points-kernels_amd", "torch_points_kernels", "libtpk_hip.so"))
    g = torch.Generator().manual_seed(2)
    unknown = torch.rand(2, 700, 3, generator=g)
    known = torch.rand(2, 900, 3, generator=g)
    u, k = unknown.to(dev), known.to(dev)
    dist2 = torch.empty(2, 700, 3, device=dev)
    idx = torch.empty(2, 700, 3, dtype=torch.int32, device=dev)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    wd, wi = oracle.three_nn(unknown.numpy(), known.numpy())
    lib.tpk_three_nn_workspace_bytes.restype = ctypes.c_size_t
    ws_bytes = lib.tpk_three_nn_workspace_bytes(2, 700, 900)
    assert ws_bytes > 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    # without workspace (all pairs), then with it (search over cells): same answers
    for ws_ptr, nbytes in ((None, 0), (ctypes.c_void_p(ws.data_ptr()), ws_bytes)):
        dist2.fill_(-1.0)
        idx.fill_(-1)
        stream.wait_stream(torch.cuda.current_stream())
        st = lib.tpk_three_nn_f32(2, 700, 900, ctypes.c_void_p(u.data_ptr()), ctypes.c_void_p(k.data_ptr()),
                                  ctypes.c_void_p(dist2.data_ptr()), ctypes.c_void_p(idx.data_ptr()),
                                  ws_ptr, ctypes.c_size_t(nbytes), ctypes.c_void_p(stream.cuda_stream))
        assert st == 0
        stream.synchronize()
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist2), wd)
    # the scan of all pairs by name
    dist2.fill_(-1.0)
    idx.fill_(-1)
    stream.wait_stream(torch.cuda.current_stream())
    st = lib.tpk_three_nn_all_pairs_f32(2, 700, 900, ctypes.c_void_p(u.data_ptr()), ctypes.c_void_p(k.data_ptr()),
                                        ctypes.c_void_p(dist2.data_ptr()), ctypes.c_void_p(idx.data_ptr()),
                                        ctypes.c_void_p(stream.cuda_stream))
    assert st == 0
    stream.synchronize()
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist2), wd)
    # a workspace that is too small is refused before any launch
    st = lib.tpk_three_nn_f32(2, 700, 900, ctypes.c_void_p(u.data_ptr()), ctypes.c_void_p(k.data_ptr()),
                              ctypes.c_void_p(dist2.data_ptr()), ctypes.c_void_p(idx.data_ptr()),
                              ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(1024), ctypes.c_void_p(stream.cuda_stream))
    assert st == -3
    # an undersized FPS workspace is refused before any launch
    pts = torch.rand(1, 20000, 3).to(dev)
    out = torch.empty(1, 4, dtype=torch.int32, device=dev)
    st = lib.tpk_fps_f32(1, 20000, 4, ctypes.c_void_p(pts.data_ptr()), None, ctypes.c_size_t(0),
                         ctypes.c_void_p(out.data_ptr()), None)
    assert st == -3


def test_c_abi_direct_call_every_family(oracle, dev):
    """One call per family of entry points through ctypes (no extension in between): furthest point sampling, ball query
    in both layouts with and without workspace, the gathers forward and backward, Chamfer forward and backward -
    compared with the checker like the calls through the Python layer."""
    import ctypes
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = ctypes.CDLL(os.path.join(root, "torch-points-kernels_amd", "torch_points_kernels", "libtpk_hip.so"))
    for name in ("tpk_fps_workspace_bytes", "tpk_ball_query_partial_workspace_bytes", "tpk_three_interpolate_grad_workspace_bytes",
                 "tpk_group_grad_workspace_bytes", "tpk_chamfer_fwd_workspace_bytes"):
        getattr(lib, name).restype = ctypes.c_size_t
    lib.tpk_ball_query_partial_workspace_bytes.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    F = ctypes.c_float
    Z = ctypes.c_size_t
    L = ctypes.c_int64
    stream = torch.cuda.Stream()
    S = ctypes.c_void_p(stream.cuda_stream)
    g = torch.Generator().manual_seed(31)

    def workspace(nbytes):
        return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=dev)

    def run(call):
        stream.wait_stream(torch.cuda.current_stream())
        assert call() == 0
        stream.synchronize()

    # furthest point sampling: a cloud held in registers, and one that needs the workspace
    for n, npoint in ((3000, 100), (20000, 40)):
        xyz = torch.rand(2, n, 3, generator=g) + 0.2
        d = xyz.to(dev)
        out = torch.full((2, npoint), -1, dtype=torch.int32, device=dev)
        nbytes = lib.tpk_fps_workspace_bytes(2, n)
        ws = workspace(nbytes)
        run(lambda: lib.tpk_fps_f32(2, n, npoint, P(d), P(ws) if nbytes else None, Z(nbytes), P(out), S))
        np.testing.assert_array_equal(_np(out), oracle.furthest_point_sample(xyz.numpy(), npoint))

    # ball query, dense layout
    xyz, centres = torch.rand(2, 2500, 3, generator=g), torch.rand(2, 300, 3, generator=g)
    dx, dc = xyz.to(dev), centres.to(dev)
    idx = torch.full((2, 300, 12), -7, dtype=torch.int64, device=dev)
    dist = torch.full((2, 300, 12), -7.0, device=dev)
    run(lambda: lib.tpk_ball_query_dense_f32(2, 2500, 300, F(0.12), 12, P(dc), P(dx), P(idx), P(dist), S))
    wi, wd = oracle.ball_query_dense(0.12, 12, xyz.numpy(), centres.numpy())
    np.testing.assert_array_equal(_np(idx), wi)
    np.testing.assert_array_equal(_np(dist), wd)

    # ball query, packed layout: all pairs (no workspace) and the walk over bins (workspace)
    sizes = [9000, 400, 12000]
    x = torch.rand(sum(sizes), 3, generator=g)
    bx = torch.repeat_interleave(torch.arange(3), torch.tensor(sizes))
    pick = torch.sort(torch.randperm(sum(sizes), generator=g)[:5000])[0]
    y, by = x[pick].contiguous(), bx[pick].contiguous()
    dxp, dyp, dbx, dby = x.to(dev), y.to(dev), bx.to(dev), by.to(dev)
    wi, wd = oracle.ball_query_partial_dense(0.05, 16, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
    nbytes = lib.tpk_ball_query_partial_workspace_bytes(L(x.shape[0]), L(y.shape[0]), 16)
    assert nbytes > 0
    ws = workspace(nbytes)
    for ws_ptr, ws_bytes in ((None, 0), (P(ws), nbytes)):
        idx = torch.full((y.shape[0], 16), -7, dtype=torch.int64, device=dev)
        dist = torch.full((y.shape[0], 16), -7.0, device=dev)
        run(lambda: lib.tpk_ball_query_partial_f32(L(x.shape[0]), L(y.shape[0]), F(0.05), 16, P(dxp), P(dyp), P(dbx), P(dby),
                                                   P(idx), P(dist), ws_ptr, Z(ws_bytes), S))
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist), wd)

    # three_interpolate forward and backward (lists in the workspace, then global atomics without it)
    b, c, m, n = 2, 9, 700, 5000
    feats = torch.randn(b, c, m, generator=g)
    nn = torch.randint(0, m, (b, n, 3), generator=g).int()
    w = torch.rand(b, n, 3, generator=g)
    gout = torch.randn(b, c, n, generator=g)
    df, dn, dw, dg = feats.to(dev), nn.to(dev), w.to(dev), gout.to(dev)
    out = torch.empty(b, c, n, device=dev)
    run(lambda: lib.tpk_three_interpolate_f32(b, c, m, n, P(df), P(dn), P(dw), P(out), S))
    np.testing.assert_array_equal(_np(out), oracle.three_interpolate(feats.numpy(), nn.numpy(), w.numpy()))
    want = oracle.three_interpolate_grad(gout.numpy(), nn.numpy(), w.numpy(), m)
    abs_sum = oracle.three_interpolate_grad(gout.abs().numpy(), nn.numpy(), w.numpy(), m)
    nbytes = lib.tpk_three_interpolate_grad_workspace_bytes(b, n, m)
    assert nbytes > 0
    ws = workspace(nbytes)
    for ws_ptr, ws_bytes in ((P(ws), nbytes), (None, 0)):
        grad = torch.full((b, c, m), 7.0, device=dev)
        run(lambda: lib.tpk_three_interpolate_grad_f32(b, c, n, m, P(dg), P(dn), P(dw), P(grad), ws_ptr, Z(ws_bytes), S))
        _assert_scatter_sum_close(_np(grad), want, abs_sum)

    # grouping forward and backward
    b, c, n, npoint, nsample = 2, 6, 900, 300, 8
    feats = torch.randn(b, c, n, generator=g)
    gi = torch.randint(0, n, (b, npoint, nsample), generator=g)
    gout = torch.randn(b, c, npoint, nsample, generator=g)
    df, di, dg = feats.to(dev), gi.to(dev), gout.to(dev)
    out = torch.empty(b, c, npoint, nsample, device=dev)
    run(lambda: lib.tpk_group_f32(b, c, n, npoint, nsample, P(df), P(di), P(out), S))
    np.testing.assert_array_equal(_np(out), oracle.grouping_operation(feats.numpy(), gi.numpy()))
    nbytes = lib.tpk_group_grad_workspace_bytes(b, n, npoint, nsample)
    ws = workspace(nbytes)
    grad = torch.full((b, c, n), 7.0, device=dev)
    run(lambda: lib.tpk_group_grad_f32(b, c, n, npoint, nsample, P(dg), P(di), P(grad), P(ws), Z(nbytes), S))
    _assert_scatter_sum_close(_np(grad), oracle.grouping_operation_grad(gout.numpy(), gi.numpy(), n),
                              oracle.grouping_operation_grad(gout.abs().numpy(), gi.numpy(), n))

    # Chamfer forward (all pairs, then the cell search) and backward
    b, n, m = 2, 3000, 2100
    a, c2 = torch.rand(b, n, 3, generator=g), torch.rand(b, m, 3, generator=g)
    da, dc2 = a.to(dev), c2.to(dev)
    w1, w2, wi1, wi2 = oracle.chamfer_fwd(a.numpy(), c2.numpy())
    nbytes = lib.tpk_chamfer_fwd_workspace_bytes(b, n, m)
    assert nbytes > 0
    ws = workspace(nbytes)
    for ws_ptr, ws_bytes in ((None, 0), (P(ws), nbytes)):
        d1, d2 = torch.empty(b, n, device=dev), torch.empty(b, m, device=dev)
        i1 = torch.empty(b, n, dtype=torch.int32, device=dev)
        i2 = torch.empty(b, m, dtype=torch.int32, device=dev)
        run(lambda: lib.tpk_chamfer_fwd_f32(b, n, m, P(da), P(dc2), P(d1), P(d2), P(i1), P(i2), ws_ptr, Z(ws_bytes), S))
        for got, want in ((d1, w1), (d2, w2), (i1, wi1), (i2, wi2)):
            np.testing.assert_array_equal(_np(got), want)
    g1, g2 = torch.randn(b, n, generator=g), torch.randn(b, m, generator=g)
    dg1, dg2 = g1.to(dev), g2.to(dev)
    ga, gb = torch.full((b, n, 3), 7.0, device=dev), torch.full((b, m, 3), 7.0, device=dev)
    run(lambda: lib.tpk_chamfer_bwd_f32(b, n, m, P(da), P(dc2), P(i1), P(i2), P(dg1), P(dg2), P(ga), P(gb), None, Z(0), S))
    wa, wb = oracle.chamfer_bwd(a.numpy(), c2.numpy(), wi1, wi2, g1.numpy(), g2.numpy())
    np.testing.assert_allclose(_np(ga), wa, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(_np(gb), wb, rtol=RTOL, atol=ATOL)


def test_counting_build_counts_executed_pairs(oracle, dev):
    """The counting build of the library returns the same results and counts the pair evaluations its lanes
    execute: a brute-force three_nn of 256 queries against 100 points = 256 lanes x 100 candidates; the search
    over cells of the same clouds executes fewer than all pairs and still answers identically."""
    import ctypes
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = ctypes.CDLL(os.path.join(root, "torch-points-kernels_amd", "torch_points_kernels", "libtpk_hip_counting.so"))
    lib.tpk_three_nn_workspace_bytes.restype = ctypes.c_size_t
    count = ctypes.c_ulonglong(0)

    def run(b, n, m, with_workspace):
        g = torch.Generator().manual_seed(5)
        unknown, known = torch.rand(b, n, 3, generator=g), torch.rand(b, m, 3, generator=g)
        u, k = unknown.to(dev), known.to(dev)
        dist2 = torch.empty(b, n, 3, device=dev)
        idx = torch.empty(b, n, 3, dtype=torch.int32, device=dev)
        nbytes = lib.tpk_three_nn_workspace_bytes(b, n, m) if with_workspace else 0
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
        assert lib.tpk_work_read_reset(ctypes.byref(count)) == 0
        st = lib.tpk_three_nn_f32(b, n, m, ctypes.c_void_p(u.data_ptr()), ctypes.c_void_p(k.data_ptr()),
                                  ctypes.c_void_p(dist2.data_ptr()), ctypes.c_void_p(idx.data_ptr()),
                                  ctypes.c_void_p(ws.data_ptr()) if nbytes else None, ctypes.c_size_t(nbytes),
                                  ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert st == 0
        assert lib.tpk_work_read_reset(ctypes.byref(count)) == 0
        wd, wi = oracle.three_nn(unknown.numpy(), known.numpy())
        np.testing.assert_array_equal(_np(idx), wi)
        np.testing.assert_array_equal(_np(dist2), wd)
        return int(count.value)

    assert run(1, 256, 100, False) == 256 * 100
    pruned = run(2, 4096, 2048, True)
    assert 2 * 4096 * 3 <= pruned < 2 * 4096 * 2048 // 2
    assert lib.tpk_work_read_reset(ctypes.byref(count)) == 0 and count.value == 0


def test_extension_rejects_bad_tensors(tpk, dev):
    x = torch.rand(2, 16, 3, device=dev)
    with pytest.raises(RuntimeError):
        tpk.ball_query(0.1, 4, x.transpose(0, 1), x)  # not contiguous
    with pytest.raises(RuntimeError):
        tpk.ball_query(0.1, 4, x.double(), x.double())  # wrong dtype
    with pytest.raises(RuntimeError):
        tpk.three_interpolate(torch.rand(2, 4, 16, device=dev), torch.zeros(2, 8, 3, dtype=torch.int64, device=dev),
                              torch.rand(2, 8, 3, device=dev))  # idx must be int32, as three_nn returns it


def test_lists_layout_and_fillers(dev):
    """The inverted index that the backward gathers walk, read back from the device: every index entry appears once in
    the list of its target, a target nobody refers to owns one empty entry, the last entry of every list is marked, and
    the places that fill a span's last row refer to nothing - as offset 0x7ff3fffc, which the walker relies on to lie
    beyond the LDS (reads there return zero)."""
    import ctypes
    import os

    lib = ctypes.CDLL(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "torch-points-kernels_amd",
                                   "torch_points_kernels", "libtpk_hip.so"))
    lib.tpk_three_interpolate_grad_workspace_bytes.restype = ctypes.c_size_t
    NOTHING, LAST, SPANS, WAVE, GAP = 0x7FF3FFFC, 0x80000000, 16, 64, 128
    for b, n, m in ((2, 3000, 500), (1, 20001, 130), (3, 700, 40)):
        g = torch.Generator().manual_seed(n + m)
        idx = torch.randint(0, m, (b, n, 3), generator=g, dtype=torch.int32)
        idx[idx == 7] = 8  # target 7 keeps an empty list
        weight = torch.rand(b, n, 3, generator=g)
        nbytes = lib.tpk_three_interpolate_grad_workspace_bytes(b, n, m)
        assert nbytes > 0
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        di, dw = idx.to(dev), weight.to(dev)
        st = lib.tpk_three_interpolate_lists_f32(b, n, m, ctypes.c_void_p(di.data_ptr()), ctypes.c_void_p(dw.data_ptr()),
                                                 ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(nbytes), None)
        assert st == 0
        torch.cuda.synchronize()
        raw = ws.cpu().numpy()
        # the shape the library chose: rows of grad_out staged together, columns per part (gather.hip, bwd_shape)
        span = -(-m // SPANS)
        n4 = (n + 3) & ~3
        for r in (4, 2, 1):
            room = min(40960 // r - span * SPANS, 32768 // r) & ~3
            if room >= n4 or (r == 1 and room >= 4096):
                part_len = min(n4, room)
                break
        parts = -(-n // part_len)
        cloud_parts = b * parts
        align = lambda v: (v + 255) & ~255
        capacity = ((part_len * 3 + m + 63) & ~63) + GAP * SPANS + 64
        regions = raw[: cloud_parts * SPANS * 16].view(np.int32).reshape(cloud_parts, SPANS, 4)
        off = align(cloud_parts * SPANS * 16) + align(cloud_parts * SPANS * WAVE * 4)
        entries = raw[off : off + cloud_parts * capacity * 8].view(np.uint32).reshape(cloud_parts, capacity, 2)
        weights = raw[off : off + cloud_parts * capacity * 8].view(np.float32).reshape(cloud_parts, capacity, 2)[..., 1]
        for cp in range(cloud_parts):
            cloud, part = divmod(cp, parts)
            col0 = part * part_len
            cols = min(part_len, n - col0)
            want = {}
            for j in range(cols):
                for k in range(3):
                    want.setdefault(int(idx[cloud, col0 + j, k]), []).append((j, float(weight[cloud, col0 + j, k])))
            for s in range(SPANS):
                base, length, steps, _ = (int(v) for v in regions[cp, s])
                t0, t1 = min(s * span, m), min((s + 1) * span, m)
                assert steps == -(-length // WAVE)
                ranks = np.arange(steps * WAVE)
                at = base + (ranks % max(steps, 1)) * WAVE + ranks // max(steps, 1)  # rank q -> lane q / c, step q % c
                js, ws_ = entries[cp, at, 0], weights[cp, at]
                # behind the last entry of the span: entries that refer to nothing
                assert (js[length:] == NOTHING).all() and (ws_[length:] == 0).all()
                target, got = t0, {}
                for q in range(length):
                    j = int(js[q])
                    if (j & 0x7FFFFFFF) != NOTHING:
                        got.setdefault(target, []).append(((j & 0x7FFFFFFF) >> 2, float(ws_[q])))
                    else:
                        assert j == (NOTHING | LAST) and target not in want  # the one entry of an empty list
                    if j & LAST:
                        target += 1
                assert target == t1
                for t in range(t0, t1):
                    assert sorted(got.get(t, [])) == sorted(want.get(t, [])), (cp, s, t)

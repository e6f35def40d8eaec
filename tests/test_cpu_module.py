"""The package's host module (points_cpu) behind the Python API, for CPU tensors.

Checked against: tests/golden/reference_cpu_vectors.npz (what the reference's own compiled CPU module returned for
these inputs, written by tests/golden/make_vectors.py), the known answers the reference's tests hold for CPU tensors
(test/test_ballquerry.py:25-34, 81-157; test/test_knn.py:14-30; test/test_fps.py:13-21; test/test_cluster.py:29-44;
test/test_metrics.py:16-55; test/test_interpolate.py:33-43; test/test_grouping.py), float64 brute force, and - where
oracle/_ref is built - the reference's module itself on fresh random inputs.  No GPU involved.
"""
import os

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def pkg():
    import torch_points_kernels as t
    from torch_points_kernels._native import host

    host()
    return t


@pytest.fixture(scope="module")
def vec():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_cpu_vectors.npz")
    return {k: v for k, v in np.load(path).items()}


def T(a):
    return torch.from_numpy(np.ascontiguousarray(a))


def test_host_module_exports_reference_names():
    from torch_points_kernels import points_cpu

    for name in ("dense_knn knn_interpolate knn_interpolate_grad fps ball_query batch_ball_query dense_ball_query "
                 "grow_proximity instance_iou").split():
        assert hasattr(points_cpu, name), name


# ---------------------------------------------------------------- golden vectors of the reference's CPU module
def test_knn_and_three_nn_golden(pkg, vec):
    support, query = T(vec["knn_support"]), T(vec["knn_query"])
    idx, d2 = pkg.knn(support, query, 9)
    assert idx.dtype == torch.int64 and d2.dtype == torch.float32
    assert np.array_equal(idx.numpy(), vec["knn_idx"]) and np.array_equal(d2.numpy(), vec["knn_dist2"])
    dist, idx3 = pkg.three_nn(query, support)
    assert idx3.dtype == torch.int64
    assert np.array_equal(idx3.numpy(), vec["three_nn_idx"])
    assert torch.equal(dist, torch.sqrt(T(vec["three_nn_dist2"])))


def test_knn_float64_golden(pkg, vec):
    idx, d2 = pkg.knn(T(vec["knn64_support"]), T(vec["knn64_query"]), 5)
    assert np.array_equal(idx.numpy(), vec["knn64_idx"]) and np.array_equal(d2.numpy(), vec["knn64_dist2"])
    idx, dist = pkg.ball_query(float(vec["ball64_radius"]), 10, T(vec["knn64_support"]), T(vec["knn64_query"]), mode="dense", sort=True)
    assert np.array_equal(idx.numpy(), vec["ball64_idx"]) and np.array_equal(dist.numpy(), vec["ball64_dist"])


def test_sorted_ball_query_golden(pkg, vec):
    support, query = T(vec["knn_support"]), T(vec["knn_query"])
    idx, dist = pkg.ball_query(float(vec["ball_sorted_radius"]), 12, support, query, mode="dense", sort=True)
    assert idx.dtype == torch.int64 and dist.dtype == torch.float32
    assert np.array_equal(idx.numpy(), vec["ball_sorted_idx"]) and np.array_equal(dist.numpy(), vec["ball_sorted_dist"])
    idx, dist = pkg.ball_query(float(vec["packed_radius"]), 10, T(vec["packed_x"]), T(vec["packed_y"]), mode="partial_dense",
                               batch_x=T(vec["packed_batch_x"]), batch_y=T(vec["packed_batch_y"]), sort=True)
    assert np.array_equal(idx.numpy(), vec["packed_sorted_idx"]) and np.array_equal(dist.numpy(), vec["packed_sorted_dist"])


def _check_unsorted_rows(idx, dist, all_idx, all_dist, nsample, dense):
    """Every row: min(nsample, hits) distinct members of the reference's complete hit list with their distances, then
    the padding of the layout."""
    idx, dist = idx.reshape(-1, idx.shape[-1]), dist.reshape(-1, dist.shape[-1])
    all_idx, all_dist = all_idx.reshape(-1, all_idx.shape[-1]), all_dist.reshape(-1, all_dist.shape[-1])
    assert idx.shape == (all_idx.shape[0], nsample)
    for q in range(idx.shape[0]):
        hits = {int(i): d for i, d in zip(all_idx[q], all_dist[q]) if d >= 0}
        kept = min(nsample, len(hits))
        row = [int(i) for i in idx[q, :kept]]
        assert len(set(row)) == kept and all(i in hits for i in row), q
        assert all(dist[q, j] == hits[row[j]] for j in range(kept)), q
        if len(hits) <= nsample:
            assert set(row) == set(hits), q
        pad = (row[0] if row else 0) if dense else -1
        assert all(int(i) == pad for i in idx[q, kept:]) and np.all(dist[q, kept:] == -1), q


def test_unsorted_ball_query_draws_from_the_reference_hit_lists(pkg, vec):
    support, query = T(vec["knn_support"]), T(vec["knn_query"])
    r = float(vec["ball_sorted_radius"])
    idx, dist = pkg.ball_query(r, 12, support, query, mode="dense")
    _check_unsorted_rows(idx.numpy(), dist.numpy(), vec["ball_all_idx"], vec["ball_all_dist"], 12, dense=True)
    # two unsorted calls differ, two sorted calls agree (the reference's own test: test/test_ballquerry.py:108-157)
    idx2, _ = pkg.ball_query(r, 12, support, query, mode="dense")
    assert not np.array_equal(idx.numpy(), idx2.numpy())
    args = (float(vec["packed_radius"]), 10, T(vec["packed_x"]), T(vec["packed_y"]))
    kw = dict(mode="PARTIAL_DENSE", batch_x=T(vec["packed_batch_x"]), batch_y=T(vec["packed_batch_y"]))
    idx, dist = pkg.ball_query(*args, **kw)
    _check_unsorted_rows(idx.numpy(), dist.numpy(), vec["packed_all_idx"], vec["packed_all_dist"], 10, dense=False)
    idx2, _ = pkg.ball_query(*args, **kw)
    assert not np.array_equal(idx.numpy(), idx2.numpy())
    a, _ = pkg.ball_query(*args, sort=True, **kw)
    b, _ = pkg.ball_query(*args, sort=True, **kw)
    assert np.array_equal(a.numpy(), b.numpy())


def test_fps_golden(pkg, vec):
    from torch_points_kernels import points_cpu

    cloud = T(vec["fps_xyz"])
    idx = points_cpu.fps(cloud, 64, False)
    assert idx.dtype == torch.int64 and np.array_equal(idx.numpy(), vec["fps_idx"])
    # the Python API starts at a random point drawn from torch's default generator, like the reference
    torch.manual_seed(int(vec["fps_random_seed"]))
    idx = pkg.furthest_point_sample(cloud, 64)
    assert np.array_equal(idx.numpy(), vec["fps_random_idx"])


def test_interpolate_golden(pkg, vec):
    feats, idx, w = T(vec["interp_features"]), T(vec["interp_idx"]), T(vec["interp_weight"])
    feats.requires_grad_(True)
    out = pkg.three_interpolate(feats, idx, w)
    assert np.array_equal(out.detach().numpy(), vec["interp_out"])
    out.backward(T(vec["interp_grad_out"]))
    assert np.array_equal(feats.grad.numpy(), vec["interp_grad"])


# ---------------------------------------------------------------- known answers of the reference's tests
def test_reference_kats_ball_query(pkg):
    a = torch.tensor([[[0, 0, 0], [1, 0, 0], [2, 0, 0]], [[0, 0, 0], [1, 0, 0], [2, 0, 0]]]).float()
    b = torch.tensor([[[0, 0, 0]], [[3, 0, 0]]]).float()
    idx, dist = pkg.ball_query(1.01, 2, a, b, sort=True)  # test/test_ballquerry.py:25-30
    assert idx.tolist() == [[[0, 1]], [[2, 2]]] and dist.tolist() == [[[0.0, 1.0]], [[1.0, -1.0]]]
    a = torch.tensor([[[0, 0, 0], [1, 0, 0], [1, 1, 0]]]).float()
    idx, _ = pkg.ball_query(1.01, 3, a, a, sort=True)  # :32-34
    assert idx.tolist() == [[[0, 1, 0], [1, 0, 2], [2, 1, 2]]]
    x = torch.tensor([[10, 0, 0], [0.1, 0, 0], [10, 0, 0], [10.1, 0, 0]]).float()
    y = torch.tensor([[0, 0, 0]]).float()
    idx, d2 = pkg.ball_query(1.0, 2, x, y, mode="PARTIAL_DENSE", batch_x=torch.zeros(4, dtype=torch.long),
                             batch_y=torch.zeros(1, dtype=torch.long))  # :81-96
    assert idx.tolist() == [[1, -1]]
    np.testing.assert_array_almost_equal(d2.numpy(), np.asarray([[0.01, -1.0]], dtype=np.float32))
    with pytest.raises(RuntimeError):  # :98-106
        pkg.ball_query(1.0, 2, x, y, mode="PARTIAL_DENSE", batch_x=torch.tensor([0, 0, 1, 1]), batch_y=torch.tensor([0]))
    # no hit in the dense layout: index 0, distance -1 (cpu/src/neighbors.cpp:66-67)
    idx, dist = pkg.ball_query(0.5, 3, a, torch.tensor([[[9.0, 9.0, 9.0]]]), sort=True)
    assert idx.tolist() == [[[0, 0, 0]]] and dist.tolist() == [[[-1.0, -1.0, -1.0]]]
    # a point at exactly the radius is not a hit (strict comparison)
    idx, dist = pkg.ball_query(1.0, 2, a, torch.tensor([[[2.0, 0.0, 0.0]]]), sort=True)
    assert idx.tolist() == [[[0, 0]]] and dist.tolist() == [[[-1.0, -1.0]]]


def test_reference_kats_knn_fps(pkg):
    from torch_points_kernels import points_cpu

    support = torch.tensor([[[0, 0, 0], [1, 0, 0], [2, 0, 0]]]).float()
    query = torch.tensor([[[0, 0, 0]]]).float()
    idx, dist = pkg.knn(support, query, 3)  # test/test_knn.py:14-23
    assert idx.tolist() == [[[0, 1, 2]]] and dist.tolist() == [[[0.0, 1.0, 4.0]]]
    assert pkg.knn(support, query, 2)[0].tolist() == [[[0, 1]]]
    with pytest.raises(RuntimeError):
        pkg.knn(support, query, 5)
    pkg.knn(torch.randn(2, 10, 3), torch.randn(2, 10, 3), 3)
    points = torch.tensor([[[0, 0, 0], [1, 0, 0], [2, 0, 0]], [[-1, 1, 0], [0, 0, 10], [0, 0, 2]]]).float()
    assert points_cpu.fps(points, 2, False).tolist() == [[0, 2], [0, 1]]  # test/test_fps.py:13-16
    starts = {int(points_cpu.fps(torch.randn(1, 100, 3), 2, True)[0, 0]) for _ in range(8)}
    assert len(starts) > 1  # random start (:18-21)
    with pytest.raises(ValueError):
        pkg.furthest_point_sample(points, 4)
    with pytest.raises(ValueError):
        pkg.three_nn(torch.rand(1, 2, 3), torch.rand(1, 5, 3))


def test_reference_kats_cluster(pkg):
    pos = torch.tensor([[0, 0, 0], [1, 0, 0], [2, 0, 0], [10, 0, 0], [0, 0, 0], [1, 0, 0], [2, 0, 0], [10, 0, 0]])
    batch = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1])
    labels = torch.tensor([0, 0, 1, 1, 0, 1, 1, 10])
    # test/test_cluster.py:29-44 (integer positions, as there)
    assert pkg.grow_proximity(pos, batch, radius=2, min_cluster_size=1) == [[0, 1, 2], [3], [4, 5, 6], [7]]
    assert pkg.grow_proximity(pos, batch, radius=2, min_cluster_size=3) == [[0, 1, 2], [4, 5, 6]]
    clusters = pkg.region_grow(pos, labels, batch, radius=2, min_cluster_size=1)
    assert [c.tolist() for c in clusters] == [[0, 1], [4], [2], [3], [5, 6], [7]]
    clusters = pkg.region_grow(pos.float(), labels, batch, radius=2, min_cluster_size=1)
    assert [c.tolist() for c in clusters] == [[0, 1], [4], [2], [3], [5, 6], [7]]


def test_grow_proximity_walk_order_and_sets():
    """The walk of the reference's host routine (cluster.py:9-37), on matrices no ball query produces: stack order,
    rows ending at -1, one-directional rows; clusters as sets against a transitive closure."""
    from torch_points_kernels import points_cpu

    nb = torch.tensor([[0, 1, 2], [1, 3, -1], [2, -1, 0], [3, -1, -1], [4, 0, -1]])
    members, starts = points_cpu.grow_proximity(nb, 1)
    # 0 pushes 1, 2; 2 is taken off first (nothing new), then 1 adds 3; 4 reaches only seen points
    assert members.tolist() == [0, 1, 2, 3, 4] and starts.tolist() == [0, 4, 5]
    members, starts = points_cpu.grow_proximity(nb, 2)
    assert members.tolist() == [0, 1, 2, 3] and starts.tolist() == [0, 4]
    rng = np.random.default_rng(5)
    n, width = 60, 3
    nb = rng.integers(0, n, size=(n, width))
    nb[rng.random((n, width)) < 0.4] = -1
    members, starts = points_cpu.grow_proximity(T(nb), 1)
    reach = np.eye(n, dtype=bool)
    for i in range(n):
        for v in nb[i]:
            if v == -1:
                break
            reach[i, v] = True
    for k in range(n):
        reach |= reach[:, [k]] & reach[[k], :]
    seen = np.zeros(n, dtype=bool)
    want = []
    for i in range(n):
        if not seen[i]:
            cluster = {int(j) for j in np.nonzero(reach[i] & ~seen)[0]}
            seen[list(cluster)] = True
            want.append(cluster)
    got = [set(members[a:b].tolist()) for a, b in zip(starts[:-1].tolist(), starts[1:].tolist())]
    assert got == want


def test_reference_kats_instance_iou(pkg):
    gt = torch.tensor([1, 2, 1, 2, 2, 3, 0])
    proposals = [torch.tensor([0, 2]), torch.tensor([1, 4]), torch.tensor([3, 5])]
    ious = pkg.instance_iou(proposals, gt)  # test/test_metrics.py:16-31
    torch.testing.assert_close(ious, torch.tensor([[1, 0, 0], [0, 2 / 3.0, 0], [0, 1.0 / 4.0, 1.0 / 2.0]]))
    batch = torch.tensor([0, 0, 1, 1, 1, 1, 1])
    proposals = [torch.tensor([0, 1]), torch.tensor([3, 4]), torch.tensor([5])]
    ious = pkg.instance_iou(proposals, gt, batch=batch)  # :33-55
    torch.testing.assert_close(ious, torch.tensor([[0.5, 0.5, 0, 0, 0], [0, 0, 0, 1, 0], [0, 0, 0, 0, 1.0]]))
    # random proposals against Python sets: |P n G| / |P u G|, no epsilon on the host (metrics.py:30-32)
    rng = np.random.default_rng(3)
    gt = T(rng.integers(0, 6, size=400))
    gt[0] = 5
    proposals = [T(rng.choice(400, size=rng.integers(1, 60), replace=False)) for _ in range(20)]
    ious = pkg.instance_iou(proposals, gt).numpy()
    for p, prop in enumerate(proposals):
        ps = set(prop.tolist())
        for inst in range(1, 6):
            gs = set(np.nonzero(gt.numpy() == inst)[0].tolist())
            assert ious[p, inst - 1] == np.float32(len(ps & gs) / float(len(ps | gs)))


def test_interpolate_gradcheck_and_grouping(pkg):
    torch.manual_seed(0)
    b, n = 2, 10  # test/test_interpolate.py:33-43
    pos, pos_skip = torch.randn(b, n, 3).double(), torch.randn(b, 2 * n, 3).double()
    x = torch.randn(b, 30, n, dtype=torch.float64, requires_grad=True)
    dist, idx = pkg.three_nn(pos_skip, pos)
    recip = 1.0 / (dist + 1e-8)
    weight = (recip / recip.sum(dim=2, keepdim=True)).double()
    assert torch.autograd.gradcheck(pkg.three_interpolate, (x, idx, weight), eps=1e-6, atol=1e-4)
    # grouping on CPU tensors and other dtypes: torch's gather, as in the reference (test/test_grouping.py:13-41)
    feats = torch.randn(2, 4, 9, dtype=torch.float64, requires_grad=True)
    gidx = torch.randint(0, 9, (2, 5, 3))
    out = pkg.grouping_operation(feats, gidx)
    want = torch.stack([feats[bi][:, gidx[bi]] for bi in range(2)])
    assert out.shape == (2, 4, 5, 3) and torch.equal(out, want)
    assert torch.autograd.gradcheck(pkg.grouping_operation, (feats, gidx))


# ---------------------------------------------------------------- brute force and the reference module on fresh inputs
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_searches_against_brute_force(pkg, dtype):
    g = torch.Generator().manual_seed(11)
    support = torch.rand(2, 1500, 3, generator=g, dtype=dtype)
    support[1, :40] = support[1, 40:80]  # duplicated points: equal distances, lower index first
    query = torch.rand(2, 200, 3, generator=g, dtype=dtype)
    query[1, :10] = support[1, :10]
    k, r = 7, 0.11
    idx, d2 = pkg.knn(support, query, k)
    ridx, rdist = pkg.ball_query(r, 9, support, query, mode="dense", sort=True)
    r2 = np.float32(r) * np.float32(r)
    for b in range(2):
        s, q = support[b].numpy(), query[b].numpy()
        diff = q[:, None, :] - s[None, :, :]
        all_d2 = (diff[..., 0] * diff[..., 0] + diff[..., 1] * diff[..., 1]) + diff[..., 2] * diff[..., 2]
        order = np.argsort(all_d2, axis=1, kind="stable")
        assert np.array_equal(idx[b].numpy(), order[:, :k])
        assert np.array_equal(d2[b].numpy(), np.take_along_axis(all_d2, order[:, :k], 1).astype(np.float32))
        for i in range(q.shape[0]):
            hits = [j for j in order[i] if all_d2[i, j] < s.dtype.type(r2)][:9]
            want = hits + [hits[0] if hits else 0] * (9 - len(hits))
            assert ridx[b, i].tolist() == want
            assert np.array_equal(rdist[b, i, :len(hits)].numpy(), all_d2[i, hits].astype(np.float32))


def test_against_reference_module_on_fresh_inputs(pkg, ref_cpu):
    if ref_cpu is None:
        pytest.skip("oracle/_ref is not built (needs the reference checkout)")
    from torch_points_kernels import points_cpu

    g = torch.Generator().manual_seed(77)
    support, query = torch.rand(3, 2000, 3, generator=g), torch.rand(3, 500, 3, generator=g)
    for got, want in zip(points_cpu.dense_knn(support, query, 16), ref_cpu.dense_knn(support, query, 16)):
        assert torch.equal(got, want)
    for got, want in zip(points_cpu.dense_ball_query(query, support, 0.1, 20, 0, True),
                         ref_cpu.dense_ball_query(query, support, 0.1, 20, 0, True)):
        assert torch.equal(got, want)
    x, y = torch.rand(5000, 3, generator=g), torch.rand(900, 3, generator=g)
    bx = torch.sort(torch.randint(0, 4, (5000,), generator=g))[0]
    by = torch.sort(torch.randint(0, 4, (900,), generator=g))[0]
    for got, want in zip(points_cpu.batch_ball_query(x, y, bx, by, 0.08, 16, 0, True),
                         ref_cpu.batch_ball_query(x, y, bx, by, 0.08, 16, 0, True)):
        assert torch.equal(got, want)
    cloud = torch.rand(4, 3000, 3, generator=g)
    torch.manual_seed(9)
    want = ref_cpu.fps(cloud, 200, True)
    torch.manual_seed(9)
    assert torch.equal(points_cpu.fps(cloud, 200, True), want)
    feats = torch.randn(3, 7, 2000, generator=g)
    idx = ref_cpu.dense_knn(support, query, 3)[0]
    w = torch.rand(3, 500, 3, generator=g)
    assert torch.equal(points_cpu.knn_interpolate(feats, idx, w), ref_cpu.knn_interpolate(feats, idx, w))
    go = torch.randn(3, 7, 500, generator=g)
    assert torch.equal(points_cpu.knn_interpolate_grad(go, idx, w, 2000), ref_cpu.knn_interpolate_grad(go, idx, w, 2000))


def test_packed_edge_cases(pkg):
    x = torch.rand(50, 3)
    bx = torch.tensor([0] * 20 + [2] * 30)  # cloud 1 has no support points
    y = torch.cat([x[:3], torch.rand(2, 3), x[20:23]])
    by = torch.tensor([0, 0, 0, 1, 1, 2, 2, 2])
    idx, dist = pkg.ball_query(0.01, 4, x, y, mode="partial_dense", batch_x=bx, batch_y=by, sort=True)
    assert idx[:3, 0].tolist() == [0, 1, 2] and idx[5:, 0].tolist() == [20, 21, 22]
    assert (idx[3:5] == -1).all() and (dist[3:5] == -1).all()
    idx, dist = pkg.ball_query(0.5, 4, x, torch.zeros(0, 3), mode="partial_dense", batch_x=bx,
                               batch_y=torch.zeros(0, dtype=torch.long))
    assert idx.shape == (0, 4) and dist.shape == (0, 4)


def test_gpu_only_operators_refuse_cpu_tensors(pkg):
    with pytest.raises(NotImplementedError):
        pkg.chamfer_dist.chamfer_dist(torch.rand(1, 4, 3), torch.rand(1, 4, 3))
    with pytest.raises(NotImplementedError):
        pkg.gridding(torch.rand(1, 4, 3) * 2 - 1, 8)


def test_edge_list_mode(pkg, ref_cpu):
    """mode = 1 (cpu/src/neighbors.cpp:107-135, :257-291): edges (support index, query row) with distances (E, 1)."""
    from torch_points_kernels import points_cpu

    g = torch.Generator().manual_seed(5)
    support, query = torch.rand(300, 3, generator=g), torch.rand(40, 3, generator=g)
    query[7] = 5.0  # a query without neighbours
    idx, dist = points_cpu.ball_query(support, query, 0.15, 6, 0, True)
    edges, d2 = points_cpu.ball_query(support, query, 0.15, 6, 1, True)
    assert edges.shape[1] == 2 and d2.shape == (edges.shape[0], 1) and edges.dtype == torch.int64 and d2.dtype == torch.float32
    want = []
    for i in range(40):
        used = int((dist[i] != -1).sum())
        if used == 0:
            want.append((0, i, -1.0))  # the reference's stand-in for "no neighbour" is kept as an edge
        want += [(int(idx[i, j]), i, float(dist[i, j])) for j in range(used)]
    assert [(int(a), int(b), float(c)) for (a, b), c in zip(edges.tolist(), d2[:, 0].tolist())] == want
    assert (7 in edges[:, 1].tolist()) and d2[edges[:, 1] == 7, 0].tolist() == [-1.0]
    x, y = torch.rand(900, 3, generator=g), torch.rand(120, 3, generator=g)
    y[3] = -4.0
    bx = torch.sort(torch.randint(0, 3, (900,), generator=g))[0]
    by = torch.sort(torch.randint(0, 3, (120,), generator=g))[0]
    idx, dist = points_cpu.batch_ball_query(x, y, bx, by, 0.12, 5, 0, True)
    edges, d2 = points_cpu.batch_ball_query(x, y, bx, by, 0.12, 5, 1, True)
    keep = dist != -1
    rows = torch.arange(120).unsqueeze(1).expand_as(idx)
    assert torch.equal(edges[:, 0], idx[keep]) and torch.equal(edges[:, 1], rows[keep]) and torch.equal(d2[:, 0], dist[keep])
    assert 3 not in edges[:, 1].tolist()  # packed layout: a row without neighbours contributes nothing
    if ref_cpu is not None:
        for got, want in zip(points_cpu.ball_query(support, query, 0.15, 6, 1, True), ref_cpu.ball_query(support, query, 0.15, 6, 1, True)):
            assert torch.equal(got, want)
        for got, want in zip(points_cpu.ball_query(support, query, 0.15, -1, 1, True), ref_cpu.ball_query(support, query, 0.15, -1, 1, True)):
            assert torch.equal(got, want)
        for got, want in zip((edges, d2), ref_cpu.batch_ball_query(x, y, bx, by, 0.12, 5, 1, True)):
            assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_rows_that_are_not_finite(pkg, dtype):
    """A NaN or infinite coordinate in the support cloud: never a neighbour inside a radius, last among the nearest;
    every other answer is what the cloud without those rows gives."""
    g = torch.Generator().manual_seed(21)
    clean = torch.rand(1, 700, 3, generator=g, dtype=dtype)
    bad_rows = [0, 5, 333, 699, 700, 701]
    support = torch.empty(1, 706, 3, dtype=dtype)
    keep = [i for i in range(706) if i not in bad_rows]
    support[0, keep] = clean[0, :700]
    support[0, 0] = torch.tensor([float("nan"), 0.5, 0.5], dtype=dtype)
    support[0, 5] = torch.tensor([0.5, float("inf"), 0.5], dtype=dtype)
    support[0, 333] = torch.tensor([float("-inf"), float("nan"), 0.1], dtype=dtype)
    support[0, 699] = float("nan")
    support[0, 700] = float("inf")
    support[0, 701] = torch.tensor([0.2, 0.2, float("-inf")], dtype=dtype)
    query = torch.rand(1, 90, 3, generator=g, dtype=dtype)
    remap = torch.tensor(keep)
    idx, d2 = pkg.knn(support, query, 9)
    cidx, cd2 = pkg.knn(clean, query, 9)
    assert torch.equal(idx, remap[cidx]) and torch.equal(d2, cd2)
    ridx, rd = pkg.ball_query(0.2, 12, support, query, mode="dense", sort=True)
    cridx, crd = pkg.ball_query(0.2, 12, clean, query, mode="dense", sort=True)
    hit = crd != -1
    assert torch.equal(rd, crd) and torch.equal(ridx[hit], remap[cridx][hit])
    dist, i3 = pkg.three_nn(query, support)
    cdist, ci3 = pkg.three_nn(query, clean)
    assert torch.equal(i3.long(), remap[ci3.long()]) and torch.equal(dist, cdist)
    # more neighbours asked for than finite rows exist: the others follow, in index order
    few = support[:, :8].clone()
    idx, d2 = pkg.knn(few, query[:, :4], 8)
    assert idx[0, :, 6:].tolist() == [[0, 5]] * 4 and not torch.isfinite(d2[0, :, 6:]).any()
    # a query that is not finite has no neighbour inside any radius
    q = torch.tensor([[[float("nan"), 0.5, 0.5], [float("inf"), 0.5, 0.5]]], dtype=dtype)
    ridx, rd = pkg.ball_query(0.5, 4, clean, q, mode="dense", sort=True)
    assert (rd == -1).all() and (ridx == 0).all()

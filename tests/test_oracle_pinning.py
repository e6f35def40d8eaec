"""Pins every function of oracle/tpk_oracle.c before anything is compared with it.

Three kinds of evidence, none of which restates the oracle's own formulas:
  * the known-answer vectors held by the reference's own tests (cited per test);
  * the reference's own CPU implementation, compiled from its sources into oracle/_ref
    (skipped where that build is absent);
  * independent mathematics: float64 brute force in numpy, scipy's cKDTree, torch.gather and
    autograd, hand-worked cases for the tie and padding rules.
"""
import numpy as np
import pytest
import torch
from scipy.spatial import cKDTree


def _need_ref(ref_cpu):
    if ref_cpu is None:
        pytest.skip("oracle/_ref/points_cpu.so not built (needs the reference checkout)")


# ----------------------------------------------------------------------------- ball query


def test_ball_dense_reference_kat(oracle):
    # reference test/test_ballquerry.py:18-23 (GPU known answer: pad idx with first hit, dist -1)
    a = np.array([[[0, 0, 0], [1, 0, 0], [2, 0, 0]], [[0, 0, 0], [1, 0, 0], [2, 0, 0]]], np.float32)
    b = np.array([[[0, 0, 0]], [[3, 0, 0]]], np.float32)
    idx, dist = oracle.ball_query_dense(1.01, 2, a, b)
    np.testing.assert_array_equal(idx, [[[0, 1]], [[2, 2]]])
    np.testing.assert_allclose(dist, [[[0, 1]], [[1, -1]]])


def test_ball_dense_no_hit_and_strict_radius(oracle):
    # No hit: idx row 0, dist row -1 (reference cuda/src/ball_query.cpp:26-29 pre-fill).
    # A point at exactly r is NOT returned in dense mode (strict <, ball_query_gpu.cu:37).
    xyz = np.array([[[0, 0, 0], [0.5, 0, 0], [5, 5, 5]]], np.float32)
    q = np.array([[[100, 0, 0], [1.0, 0, 0]]], np.float32)
    idx, dist = oracle.ball_query_dense(0.5, 3, xyz, q)
    np.testing.assert_array_equal(idx[0, 0], [0, 0, 0])
    np.testing.assert_array_equal(dist[0, 0], [-1, -1, -1])
    # query (1,0,0): point 1 is at distance exactly 0.5 -> excluded; nothing else within 0.5
    np.testing.assert_array_equal(idx[0, 1], [0, 0, 0])
    np.testing.assert_array_equal(dist[0, 1], [-1, -1, -1])


def test_ball_partial_reference_kat(oracle):
    # reference test/test_ballquerry.py:63-78: point at exactly r returned (<=), other cloud
    # ignored, -1 padding.
    x = np.array([[10, 0, 0], [0.1, 0, 0], [0.2, 0, 0], [0.1, 0, 0]], np.float32)
    y = np.array([[0, 0, 0]], np.float32)
    idx, dist2 = oracle.ball_query_partial_dense(0.2, 4, x, y, [0, 0, 0, 1], [0])
    np.testing.assert_array_equal(idx, [[1, 2, -1, -1]])
    np.testing.assert_array_almost_equal(dist2, np.array([[0.01, 0.04, -1, -1]], np.float32))


def test_ball_partial_reference_kat_cpu_vector(oracle):
    # reference test/test_ballquerry.py:81-96 (CPU known answer; also valid for the GPU rule)
    x = np.array([[10, 0, 0], [0.1, 0, 0], [10, 0, 0], [10.1, 0, 0]], np.float32)
    y = np.array([[0, 0, 0]], np.float32)
    idx, dist2 = oracle.ball_query_partial_dense(1.0, 2, x, y, [0, 0, 0, 0], [0])
    np.testing.assert_array_equal(idx, [[1, -1]])
    np.testing.assert_array_almost_equal(dist2, np.array([[0.01, -1.0]], np.float32))


def _brute_ball(xyz, q, r, strict):
    """float64 membership, independent of the oracle's arithmetic."""
    d = ((q[:, None, :].astype(np.float64) - xyz[None, :, :].astype(np.float64)) ** 2).sum(-1)
    return d, (d < r * r) if strict else (d <= r * r)


def test_ball_dense_first_nsample_in_index_order(oracle):
    rng = np.random.default_rng(0)
    xyz = rng.random((3, 700, 3), dtype=np.float32)
    q = rng.random((3, 90, 3), dtype=np.float32)
    r, ns = 0.2, 12
    idx, dist, pairs = oracle.ball_query_dense(r, ns, xyz, q, return_pairs=True)
    total_scan = 0
    for b in range(3):
        d64, inside = _brute_ball(xyz[b], q[b], np.float32(r), True)
        for j in range(90):
            hits = np.nonzero(inside[j])[0]
            # float64 membership can differ from fp32 only within rounding of the boundary
            margin = np.abs(d64[j] - np.float32(r) * np.float32(r)) < 1e-6
            assert not margin[hits].any(), "test data too close to the boundary"
            want = hits[:ns]
            cnt = len(want)
            np.testing.assert_array_equal(idx[b, j, :cnt], want)
            np.testing.assert_allclose(dist[b, j, :cnt], d64[j, want], rtol=1e-5)
            pad = want[0] if cnt else 0
            np.testing.assert_array_equal(idx[b, j, cnt:], np.full(ns - cnt, pad))
            np.testing.assert_array_equal(dist[b, j, cnt:], np.full(ns - cnt, -1.0, np.float32))
            total_scan += (hits[ns - 1] + 1) if len(hits) >= ns else 700
    assert pairs == total_scan


def test_ball_partial_matches_kdtree_sets(oracle):
    # Independent library: scipy cKDTree.query_ball_point per cloud (float64), as the
    # reference's tests use sklearn's KDTree for membership (test/test_ballquerry.py:163-169).
    rng = np.random.default_rng(1)
    sizes = [150, 1, 400]
    x = rng.random((sum(sizes), 3)).astype(np.float32)
    bx = np.repeat(np.arange(3), sizes)
    qsel = np.sort(rng.choice(len(x), 120, replace=False))
    y, by = x[qsel] + np.float32(0.01), bx[qsel]
    r, ns = 0.25, 1000
    idx, dist = oracle.ball_query_partial_dense(r, ns, x, y, bx, by)
    starts = np.concatenate([[0], np.cumsum(sizes)])
    for c in range(3):
        tree = cKDTree(x[starts[c]:starts[c + 1]].astype(np.float64))
        for row in np.nonzero(by == c)[0]:
            want = np.sort(np.array(tree.query_ball_point(y[row].astype(np.float64), float(np.float32(r))))) + starts[c]
            got = idx[row][idx[row] >= 0]
            np.testing.assert_array_equal(got, want)  # ascending global indices, own cloud only
            assert (dist[row][len(got):] == -1).all() and (idx[row][len(got):] == -1).all()


def test_ball_vs_reference_cpu_module(oracle, ref_cpu):
    # The reference CPU path returns the same SETS when nsample covers every neighbour
    # (reference test/test_ballquerry.py:43-58 compares its CPU and GPU paths this way).
    _need_ref(ref_cpu)
    g = torch.Generator().manual_seed(3)
    a = torch.randn(3, 300, 3, generator=g)
    b = torch.randn(3, 80, 3, generator=g)
    for r in (1.0, 0.3):
        idx_o, dist_o = oracle.ball_query_dense(r, 300, a.numpy(), b.numpy())
        idx_r, dist_r = ref_cpu.dense_ball_query(b, a, r, 300, 0, True)
        for i in range(3):
            for j in range(80):
                k = int((dist_o[i, j] >= 0).sum())
                assert set(idx_o[i, j, :k].tolist()) == set(idx_r[i, j, :k].tolist()) or k == 0
                assert int((dist_r[i, j] >= 0).sum()) == k
                np.testing.assert_array_equal(np.sort(dist_o[i, j, :k]), dist_r[i, j, :k].numpy())
    # packed layout, sorted CPU result vs oracle as sets + identical distances
    x = torch.randn(500, 3, generator=g)
    y = torch.randn(90, 3, generator=g)
    bx = torch.cat([torch.zeros(200), torch.ones(300)]).long()
    by = torch.cat([torch.zeros(40), torch.ones(50)]).long()
    idx_o, dist_o = oracle.ball_query_partial_dense(0.8, 500, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
    idx_r, dist_r = ref_cpu.batch_ball_query(x, y, bx, by, 0.8, 500, 0, True)
    for j in range(90):
        k = int((idx_o[j] >= 0).sum())
        assert set(idx_o[j, :k].tolist()) == set(idx_r[j][idx_r[j] >= 0].tolist())
        np.testing.assert_array_equal(np.sort(dist_o[j, :k]), dist_r[j, :k].numpy())


# ----------------------------------------------------------------------------- FPS


def test_fps_reference_kat(oracle):
    # reference test/test_fps.py:13-16 (CPU known answer; it also holds under the GPU rule:
    # point 0 of cloud 0 is the origin, skipped as a candidate, which changes nothing here).
    pts = np.array([[[0, 0, 0], [1, 0, 0], [2, 0, 0]], [[-1, 1, 0], [0, 0, 10], [0, 0, 2]]], np.float32)
    np.testing.assert_array_equal(oracle.furthest_point_sample(pts, 2), [[0, 2], [0, 1]])


def test_fps_tie_rule_hand_worked(oracle):
    # n = 8 -> the reference's block has 8 threads, one point each.  Points 3 and 4 are the
    # two furthest from point 0, at exactly the same distance.  Reduction tree
    # (cuda/src/sampling_gpu.cu:6-12, :67-138): stride 4: slot 0 takes point 4's entry
    # (25 > 0), slot 3 keeps point 3's; stride 2: slot 1 takes slot 3's entry; stride 1:
    # slot 0 (point 4) vs slot 1 (point 3) tie -> slot 0 keeps its own.  Winner: point 4.
    pts = np.full((1, 8, 3), 0, np.float32)
    pts[0, :, 0] = 10
    pts[0, :, 1] = [0, 1, 1, 5, -5, 1, 1, 1]
    out = oracle.furthest_point_sample(pts, 2)
    np.testing.assert_array_equal(out, [[0, 4]])
    # Mirror case: tie between points 1 and 2 -> stride 2: slot 0 takes point 2 (25 > 0);
    # stride 1: slot 0 (point 2) vs slot 1 (point 1) tie -> point 2 wins.
    pts[0, :, 1] = [0, 5, -5, 1, 1, 1, 1, 1]
    np.testing.assert_array_equal(oracle.furthest_point_sample(pts, 2), [[0, 2]])
    # Tie inside one reference thread: n = 1024 -> 512 threads, thread t owns t and t+512 and
    # keeps the first (lower index) of equal values.
    big = np.zeros((1, 1024, 3), np.float32)
    big[0, :, 0] = 10
    big[0, 7, 1] = 3
    big[0, 7 + 512, 1] = -3
    np.testing.assert_array_equal(oracle.furthest_point_sample(big, 2), [[0, 7]])


def test_fps_origin_skip_and_all_skipped(oracle):
    # Points with squared norm <= 1e-3 never become samples (cuda/src/sampling_gpu.cu:52-54).
    pts = np.array([[[1, 0, 0], [0.01, 0.01, 0.01], [1.5, 0, 0], [0, 0.03, 0]]], np.float32)
    out = oracle.furthest_point_sample(pts, 4)
    # eligible: 0 and 2 only; after both are taken every eligible distance is 0 and the
    # two-thread-per... reduction keeps returning an eligible index, never 1 or 3.
    assert out[0, 0] == 0 and out[0, 1] == 2
    assert set(out[0].tolist()) <= {0, 2}
    # nothing eligible: the reduction falls back to index 0 every round.
    tiny = np.full((1, 5, 3), 0.001, np.float32)
    np.testing.assert_array_equal(oracle.furthest_point_sample(tiny, 3), [[0, 0, 0]])


def _fps_float64(xyz, npoint):
    """Textbook FPS in float64 (no tie handling needed on generic data)."""
    n = xyz.shape[0]
    p = xyz.astype(np.float64)
    sel = [0]
    mind = np.full(n, np.inf)
    for _ in range(1, npoint):
        mind = np.minimum(mind, ((p - p[sel[-1]]) ** 2).sum(1))
        sel.append(int(np.argmax(mind)))
    return np.array(sel)


def test_fps_matches_float64_textbook(oracle):
    rng = np.random.default_rng(5)
    for n, m in ((100, 30), (700, 64), (2500, 100)):
        xyz = (rng.random((2, n, 3)) + 1.0).astype(np.float32)  # away from the origin
        out = oracle.furthest_point_sample(xyz, m)
        for b in range(2):
            np.testing.assert_array_equal(out[b], _fps_float64(xyz[b], m))


def test_fps_vs_reference_cpu_module(oracle, ref_cpu):
    # The reference's CPU FPS (cpu/src/fps.cpp) uses sqrt distances and no origin skip; on
    # clouds away from the origin it selects the same points when started at 0.
    _need_ref(ref_cpu)
    g = torch.Generator().manual_seed(11)
    pts = torch.rand(4, 600, 3, generator=g) + 1.0
    want = ref_cpu.fps(pts, 48, False).numpy()
    np.testing.assert_array_equal(oracle.furthest_point_sample(pts.numpy(), 48), want)


# ----------------------------------------------------------------------------- three_nn


def test_three_nn_reference_kat(oracle):
    # reference test/test_knn.py:14-20: idx [0,1,2], squared distances [0,1,4]
    support = np.array([[[0, 0, 0], [1, 0, 0], [2, 0, 0]]], np.float32)
    query = np.array([[[0, 0, 0]]], np.float32)
    dist2, idx = oracle.three_nn(query, support)
    np.testing.assert_array_equal(idx, [[[0, 1, 2]]])
    np.testing.assert_array_equal(dist2, [[[0.0, 1.0, 4.0]]])


def test_three_nn_ties_keep_lower_index_and_short_clouds(oracle):
    known = np.array([[[1, 0, 0], [-1, 0, 0], [0, 1, 0], [0, -1, 0], [0, 0, 3]]], np.float32)
    q = np.zeros((1, 1, 3), np.float32)
    dist2, idx = oracle.three_nn(q, known)
    np.testing.assert_array_equal(idx, [[[0, 1, 2]]])  # four equidistant points: first three
    np.testing.assert_array_equal(dist2, [[[1, 1, 1]]])
    dist2, idx = oracle.three_nn(q, known[:, :2])  # only two known points
    np.testing.assert_array_equal(idx, [[[0, 1, 0]]])
    assert dist2[0, 0, 0] == 1 and dist2[0, 0, 1] == 1 and np.isinf(dist2[0, 0, 2])


def test_three_nn_matches_kdtree(oracle):
    rng = np.random.default_rng(7)
    known = rng.standard_normal((3, 900, 3)).astype(np.float32)
    unknown = rng.standard_normal((3, 400, 3)).astype(np.float32)
    dist2, idx = oracle.three_nn(unknown, known)
    for b in range(3):
        d, i = cKDTree(known[b].astype(np.float64)).query(unknown[b].astype(np.float64), k=3)
        np.testing.assert_array_equal(idx[b], i)
        np.testing.assert_allclose(dist2[b], d ** 2, rtol=2e-5, atol=1e-7)


def test_three_nn_vs_reference_cpu_module(oracle, ref_cpu):
    # reference test/test_knn.py:36-46 compares CPU and GPU three_nn distances this way.
    _need_ref(ref_cpu)
    g = torch.Generator().manual_seed(13)
    known = torch.randn(4, 500, 3, generator=g)
    unknown = torch.randn(4, 250, 3, generator=g)
    idx_r, dist2_r = ref_cpu.dense_knn(known, unknown, 3)
    dist2, idx = oracle.three_nn(unknown.numpy(), known.numpy())
    np.testing.assert_array_equal(dist2, dist2_r.numpy())  # same unfused fp32 arithmetic
    np.testing.assert_array_equal(idx, idx_r.numpy())


# ----------------------------------------------------------------------------- knn (general k)


def test_knn_reference_kat(oracle):
    # reference test/test_knn.py:14-23
    support = np.array([[[0, 0, 0], [1, 0, 0], [2, 0, 0]]], np.float32)
    query = np.array([[[0, 0, 0]]], np.float32)
    idx, dist2 = oracle.knn(support, query, 3)
    np.testing.assert_array_equal(idx, [[[0, 1, 2]]])
    np.testing.assert_array_equal(dist2, [[[0.0, 1.0, 4.0]]])
    idx, _ = oracle.knn(support, query, 2)
    np.testing.assert_array_equal(idx, [[[0, 1]]])
    with pytest.raises(RuntimeError):
        oracle.knn(support, query, 5)


def test_knn_is_a_stable_sort_of_the_distances(oracle):
    # ascending (distance, index) = a stable argsort of the fp32 distances; duplicated points and a
    # quantised cloud give many exactly equal distances
    rng = np.random.default_rng(5)
    base = rng.random((2, 60, 3)).astype(np.float32)
    support = np.concatenate([base, base[:, ::-1], np.round(rng.random((2, 50, 3)) * 4).astype(np.float32) / 4], 1)
    query = np.concatenate([base[:, :20], rng.random((2, 30, 3)).astype(np.float32)], 1)
    for k in (1, 7, 33, support.shape[1]):
        idx, dist2 = oracle.knn(support, query, k)
        dx, dy, dz = (query[:, :, None, a] - support[:, None, :, a] for a in range(3))
        full = (dx * dx + dy * dy) + dz * dz  # fp32, unfused, the oracle's order of operations
        order = np.argsort(full, axis=2, kind="stable")[:, :, :k]
        np.testing.assert_array_equal(idx, order)
        np.testing.assert_array_equal(dist2, np.take_along_axis(full, order, 2))


def test_knn_with_three_neighbours_is_three_nn(oracle):
    rng = np.random.default_rng(6)
    known = np.round(rng.random((3, 90, 3)) * 6).astype(np.float32) / 3  # ties included
    unknown = rng.random((3, 70, 3)).astype(np.float32) * 2
    idx, dist2 = oracle.knn(known, unknown, 3)
    d3, i3 = oracle.three_nn(unknown, known)
    np.testing.assert_array_equal(idx, i3)
    np.testing.assert_array_equal(dist2, d3)


def test_knn_vs_reference_cpu_module(oracle, ref_cpu):
    # tie-free data: nanoflann's order is then fixed by the distances alone
    _need_ref(ref_cpu)
    g = torch.Generator().manual_seed(17)
    support = torch.randn(3, 400, 3, generator=g)
    query = torch.randn(3, 150, 3, generator=g)
    for k in (1, 5, 16, 40):
        idx_r, dist2_r = ref_cpu.dense_knn(support, query, k)
        idx, dist2 = oracle.knn(support.numpy(), query.numpy(), k)
        np.testing.assert_array_equal(dist2, dist2_r.numpy())
        np.testing.assert_array_equal(idx, idx_r.numpy())


# ----------------------------------------------------------------------------- interpolate


def _interp_inputs(seed, b=2, c=5, m=40, n=70):
    g = torch.Generator().manual_seed(seed)
    feats = torch.randn(b, c, m, generator=g)
    idx = torch.randint(0, m, (b, n, 3), generator=g)
    w = torch.rand(b, n, 3, generator=g)
    w = w / w.sum(2, keepdim=True)
    return feats, idx, w


def test_three_interpolate_closed_form_and_autograd(oracle):
    feats, idx, w = _interp_inputs(17)
    feats.requires_grad_(True)
    b, c, m = feats.shape
    n = idx.shape[1]
    gathered = torch.gather(feats.unsqueeze(2).expand(b, c, n, m), 3, idx.unsqueeze(1).expand(b, c, n, 3))
    want = (gathered * w.unsqueeze(1)).sum(-1)
    out = oracle.three_interpolate(feats.detach().numpy(), idx.numpy(), w.numpy())
    np.testing.assert_allclose(out, want.detach().numpy(), rtol=1e-6, atol=1e-6)
    gout = torch.randn(b, c, n, generator=torch.Generator().manual_seed(18))
    want.backward(gout)
    grad = oracle.three_interpolate_grad(gout.numpy(), idx.numpy(), w.numpy(), m)
    np.testing.assert_allclose(grad, feats.grad.numpy(), rtol=1e-5, atol=1e-6)


def test_three_interpolate_vs_reference_cpu_module(oracle, ref_cpu):
    # cpu/src/interpolate.cpp accumulates 0 + f1*w1 + f2*w2 + f3*w3 in the same order.
    _need_ref(ref_cpu)
    feats, idx, w = _interp_inputs(19, b=3, c=7, m=64, n=200)
    want = ref_cpu.knn_interpolate(feats, idx, w).numpy()
    np.testing.assert_array_equal(oracle.three_interpolate(feats.numpy(), idx.numpy(), w.numpy()), want)
    gout = torch.randn(3, 7, 200, generator=torch.Generator().manual_seed(20))
    want_g = ref_cpu.knn_interpolate_grad(gout, idx, w, 64).numpy()
    got_g = oracle.three_interpolate_grad(gout.numpy(), idx.numpy(), w.numpy(), 64)
    np.testing.assert_allclose(got_g, want_g, rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------------------- grouping


def test_grouping_reference_kat(oracle):
    # reference test/test_grouping.py:13-41
    features = np.array(
        [[[0, 10, 0], [1, 11, 0], [2, 12, 0]], [[100, 110, 120], [101, 111, 121], [102, 112, 122]]], np.float32
    )
    idx = np.array([[[1, 0], [0, 0]], [[0, 1], [1, 2]]], np.int64)
    expected = np.array(
        [
            [[[10, 0], [0, 0]], [[11, 1], [1, 1]], [[12, 2], [2, 2]]],
            [[[100, 110], [110, 120]], [[101, 111], [111, 121]], [[102, 112], [112, 122]]],
        ]
    )
    np.testing.assert_array_equal(oracle.grouping_operation(features, idx), expected)


def test_grouping_matches_torch_gather_and_autograd(oracle):
    # The reference implementation IS this torch expression (torchpoints.py:129-146).
    g = torch.Generator().manual_seed(23)
    feats = torch.randn(3, 6, 50, generator=g, requires_grad=True)
    idx = torch.randint(0, 50, (3, 9, 4), generator=g)
    all_idx = idx.reshape(3, -1).unsqueeze(1).repeat(1, 6, 1)
    want = feats.gather(2, all_idx).reshape(3, 6, 9, 4)
    np.testing.assert_array_equal(oracle.grouping_operation(feats.detach().numpy(), idx.numpy()), want.detach().numpy())
    gout = torch.randn(3, 6, 9, 4, generator=g)
    want.backward(gout)
    got = oracle.grouping_operation_grad(gout.numpy(), idx.numpy(), 50)
    np.testing.assert_allclose(got, feats.grad.numpy(), rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------------------- chamfer


def test_chamfer_reference_kats(oracle):
    # reference test/test_chamfer_dist.py:28-32 (2.333333) and :35-39 (ignore_zeros: 3.0)
    xyz1 = np.array([[[0, 0, 0], [1, 1, 1], [2, 0, 1]]], np.float32)
    xyz2 = np.array([[[1, 0, 0], [1, 2, 1]]], np.float32)
    d1, d2, i1, i2 = oracle.chamfer_fwd(xyz1, xyz2)
    assert abs(float(d1.mean() + d2.mean()) - 2.333333) < 1e-5
    np.testing.assert_array_equal(i1, [[0, 1, 0]])  # squared distances (1, 1, 2) by hand
    np.testing.assert_array_equal(i2, [[0, 1]])
    keep = xyz1.sum(2) != 0
    d1, d2, _, _ = oracle.chamfer_fwd(xyz1[keep][None], xyz2)
    assert abs(float(d1.mean() + d2.mean()) - 3.0) < 1e-5


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_chamfer_matches_brute_force(oracle, dtype):
    rng = np.random.default_rng(29)
    # sizes straddle the reference kernel's 512-point tile and its 4-way unrolled remainder
    for n, m in ((300, 515), (1030, 700), (64, 1)):
        a = rng.random((2, n, 3)).astype(dtype)
        b = rng.random((2, m, 3)).astype(dtype)
        d1, d2, i1, i2 = oracle.chamfer_fwd(a, b)
        dd = ((a[:, :, None, :].astype(np.float64) - b[:, None, :, :].astype(np.float64)) ** 2).sum(-1)
        np.testing.assert_array_equal(i1, dd.argmin(2))
        np.testing.assert_array_equal(i2, dd.argmin(1))
        tol = 1e-5 if dtype == np.float32 else 1e-12
        np.testing.assert_allclose(d1, dd.min(2), rtol=tol, atol=1e-7)
        np.testing.assert_allclose(d2, dd.min(1), rtol=tol, atol=1e-7)


def test_chamfer_first_index_on_exact_ties(oracle):
    a = np.zeros((1, 2, 3), np.float32)
    b = np.zeros((1, 1200, 3), np.float32)
    b[0, :, 0] = 5
    b[0, [3, 600, 1100], 0] = 1  # three equal minima, in different 512-tiles
    _, _, i1, _ = oracle.chamfer_fwd(a, b)
    np.testing.assert_array_equal(i1, [[3, 3]])


def test_chamfer_backward_closed_form(oracle):
    # d/dp |p - q|^2 = 2 (p - q): autograd through the matched pairs in float64.
    rng = np.random.default_rng(31)
    a = torch.tensor(rng.random((2, 40, 3)), dtype=torch.float64, requires_grad=True)
    b = torch.tensor(rng.random((2, 55, 3)), dtype=torch.float64, requires_grad=True)
    d1, d2, i1, i2 = oracle.chamfer_fwd(a.detach().numpy(), b.detach().numpy())
    g1 = torch.tensor(rng.standard_normal((2, 40)))
    g2 = torch.tensor(rng.standard_normal((2, 55)))
    i1t, i2t = torch.tensor(i1).long(), torch.tensor(i2).long()
    near1 = torch.gather(b, 1, i1t.unsqueeze(-1).expand(-1, -1, 3))
    near2 = torch.gather(a, 1, i2t.unsqueeze(-1).expand(-1, -1, 3))
    loss = (((a - near1) ** 2).sum(-1) * g1).sum() + (((b - near2) ** 2).sum(-1) * g2).sum()
    loss.backward()
    ga, gb = oracle.chamfer_bwd(a.detach().numpy(), b.detach().numpy(), i1, i2, g1.numpy(), g2.numpy())
    np.testing.assert_allclose(ga, a.grad.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(gb, b.grad.numpy(), rtol=1e-10, atol=1e-12)
    # float32 instantiation against the same closed form
    ga32, gb32 = oracle.chamfer_bwd(
        a.detach().numpy().astype(np.float32), b.detach().numpy().astype(np.float32), i1, i2,
        g1.numpy().astype(np.float32), g2.numpy().astype(np.float32))
    np.testing.assert_allclose(ga32, a.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(gb32, b.grad.numpy(), rtol=1e-4, atol=1e-5)


# ------------------------------------------------------------------ region growing


def test_grow_proximity_reference_vectors(oracle):
    # reference test/test_cluster.py:14-44
    pos = np.array([[0, 0, 0], [1, 0, 0], [2, 0, 0], [10, 0, 0]] * 2, np.float32)
    batch = np.array([0, 0, 0, 0, 1, 1, 1, 1])
    labels = np.array([0, 0, 1, 1, 0, 1, 1, 10])
    assert oracle.grow_proximity(pos, batch, radius=2, min_cluster_size=1) == [[0, 1, 2], [3], [4, 5, 6], [7]]
    assert oracle.grow_proximity(pos, batch, radius=2, min_cluster_size=3) == [[0, 1, 2], [4, 5, 6]]
    clusters = oracle.region_grow(pos, labels, batch, radius=2, min_cluster_size=1)
    assert [c.tolist() for c in clusters] == [[0, 1], [4], [2], [3], [5, 6], [7]]


def test_grow_proximity_walk_order_by_hand(oracle):
    # 0 lists 3 then 1; the last pushed (1) is expanded first and brings 2, then 3 brings 4.
    rows = np.array([[3, 1, -1], [2, 0, -1], [-1, 4, 4], [4, -1, 0], [-1, -1, -1], [5, -1, -1]], np.int64)
    assert oracle.grow_proximity_core(rows, 1) == [[0, 3, 1, 2, 4], [5]]
    assert oracle.grow_proximity_core(rows, 2) == [[0, 3, 1, 2, 4]]
    # one-directional rows: 2 lists 0, nobody lists 2 -> 2 stays alone although it "touches" the first cluster
    rows = np.array([[1, -1], [0, -1], [0, 1]], np.int64)
    assert oracle.grow_proximity_core(rows, 1) == [[0, 1], [2]]


def test_grow_proximity_clusters_are_classes_of_the_smallest_reaching_point(oracle):
    """Independent statement of what the walk computes: v belongs to the cluster started by the smallest point
    that reaches v along rows (transitive closure by repeated squaring of the boolean matrix)."""
    rng = np.random.default_rng(3)
    for n, ns, fill in ((12, 2, 0.6), (40, 3, 0.5), (90, 2, 0.8), (64, 4, 0.3)):
        rows = np.full((n, ns), -1, np.int64)
        for i in range(n):
            take = rng.permutation(n)[: rng.binomial(ns, fill)]
            rows[i, : len(take)] = take
        reach = np.eye(n, dtype=bool)
        for i in range(n):
            for j in rows[i]:
                if j < 0:
                    break
                reach[i, j] = True
        for _ in range(8):
            reach = reach | ((reach.astype(np.int32) @ reach.astype(np.int32)) > 0)
        first = reach.argmax(axis=0)  # smallest i with reach[i, v]
        want = [sorted(np.nonzero(first == s)[0].tolist()) for s in sorted(set(first.tolist()))]
        got = oracle.grow_proximity_core(rows, 1)
        assert [sorted(c) for c in got] == want
        assert [c[0] for c in got] == [c[0] for c in want]  # a cluster starts with its smallest point


# ------------------------------------------------------------------ ball query, sort=True


def test_ball_query_sorted_reference_vectors(oracle):
    # reference test/test_ballquerry.py:25-34
    a = np.array([[[0, 0, 0], [1, 0, 0], [2, 0, 0]], [[0, 0, 0], [1, 0, 0], [2, 0, 0]]], np.float32)
    b = np.array([[[0, 0, 0]], [[3, 0, 0]]], np.float32)
    idx, dist = oracle.ball_query_sorted_dense(1.01, 2, a, b)
    np.testing.assert_array_equal(idx, [[[0, 1]], [[2, 2]]])
    np.testing.assert_array_equal(dist, np.array([[[0, 1]], [[1, -1]]], np.float32))
    a = np.array([[[0, 0, 0], [1, 0, 0], [1, 1, 0]]], np.float32)
    idx, _ = oracle.ball_query_sorted_dense(1.01, 3, a, a)
    np.testing.assert_array_equal(idx, [[[0, 1, 0], [1, 0, 2], [2, 1, 2]]])
    # reference test/test_ballquerry.py:81-96 (one hit, so the order plays no part)
    x = np.array([[10, 0, 0], [0.1, 0, 0], [10, 0, 0], [10.1, 0, 0]], np.float32)
    idx, dist = oracle.ball_query_sorted_partial(1.0, 2, x, np.zeros((1, 3), np.float32), np.zeros(4, np.int64), np.zeros(1, np.int64))
    np.testing.assert_array_equal(idx, [[1, -1]])
    np.testing.assert_allclose(dist, [[0.01, -1]], rtol=1e-6)


def test_ball_query_sorted_is_a_stable_sort_of_the_hits(oracle):
    """Independent statement: hits = d2 < r2 (float32, strict), order = stable argsort of their distances; duplicated
    points and a lattice give equal distances, lattice spacing = radius gives points exactly on the sphere."""
    rng = np.random.default_rng(11)
    base = rng.random((2, 150, 3), dtype=np.float32)
    ax = np.arange(6, dtype=np.float32) * 0.25
    lattice = np.stack(np.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(1, -1, 3)
    for support, query, r, ns in ((np.concatenate([base, base[:, ::-1]], 1), base[:, :40], 0.3, 12), (lattice, lattice, 0.25, 5),
                                  (lattice, lattice, 0.5, 30), (base, base[:, :10], 0.01, 4)):
        idx, dist = oracle.ball_query_sorted_dense(r, ns, support, query)
        d = ((query[:, :, None, :] - support[:, None, :, :]) ** 2)
        d = (d[..., 0] + d[..., 1]) + d[..., 2]
        r2 = np.float32(r) * np.float32(r)
        for b in range(support.shape[0]):
            for j in range(query.shape[1]):
                hits = np.nonzero(d[b, j] < r2)[0]
                order = hits[np.argsort(d[b, j][hits], kind="stable")][:ns]
                k = len(order)
                np.testing.assert_array_equal(idx[b, j, :k], order)
                np.testing.assert_array_equal(dist[b, j, :k], d[b, j][order])
                assert (dist[b, j, k:] == -1).all() and (idx[b, j, k:] == (order[0] if k else 0)).all()


def test_ball_query_sorted_against_reference_cpu_module(oracle, ref_cpu):
    # the reference's own sort=True path (cpu/src/ball_query.cpp, nanoflann) on data without equal distances: bit-exact
    if ref_cpu is None:
        pytest.skip("oracle/_ref not built")
    import torch

    g = torch.Generator().manual_seed(4)
    for n, m, r, ns in ((500, 200, 0.6, 12), (64, 300, 1.0, 70), (2000, 100, 0.2, 5), (30, 20, 0.01, 4)):
        support, query = torch.randn(3, n, 3, generator=g), torch.randn(3, m, 3, generator=g)
        ri, rd = ref_cpu.dense_ball_query(query, support, r, ns, 0, True)
        oi, od = oracle.ball_query_sorted_dense(r, ns, support.numpy(), query.numpy())
        np.testing.assert_array_equal(oi, ri.numpy())
        np.testing.assert_array_equal(od, rd.numpy())
    x, y = torch.randn(900, 3, generator=g), torch.randn(300, 3, generator=g)
    bx = torch.sort(torch.randint(0, 3, (900,), generator=g))[0]
    by = torch.sort(torch.randint(0, 3, (300,), generator=g))[0]
    for r, ns in ((0.5, 9), (1.5, 40), (0.05, 3)):
        ri, rd = ref_cpu.batch_ball_query(x, y, bx, by, r, ns, 0, True)
        oi, od = oracle.ball_query_sorted_partial(r, ns, x.numpy(), y.numpy(), bx.numpy(), by.numpy())
        np.testing.assert_array_equal(oi, ri.numpy())
        np.testing.assert_array_equal(od, rd.numpy())


# ------------------------------------------------------------------ instance IoU


def test_instance_iou_reference_vectors(oracle):
    # reference test/test_metrics.py:16-55 (its own tolerance: assert_allclose defaults)
    gt = np.array([1, 2, 1, 2, 2, 3, 0])
    ious = oracle.instance_iou([[0, 2], [1, 4], [3, 5]], gt)
    np.testing.assert_allclose(ious, [[1, 0, 0], [0, 2 / 3.0, 0], [0, 1.0 / 4.0, 1.0 / 2.0]], rtol=1e-4, atol=1e-5)
    ious = oracle.instance_iou([[0, 1], [3, 4], [5]], gt, np.array([0, 0, 1, 1, 1, 1, 1]))
    np.testing.assert_allclose(ious, [[0.5, 0.5, 0, 0, 0], [0, 0, 0, 1, 0], [0, 0, 0, 0, 1]], rtol=1e-4, atol=1e-5)


def test_instance_iou_is_intersection_over_union_of_sets(oracle):
    rng = np.random.default_rng(9)
    n = 400
    batch = np.sort(rng.integers(0, 3, n))
    batch[0], batch[-1] = 0, 2
    gt = rng.integers(0, 7, n)
    for s in range(3):
        gt[np.nonzero(batch == s)[0][0]] = 6
    props = [rng.choice(np.nonzero(batch == s)[0], size=rng.integers(1, 60), replace=False) for s in (0, 1, 2, 1, 0)]
    ious = oracle.instance_iou(props, gt, batch)
    assert ious.shape == (5, 18)
    for p, prop in enumerate(props):
        s = batch[prop[0]]
        for k in range(6):
            inst = set(np.nonzero((batch == s) & (gt == k + 1))[0].tolist())
            want = len(inst & set(prop.tolist())) / (len(inst | set(prop.tolist())) + 1e-5)
            assert abs(ious[p, s * 6 + k] - want) < 1e-6
        other = np.ones(18, bool)
        other[s * 6 : s * 6 + 6] = False
        assert (ious[p, other] == 0).all()


# ------------------------------------------------------------------ gridding, cubic feature sampling


def _trilinear_grid(p, scale):
    """Independent float64 statement of gridding: cell = floor, fractions t, vertex weights (1 - t) / t per axis."""
    side = 2 * scale
    grid = np.zeros((p.shape[0], side, side, side))
    for b in range(p.shape[0]):
        for x, y, z in p[b]:
            cell = np.floor([x, y, z]).astype(int)
            t = np.array([x, y, z]) - cell
            for dx in (0, 1):
                for dy in (0, 1):
                    for dz in (0, 1):
                        w = (t[0] if dx else 1 - t[0]) * (t[1] if dy else 1 - t[1]) * (t[2] if dz else 1 - t[2])
                        i, j, k = cell + scale + (dx, dy, dz)
                        if 0 <= i < side and 0 <= j < side and 0 <= k < side:
                            grid[b, i, j, k] += w
    return grid.reshape(p.shape[0], -1)


def test_gridding_matches_trilinear_closed_form(oracle):
    rng = np.random.default_rng(1)
    scale = 4
    p = (rng.random((2, 60, 3)) * 2 - 1) * scale  # some points fall into the last cell: their outer vertices are dropped
    p[0, 0] = [1.0, -2.0, 0.0]  # on a vertex: all weight there
    p[0, 1] = [-4.0, -4.0, -4.0]  # the grid's first vertex
    for dtype, tol in ((np.float64, 1e-12), (np.float32, 1e-5)):
        grid, weights, indexes = oracle.gridding(p.astype(dtype), scale)
        np.testing.assert_allclose(grid, _trilinear_grid(p.astype(dtype).astype(np.float64), scale), rtol=tol, atol=tol)
        assert grid.dtype == dtype and indexes.dtype == np.int32
        # vertex order LLL .. UUU and the weights stored per axis
        prod = weights.prod(axis=3)
        inside = indexes >= 0
        np.testing.assert_allclose(np.where(inside, prod, 0).sum(), grid.sum(), rtol=1e-5)
        assert indexes[0, 0, 0] == (1 + 4) * 64 + (-2 + 4) * 8 + 4 and prod[0, 0, 0] == 1 and (prod[0, 0, 1:] == 0).all()
        assert indexes[0, 1, 0] == 0
    inner = (rng.random((1, 40, 3)) * 2 - 1) * (scale - 1)  # all 8 vertices inside: every point deposits exactly 1
    np.testing.assert_allclose(oracle.gridding(inner, scale)[0].sum(), 40, rtol=1e-12)


def reference_formula_vertices(point, scale):
    """The 8 (linear index, weight) pairs gridding_gpu.cu:43-131 forms for one point in grid units: floor / ceil per
    axis (ceil + 1 on a vertex), offsets from -scale, index = (ox * len + oy) * len + oz formed WITHOUT a range check,
    weight = product of 1 - |p - vertex| per axis.  Order LLL, LLU, LUL, LUU, ULL, ULU, UUL, UUU."""
    side = 2 * scale
    lo = np.floor(point).astype(int)
    hi = np.ceil(point).astype(int)
    hi = np.where(hi == lo, lo + 1, hi)
    out = []
    for cx in (lo[0], hi[0]):
        for cy in (lo[1], hi[1]):
            for cz in (lo[2], hi[2]):
                index = ((cx + scale) * side + (cy + scale)) * side + (cz + scale)
                weight = (1 - abs(point[0] - cx)) * (1 - abs(point[1] - cy)) * (1 - abs(point[2] - cz))
                inside = all(0 <= c + scale < side for c in (cx, cy, cz))
                out.append((index, weight, inside))
    return out


LAST_CELL_POINTS = {
    # a point in the last cell of one axis: its upper vertices on that axis lie outside the grid
    "z": np.array([0.25, -1.5, 2.6]), "y": np.array([-2.75, 2.3, 0.5]), "x": np.array([2.4, 1.25, -0.5]),
}


def check_last_cell_behaviour(gridding, scale=3):
    """For a vertex outside the grid the reference's formula still yields an index: past the last z it is the cell
    (x, y + 1, 0), past the last y the cell (x + 1, 0, z) - the weight lands in a cell far from the point - and past
    the last x it lies beyond the cloud's grid (the next cloud's memory).  Here such a vertex gets index -1 and deposits
    nothing; every vertex inside the grid has exactly the reference formula's index and weight."""
    for axis, point in LAST_CELL_POINTS.items():
        grid, weights, indexes = gridding(point[None, None, :].astype(np.float64), scale)
        want = np.zeros((2 * scale) ** 3)
        outside = 0
        for v, (index, weight, inside) in enumerate(reference_formula_vertices(point, scale)):
            if inside:
                assert indexes[0, 0, v] == index, (axis, v)
                want[index] += weight
            else:
                outside += 1
                assert indexes[0, 0, v] == -1, (axis, v)
                if axis != "x":  # where the reference would have added it: a cell of the grid, not next to the point
                    assert 0 <= index < want.size and want[index] == 0
                else:
                    assert index >= want.size
            np.testing.assert_allclose(weights[0, 0, v].prod(), weight, rtol=1e-12)
        assert outside == 4, axis
        np.testing.assert_allclose(grid[0], want, rtol=1e-12, atol=1e-15)
        assert abs(grid.sum() - sum(w for _, w, ins in reference_formula_vertices(point, scale) if ins)) < 1e-12


def test_gridding_last_cell_drops_the_vertices_outside(oracle):
    check_last_cell_behaviour(oracle.gridding)


def test_gridding_grad_matches_finite_differences(oracle):
    rng = np.random.default_rng(2)
    scale = 3
    p = (rng.random((2, 12, 3)) * 2 - 1) * (scale - 1)
    r = rng.standard_normal((2, (2 * scale) ** 3))
    grid, weights, indexes = oracle.gridding(p, scale)
    grad = oracle.gridding_grad(weights, indexes, r)
    eps = 1e-6
    for b, j, a in ((0, 0, 0), (0, 5, 1), (1, 3, 2), (1, 11, 0), (0, 7, 2)):
        hi, lo = p.copy(), p.copy()
        hi[b, j, a] += eps
        lo[b, j, a] -= eps
        fd = ((oracle.gridding(hi, scale)[0] - oracle.gridding(lo, scale)[0]) * r).sum() / (2 * eps)
        assert abs(fd - grad[b, j, a]) < 1e-6 * max(1.0, abs(fd))


def test_cubic_feature_sampling_is_a_gather(oracle):
    rng = np.random.default_rng(3)
    for ns, scale in ((1, 8), (2, 8), (3, 6)):
        p = rng.random((2, 30, 3)) * (scale + 2) - 1  # some points outside the grid
        p[0, 0] = [2.0, 3.0, 0.0]
        feats = rng.random((2, 5, scale, scale, scale))
        out, indexes = oracle.cubic_feature_sampling(p, feats, ns)
        nv = (2 * ns) ** 3
        assert out.shape == (2, 30, nv, 5) and indexes.shape == (2, 30, nv)
        for b in range(2):
            for i in range(30):
                lo = np.floor(p[b, i]).astype(int)
                hi = np.where(np.ceil(p[b, i]) == lo, lo + 1, np.ceil(p[b, i])).astype(int)
                at = 0
                for x in range(lo[0] - ns + 1, hi[0] + ns):
                    for y in range(lo[1] - ns + 1, hi[1] + ns):
                        for z in range(lo[2] - ns + 1, hi[2] + ns):
                            ok = 0 <= x < scale and 0 <= y < scale and 0 <= z < scale
                            assert indexes[b, i, at] == ((x * scale + y) * scale + z if ok else -1)
                            np.testing.assert_array_equal(out[b, i, at], feats[b, :, x, y, z] if ok else np.zeros(5))
                            at += 1
                assert at == nv
        g = rng.standard_normal(out.shape)
        grad_p, grad_f = oracle.cubic_feature_sampling_grad(scale, ns, g, indexes)
        want = np.zeros((2, 5, scale ** 3))
        for b in range(2):
            for i in range(30):
                for v in range(nv):
                    if indexes[b, i, v] >= 0:
                        want[b, :, indexes[b, i, v]] += g[b, i, v]
        np.testing.assert_allclose(grad_f.reshape(2, 5, -1), want, rtol=1e-12, atol=1e-12)
        assert (grad_p == 0).all()


# ------------------------------------------------------------------ committed reference vectors


def _golden():
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_cpu_vectors.npz")
    return np.load(path)  # arrays only (allow_pickle stays off)


def test_oracle_against_committed_reference_vectors(oracle):
    """tests/golden/reference_cpu_vectors.npz holds what the reference's CPU module returned for these inputs
    (tests/golden/make_vectors.py); it travels to machines without the reference checkout."""
    v = _golden()
    idx, dist2 = oracle.knn(v["knn_support"], v["knn_query"], 9)
    np.testing.assert_array_equal(idx, v["knn_idx"])
    np.testing.assert_array_equal(dist2, v["knn_dist2"])
    dist3, idx3 = oracle.three_nn(v["knn_query"], v["knn_support"])
    np.testing.assert_array_equal(idx3, v["three_nn_idx"])
    np.testing.assert_array_equal(dist3, v["three_nn_dist2"])
    idx, dist = oracle.ball_query_sorted_dense(float(v["ball_sorted_radius"]), 12, v["knn_support"], v["knn_query"])
    np.testing.assert_array_equal(idx, v["ball_sorted_idx"])
    np.testing.assert_array_equal(dist, v["ball_sorted_dist"])
    idx, dist = oracle.ball_query_sorted_partial(float(v["packed_radius"]), 10, v["packed_x"], v["packed_y"],
                                                 v["packed_batch_x"], v["packed_batch_y"])
    np.testing.assert_array_equal(idx, v["packed_sorted_idx"])
    np.testing.assert_array_equal(dist, v["packed_sorted_dist"])
    np.testing.assert_array_equal(oracle.furthest_point_sample(v["fps_xyz"], 64), v["fps_idx"])
    np.testing.assert_array_equal(oracle.three_interpolate(v["interp_features"], v["interp_idx"].astype(np.int32), v["interp_weight"]),
                                  v["interp_out"])

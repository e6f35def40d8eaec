"""Seeded differential run of the HIP operators against the CPU checker: a bounded number of random cases per
operator (shapes around the kernels' size thresholds, four kinds of clouds: uniform, Gaussian, clustered with
duplicated points, quantised coordinates with many exact ties), stopping at the first mismatch.  Integer outputs
and distances bit-exact, gradients within the stated tolerance.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

CASES = 24  # per operator; 11 operators


def _cloud(rng, B, n, kind, spread=1.0):
    if kind == 0:
        p = rng.random((B, n, 3))
    elif kind == 1:
        p = rng.normal(size=(B, n, 3)) * spread
    elif kind == 2:  # clustered + duplicates
        c = rng.random((B, 5, 3)) * 4 * spread
        p = c[np.arange(B)[:, None], rng.integers(0, 5, (B, n))] + 0.05 * rng.normal(size=(B, n, 3))
        if n >= 8:
            dup = rng.integers(0, n, (B, n // 8))
            p[:, : n // 8] = np.take_along_axis(p, dup[..., None].repeat(3, -1), 1)
    else:  # quantised coordinates: many exact ties
        p = np.round(rng.random((B, n, 3)) * 12) / 4
    return torch.from_numpy(p.astype(np.float32)).contiguous()


def _eq(got, want, what):
    got = got.detach().cpu().numpy()
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        pytest.fail("%s: first difference at %s: %s != %s" % (what, bad[0], got[tuple(bad[0])], want[tuple(bad[0])]))


def _packed(rng, kind, sizes_from, max_queries):
    nc = int(rng.integers(1, 5))
    sizes = [int(rng.choice(sizes_from)) for _ in range(nc)]
    xs, ys, bx, by = [], [], [], []
    for c, s in enumerate(sizes):
        p = _cloud(rng, 1, s, kind)[0]
        nq = int(rng.integers(0, min(max_queries, s) + 1))
        sel = np.sort(rng.choice(s, size=nq, replace=False)) if nq else np.zeros(0, dtype=np.int64)
        q = p[sel] + float(rng.choice([0.0, 0.01]))
        xs.append(p)
        ys.append(q)
        bx.append(torch.full((s,), c * 2, dtype=torch.long))  # (cloud ids with gaps)
        by.append(torch.full((q.shape[0],), c * 2, dtype=torch.long))
    if rng.random() < 0.3:  # a query cloud without support
        ys.append(_cloud(rng, 1, 17, 0)[0])
        by.append(torch.full((17,), 2 * nc - 1, dtype=torch.long))
        order = torch.argsort(torch.cat(by), stable=True)
        Y, BY = torch.cat(ys)[order], torch.cat(by)[order]
    else:
        Y, BY = torch.cat(ys), torch.cat(by)
    return sizes, torch.cat(xs), Y, torch.cat(bx), BY


def _fps(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 4))
    n = int(rng.choice([300, 513, 700, 1024, 1500, 3000, 5000, 9000, 16384, 16390, 21000, 33000, 40000, 70000]))
    npoint = int(rng.integers(1, min(n, 600 if n <= 16384 else 120)))
    x = _cloud(rng, B, n, kind) + (0.0 if kind != 3 else 0.3)
    _eq(tpk.furthest_point_sample(x.to(dev), npoint), oracle.furthest_point_sample(x.numpy(), npoint), "fps %s" % ((B, n, npoint, kind),))


def _three_nn(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 3))
    n = int(rng.choice([100, 512, 777, 2000, 6000, 17000]))
    m = int(rng.choice([3, 100, 512, 600, 1500, 5000, 20000]))
    u, k = _cloud(rng, B, n, kind), _cloud(rng, B, m, int(rng.integers(0, 4)))
    d, i = nat.three_nn(u.to(dev), k.to(dev))
    wd, wi = oracle.three_nn(u.numpy(), k.numpy())
    _eq(i, wi, "three_nn idx %s" % ((B, n, m, kind),))
    _eq(d, wd, "three_nn dist %s" % ((B, n, m, kind),))


def _chamfer(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 3))
    n = int(rng.choice([100, 512, 800, 3000, 7000, 18000]))
    m = int(rng.choice([64, 512, 900, 2500, 6000, 16400]))
    a, b = _cloud(rng, B, n, kind), _cloud(rng, B, m, int(rng.integers(0, 4)))
    d1, d2, i1, i2 = nat.chamfer_dist(a.to(dev), b.to(dev))
    w1, w2, wi1, wi2 = oracle.chamfer_fwd(a.numpy(), b.numpy())
    tag = " %s" % ((B, n, m, kind),)
    _eq(i1, wi1, "chamfer idx1" + tag)
    _eq(i2, wi2, "chamfer idx2" + tag)
    _eq(d1, w1, "chamfer dist1" + tag)
    _eq(d2, w2, "chamfer dist2" + tag)


def _chamfer_bwd(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 3))
    n = int(rng.choice([1, 70, 512, 3000, 9000]))
    m = int(rng.choice([1, 64, 900, 2500, 8000]))
    a, b = _cloud(rng, B, n, kind), _cloud(rng, B, m, int(rng.integers(0, 4)))
    w1, w2, wi1, wi2 = oracle.chamfer_fwd(a.numpy(), b.numpy())
    g1 = rng.normal(size=w1.shape).astype(np.float32)
    g2 = rng.normal(size=w2.shape).astype(np.float32)
    ga, gb = nat.chamfer_dist_grad(a.to(dev), b.to(dev), torch.from_numpy(wi1).to(dev), torch.from_numpy(wi2).to(dev),
                                   torch.from_numpy(g1).to(dev), torch.from_numpy(g2).to(dev))
    wa, wb = oracle.chamfer_bwd(a.numpy(), b.numpy(), wi1, wi2, g1, g2)
    # a point's gradient sums one term per point that has it as nearest neighbour (thousands on clouds with ties), in
    # another order than the checker: rtol 1e-5 / atol 1e-6 plus 1e-6 of the sum of the terms' magnitudes
    an, bn = a.numpy().astype(np.float64), b.numpy().astype(np.float64)
    mag_a, mag_b = np.zeros_like(an), np.zeros_like(bn)
    for c in range(B):
        own_a = np.abs(2 * g1[c][:, None] * (an[c] - bn[c][wi1[c]]))
        own_b = np.abs(2 * g2[c][:, None] * (bn[c] - an[c][wi2[c]]))
        mag_a[c] += own_a
        mag_b[c] += own_b
        np.add.at(mag_b[c], wi1[c], own_a)
        np.add.at(mag_a[c], wi2[c], own_b)
    for got, want, mag in ((ga, wa, mag_a), (gb, wb, mag_b)):
        err = np.abs(got.cpu().numpy() - want)
        assert (err <= 1e-6 + 1e-5 * np.abs(want) + 1e-6 * mag).all(), "chamfer bwd %s: max error %g" % ((B, n, m, kind), err.max())


def _interp(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 3))
    C = int(rng.choice([1, 3, 8, 17]))
    m = int(rng.choice([1, 5, 64, 130, 1000, 4100]))
    n = int(rng.choice([1, 7, 500, 3000, 9000, 16384, 16390, 35000]))
    feats = torch.from_numpy(rng.normal(size=(B, C, m)).astype(np.float32))
    gout = torch.from_numpy(rng.normal(size=(B, C, n)).astype(np.float32))
    idx = rng.integers(0, m, (B, n, 3))
    if kind >= 2:  # a few targets referenced by almost half of the entries: very long lists
        idx[rng.random((B, n, 3)) < 0.4] = rng.integers(0, min(m, 3))
    idx = torch.from_numpy(idx.astype(np.int32))
    w = torch.from_numpy(rng.random((B, n, 3)).astype(np.float32))
    f = feats.to(dev).requires_grad_(True)
    out = tpk.three_interpolate(f, idx.to(dev), w.to(dev))
    tag = " %s" % ((B, C, m, n, kind),)
    _eq(out, oracle.three_interpolate(feats.numpy(), idx.numpy(), w.numpy()), "interpolate fwd" + tag)
    out.backward(gout.to(dev))
    want = oracle.three_interpolate_grad(gout.numpy(), idx.numpy(), w.numpy(), m)
    tol = 1e-6 + 1e-5 * np.abs(want) + 1e-6 * oracle.three_interpolate_grad(np.abs(gout.numpy()), idx.numpy(), w.numpy(), m)
    assert (np.abs(f.grad.cpu().numpy() - want) <= tol).all(), "interpolate bwd" + tag


def _group(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 3))
    C = int(rng.choice([1, 3, 8]))
    N = int(rng.choice([1, 9, 64, 700, 5000]))
    npoint = int(rng.choice([1, 33, 512, 1300]))
    ns = int(rng.choice([1, 8, 32]))
    feats = torch.from_numpy(rng.normal(size=(B, C, N)).astype(np.float32))
    gout = torch.from_numpy(rng.normal(size=(B, C, npoint, ns)).astype(np.float32))
    idx = rng.integers(0, N, (B, npoint, ns))
    if kind >= 2:
        idx[rng.random((B, npoint, ns)) < 0.5] = 0
    idx = torch.from_numpy(idx)
    f = feats.to(dev).requires_grad_(True)
    out = tpk.grouping_operation(f, idx.to(dev))
    tag = " %s" % ((B, C, N, npoint, ns, kind),)
    _eq(out, oracle.grouping_operation(feats.numpy(), idx.numpy()), "grouping fwd" + tag)
    out.backward(gout.to(dev))
    want = oracle.grouping_operation_grad(gout.numpy(), idx.numpy(), N)
    tol = 1e-6 + 1e-5 * np.abs(want) + 1e-6 * oracle.grouping_operation_grad(np.abs(gout.numpy()), idx.numpy(), N)
    assert (np.abs(f.grad.cpu().numpy() - want) <= tol).all(), "grouping bwd" + tag


def _ball_packed(rng, kind, tpk, nat, oracle, dev):
    sizes, X, Y, BX, BY = _packed(rng, kind, [1, 40, 700, 5000, 12000, 20000], 4000)
    if Y.shape[0] == 0:
        return
    r = float(rng.choice([0.01, 0.05, 0.12, 0.3, 0.25]))
    ns = int(rng.choice([1, 5, 16, 64, 100]))
    i, d = tpk.ball_query(r, ns, X.to(dev), Y.to(dev), mode="partial_dense", batch_x=BX.to(dev), batch_y=BY.to(dev))
    wi, wd = oracle.ball_query_partial_dense(r, ns, X.numpy(), Y.numpy(), BX.numpy(), BY.numpy())
    tag = " %s" % ((sizes, Y.shape[0], r, ns, kind),)
    _eq(i, wi, "ball query packed idx" + tag)
    _eq(d, wd, "ball query packed dist" + tag)


def _ball_dense(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 4))
    n = int(rng.choice([1, 40, 512, 777, 3000, 4096, 17000, 20000, 70000]))
    m = int(rng.choice([1, 100, 512, 1024, 3000]))
    r = float(rng.choice([0.01, 0.05, 0.1, 0.3, 1.0]))
    ns = int(rng.choice([1, 5, 16, 32, 64, 100]))
    s = _cloud(rng, B, n, kind)
    q = s[:, :m].contiguous() if rng.random() < 0.5 and m <= n else _cloud(rng, B, m, int(rng.integers(0, 4)))
    i, d = tpk.ball_query(r, ns, s.to(dev), q.to(dev), mode="dense")
    wi, wd = oracle.ball_query_dense(r, ns, s.numpy(), q.numpy())
    tag = " %s" % ((B, n, q.shape[1], r, ns, kind),)
    _eq(i, wi, "ball query dense idx" + tag)
    _eq(d, wd, "ball query dense dist" + tag)


def _knn(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 3))
    n = int(rng.choice([40, 512, 777, 3000, 17000]))
    m = int(rng.choice([1, 100, 512, 2000, 6000]))
    k = min(int(rng.choice([1, 3, 8, 16, 20, 33, 70])), n)
    s, q = _cloud(rng, B, n, kind, 0.3), _cloud(rng, B, m, int(rng.integers(0, 4)), 0.3)
    i, d = tpk.knn(s.to(dev), q.to(dev), k)
    wi, wd = oracle.knn(s.numpy(), q.numpy(), k)
    _eq(i, wi, "knn idx %s" % ((B, n, m, k, kind),))
    _eq(d, wd, "knn dist %s" % ((B, n, m, k, kind),))


def _sorted_dense(rng, kind, tpk, nat, oracle, dev):
    B = int(rng.integers(1, 3))
    n = int(rng.choice([0, 40, 512, 777, 3000, 17000]))
    m = int(rng.choice([1, 100, 512, 2000, 6000]))
    r = float(rng.choice([0.01, 0.05, 0.12, 0.3, 1.0]))
    ns = int(rng.choice([1, 5, 16, 32, 40, 100]))
    s, q = _cloud(rng, B, n, kind, 0.3), _cloud(rng, B, m, int(rng.integers(0, 4)), 0.3)
    i, d = tpk.ball_query(r, ns, s.to(dev), q.to(dev), sort=True)
    wi, wd = oracle.ball_query_sorted_dense(r, ns, s.numpy(), q.numpy())
    _eq(i, wi, "sorted ball query dense idx %s" % ((B, n, m, r, ns, kind),))
    _eq(d, wd, "sorted ball query dense dist %s" % ((B, n, m, r, ns, kind),))


def _sorted_packed(rng, kind, tpk, nat, oracle, dev):
    sizes, X, Y, BX, BY = _packed(rng, kind, [1, 40, 600, 3000, 9000], 3000)
    if Y.shape[0] == 0:
        return
    r = float(rng.choice([0.01, 0.05, 0.12, 0.3]))
    ns = int(rng.choice([1, 5, 16, 40, 70]))
    i, d = tpk.ball_query(r, ns, X.to(dev), Y.to(dev), mode="partial_dense", batch_x=BX.to(dev), batch_y=BY.to(dev), sort=True)
    wi, wd = oracle.ball_query_sorted_partial(r, ns, X.numpy(), Y.numpy(), BX.numpy(), BY.numpy())
    _eq(i, wi, "sorted ball query packed idx %s" % ((sizes, Y.shape[0], r, ns, kind),))
    _eq(d, wd, "sorted ball query packed dist %s" % ((sizes, Y.shape[0], r, ns, kind),))


OPERATORS = {
    "fps": _fps, "three_nn": _three_nn, "chamfer": _chamfer, "chamfer_bwd": _chamfer_bwd, "three_interpolate": _interp,
    "grouping": _group, "ball_query_packed": _ball_packed, "ball_query_dense": _ball_dense, "knn": _knn,
    "ball_query_sorted_dense": _sorted_dense, "ball_query_sorted_packed": _sorted_packed,
}


@pytest.mark.parametrize("name", sorted(OPERATORS))
def test_random_cases_against_the_checker(name, tpk, oracle, dev):
    from torch_points_kernels._native import native

    seed = 1000 + sorted(OPERATORS).index(name)
    rng = np.random.default_rng(seed)
    for case in range(CASES):
        kind = int(rng.integers(0, 4))
        print("%s seed %d case %d kind %d" % (name, seed, case, kind), flush=True)
        OPERATORS[name](rng, kind, tpk, native(), oracle, dev)

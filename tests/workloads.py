"""Seeded synthetic inputs for the five benchmark configurations (CPU float32 tensors).

One generator per configuration; every call with the same arguments returns the same bits.
Used by the parity tests and by bench.py.  `scale` shrinks the point counts (1.0 = the full
configuration) so that the same recipe serves quick CPU-checked cases.
"""
import math

import torch

SEEDS = {"cfg1": 1001, "cfg2": 1002, "cfg3a": 1003, "cfg3b": 1013, "cfg4": 1004, "cfg5": 1005}


def _gen(name):
    g = torch.Generator(device="cpu")
    g.manual_seed(SEEDS[name])
    return g


def cfg1_ball_query_dense(B=8, N=4096, M=1024):
    """Uniform clouds in [0,1)^3; the query centres are each cloud's first M points."""
    g = _gen("cfg1")
    xyz = torch.rand(B, N, 3, generator=g, dtype=torch.float32)
    new_xyz = xyz[:, :M].contiguous()
    return {"xyz": xyz, "new_xyz": new_xyz, "radius": 0.1, "nsample": 32}


def cfg2_fps(B=16, N=16384, npoint=4096):
    """Per cloud: 8 Gaussian clusters (sigma 0.05, centres uniform in [0,1)^3) holding 90 % of
    the points, 10 % uniform background, shuffled."""
    g = _gen("cfg2")
    n_bg = N // 10
    n_cl = N - n_bg
    clouds = []
    for _ in range(B):
        centres = torch.rand(8, 3, generator=g)
        which = torch.randint(0, 8, (n_cl,), generator=g)
        pts = centres[which] + 0.05 * torch.randn(n_cl, 3, generator=g)
        bg = torch.rand(n_bg, 3, generator=g)
        cloud = torch.cat([pts, bg], 0)
        cloud = cloud[torch.randperm(N, generator=g)]
        clouds.append(cloud)
    return {"xyz": torch.stack(clouds).float().contiguous(), "npoint": npoint}


def cfg3a_interpolate(B=16, n=16384, m=4096, C=128):
    """unknown (B,n,3), known (B,m,3) uniform; features N(0,1) (B,C,m); upstream grad (B,C,n)."""
    g = _gen("cfg3a")
    unknown = torch.rand(B, n, 3, generator=g)
    known = torch.rand(B, m, 3, generator=g)
    features = torch.randn(B, C, m, generator=g)
    grad_out = torch.randn(B, C, n, generator=g)
    return {"unknown": unknown, "known": known, "features": features, "grad_out": grad_out}


def inverse_distance_weights(dist):
    """The weights the reference's own test builds from three_nn distances
    (reference test/test_interpolate.py:16-19)."""
    dist_recip = 1.0 / (dist + 1e-8)
    norm = torch.sum(dist_recip, dim=2, keepdim=True)
    return dist_recip / norm


def cfg3b_grouping(B=16, C=128, N=4096, npoint=1024, nsample=32):
    g = _gen("cfg3b")
    features = torch.randn(B, C, N, generator=g)
    idx = torch.randint(0, N, (B, npoint, nsample), generator=g, dtype=torch.int64)
    grad_out = torch.randn(B, C, npoint, nsample, generator=g)
    return {"features": features, "idx": idx, "grad_out": grad_out}


def cfg4_ball_query_partial(sizes=(20000, 45000, 70000, 100000)):
    """Packed indoor-like clouds: 80 % of the points on 6 random axis-aligned planes of
    extent 0-8 m (Gaussian noise 0.01 along the normal), 20 % uniform in the box; queries are a
    sorted random quarter of each cloud."""
    g = _gen("cfg4")
    xs, ys, bxs, bys = [], [], [], []
    for c, n in enumerate(sizes):
        n_pl = (n * 8) // 10
        n_un = n - n_pl
        axis = torch.randint(0, 3, (6,), generator=g)
        offset = 8.0 * torch.rand(6, generator=g)
        which = torch.randint(0, 6, (n_pl,), generator=g)
        pts = 8.0 * torch.rand(n_pl, 3, generator=g)
        normal = offset[which] + 0.01 * torch.randn(n_pl, generator=g)
        pts[torch.arange(n_pl), axis[which]] = normal
        uni = 8.0 * torch.rand(n_un, 3, generator=g)
        cloud = torch.cat([pts, uni], 0)
        cloud = cloud[torch.randperm(n, generator=g)].float()
        q = torch.sort(torch.randperm(n, generator=g)[: n // 4]).values
        xs.append(cloud)
        ys.append(cloud[q])
        bxs.append(torch.full((n,), c, dtype=torch.int64))
        bys.append(torch.full((q.numel(),), c, dtype=torch.int64))
    return {
        "x": torch.cat(xs).contiguous(),
        "y": torch.cat(ys).contiguous(),
        "batch_x": torch.cat(bxs),
        "batch_y": torch.cat(bys),
        "radius": 0.05,
        "nsample": 64,
    }


def cfg5_chamfer(B=32, N=16384):
    """Cloud 1: unit sphere + N(0, 0.02) noise; cloud 2: cloud 1 rotated, 5 % of its points
    jittered by N(0, 0.1); upstream gradients N(0,1)."""
    g = _gen("cfg5")
    p = torch.randn(B, N, 3, generator=g)
    p = p / p.norm(dim=2, keepdim=True)
    xyz1 = p + 0.02 * torch.randn(B, N, 3, generator=g)
    a = torch.randn(B, 3, 3, generator=g)
    qmat, _ = torch.linalg.qr(a)
    det = torch.linalg.det(qmat)
    qmat[:, :, 0] = qmat[:, :, 0] * det.sign().unsqueeze(1)  # make every det +1
    xyz2 = torch.bmm(xyz1, qmat.transpose(1, 2))
    n_j = N // 20
    for b in range(B):
        sel = torch.randperm(N, generator=g)[:n_j]
        xyz2[b, sel] += 0.1 * torch.randn(n_j, 3, generator=g)
    grad1 = torch.randn(B, N, generator=g)
    grad2 = torch.randn(B, N, generator=g)
    return {
        "xyz1": xyz1.float().contiguous(),
        "xyz2": xyz2.float().contiguous(),
        "grad_dist1": grad1,
        "grad_dist2": grad2,
    }


# Algorithmic work of each configuration (what throughput and roofline figures divide by).
def pairs_three_nn(B=16, n=16384, m=4096):
    return B * n * m


def pairs_chamfer(B=32, N=16384):
    return 2 * B * N * N


def fps_point_updates(B=16, N=16384, npoint=4096):
    return B * (npoint - 1) * N


def bytes_three_interpolate(B=16, C=128, m=4096, n=16384):
    return 4 * (B * C * m + B * C * n) + 2 * 4 * B * n * 3


def bytes_grouping(B=16, C=128, N=4096, npoint=1024, nsample=32):
    return 4 * (B * C * N + B * C * npoint * nsample) + 8 * B * npoint * nsample


def bytes_chamfer_bwd(B=32, N=16384):
    return 2 * (2 * B * N * 3 * 4) + 2 * B * N * 4 + 2 * B * N * 4


def region_cluster(num_points=100000):
    """The workload of the reference's benchmark/region_cluster.py: three unit cubes of uniform points, offset by 2,
    as one cloud; neighbours within 0.02, at most 16 (the defaults of grow_proximity)."""
    import torch

    g = torch.Generator().manual_seed(0)
    pos = torch.cat([torch.rand(num_points, 3, generator=g) + 2.0 * i for i in range(3)]).contiguous()
    batch = torch.ones(3 * num_points, dtype=torch.long)
    return {"pos": pos, "batch": batch, "radius": 0.02, "nsample": 16, "min_cluster_size": 32}


def instance_proposals(samples=4, points_per_sample=75000, instances=50, proposals=500, proposal_points=2000):
    """A PointGroup-like scoring step: proposals (index tensors) against the ground-truth instances of their sample."""
    import torch

    g = torch.Generator().manual_seed(7)
    n = samples * points_per_sample
    batch = torch.arange(samples).repeat_interleave(points_per_sample)
    gt = torch.randint(0, instances + 1, (n,), generator=g)
    gt[::points_per_sample] = instances
    props = []
    for p in range(proposals):
        s = p % samples
        props.append(torch.randint(s * points_per_sample, (s + 1) * points_per_sample, (proposal_points,), generator=g))
    return {"gt": gt, "batch": batch, "proposals": props}

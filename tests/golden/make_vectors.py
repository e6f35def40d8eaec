"""Writes tests/golden/reference_cpu_vectors.npz: inputs and the outputs the reference's own CPU
module gives for them.  The module is the one oracle/Makefile compiles from the reference's cpu/src
where it lies (oracle/_ref/points_cpu.so); this script therefore only runs where that checkout is
present.  The fixture holds data only (float32 / int64 arrays), small enough to commit, and lets the
GPU tests compare the HIP path with the reference's results directly, on machines without the
checkout.

    python tests/golden/make_vectors.py

Cases are chosen where the reference's CPU and CUDA paths compute the same thing (no equal
distances, clouds away from the origin for FPS): nearest-neighbour searches, the sorted radius
search, FPS started at point 0, three_interpolate.  For the package's host module (CPU tensors)
the fixture also holds: the complete hit lists of the radius searches (what an unsorted search
must draw its rows from), FPS with the random start the Python layer asks for (under a fixed seed
of torch's default generator, which is where the reference draws the start from), the gradient of
the interpolation, and a float64 search.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402


def main():
    ref = oracle.ref()
    if ref is None:
        sys.exit("oracle/_ref is not built (needs the reference checkout): run oracle.build_ref() first")
    g = torch.Generator().manual_seed(20240607)
    out = {}

    support = torch.rand(2, 700, 3, generator=g)
    query = torch.rand(2, 90, 3, generator=g)
    idx, dist2 = ref.dense_knn(support, query, 9)  # cpu/src/knn.cpp:43-62
    out.update(knn_support=support, knn_query=query, knn_idx=idx, knn_dist2=dist2)
    idx3, dist3 = ref.dense_knn(support, query, 3)  # what three_nn returns (int32 there)
    out.update(three_nn_idx=idx3, three_nn_dist2=dist3)

    idx, dist = ref.dense_ball_query(query, support, 0.15, 12, 0, True)  # cpu/src/ball_query.cpp:127-146, sorted
    out.update(ball_sorted_radius=np.float32(0.15), ball_sorted_idx=idx, ball_sorted_dist=dist)

    x = torch.rand(1500, 3, generator=g)
    y = torch.rand(400, 3, generator=g)
    bx = torch.sort(torch.randint(0, 3, (1500,), generator=g))[0]
    by = torch.sort(torch.randint(0, 3, (400,), generator=g))[0]
    idx, dist = ref.batch_ball_query(x, y, bx, by, 0.12, 10, 0, True)  # cpu/src/ball_query.cpp:65-124, sorted
    out.update(packed_x=x, packed_y=y, packed_batch_x=bx, packed_batch_y=by, packed_radius=np.float32(0.12),
               packed_sorted_idx=idx, packed_sorted_dist=dist)

    cloud = torch.rand(3, 900, 3, generator=g) + 1.0  # away from the origin: the CUDA kernel skips points near it
    out.update(fps_xyz=cloud, fps_idx=ref.fps(cloud, 64, False))  # cpu/src/fps.cpp, started at point 0

    feats = torch.randn(2, 5, 80, generator=g)
    nn_idx = torch.randint(0, 80, (2, 300, 3), generator=g)
    w = torch.rand(2, 300, 3, generator=g)
    w = w / w.sum(dim=2, keepdim=True)
    out.update(interp_features=feats, interp_idx=nn_idx, interp_weight=w,
               interp_out=ref.knn_interpolate(feats, nn_idx, w))  # cpu/src/interpolate.cpp

    # --- added for the host module; everything above keeps its draws from the generator
    idx, dist = ref.dense_ball_query(query, support, 0.15, 64, 0, True)  # wide enough for every hit list
    assert int((dist[..., -1] >= 0).sum()) == 0, "64 columns must hold every hit"
    out.update(ball_all_idx=idx, ball_all_dist=dist)
    idx, dist = ref.batch_ball_query(x, y, bx, by, 0.12, 64, 0, True)
    assert int((dist[..., -1] >= 0).sum()) == 0
    out.update(packed_all_idx=idx, packed_all_dist=dist)

    torch.manual_seed(4242)  # the reference draws the start point from torch's default generator (cpu/src/fps.cpp:24-25)
    out.update(fps_random_seed=np.int64(4242), fps_random_idx=ref.fps(cloud, 64, True))

    grad_out = torch.randn(2, 5, 300, generator=g)
    out.update(interp_grad_out=grad_out, interp_grad=ref.knn_interpolate_grad(grad_out, nn_idx, w, 80))

    support64 = torch.rand(2, 300, 3, generator=g, dtype=torch.float64)
    query64 = torch.rand(2, 40, 3, generator=g, dtype=torch.float64)
    idx, dist2 = ref.dense_knn(support64, query64, 5)
    out.update(knn64_support=support64, knn64_query=query64, knn64_idx=idx, knn64_dist2=dist2)
    idx, dist = ref.dense_ball_query(query64, support64, 0.2, 10, 0, True)
    out.update(ball64_radius=np.float32(0.2), ball64_idx=idx, ball64_dist=dist)

    arrays = {k: (v.numpy() if isinstance(v, torch.Tensor) else np.asarray(v)) for k, v in out.items()}
    path = os.path.join(HERE, "reference_cpu_vectors.npz")
    np.savez_compressed(path, **arrays)
    print("wrote", path, os.path.getsize(path), "bytes;", ", ".join("%s%s" % (k, v.shape) for k, v in arrays.items()))


if __name__ == "__main__":
    main()

// Host-side module for CPU tensors: torch_points_kernels.points_cpu.
//
// The reference package serves tensors that live in host memory through a module of this name
// (cpu/src/bindings.cpp:8-72, nanoflann k-d trees and ATen ops); this is the package's own
// counterpart, written over the small k-d tree of cpu/kd_tree.h.  It exports the reference's
// names with the reference's argument order - dense_knn, knn_interpolate, knn_interpolate_grad,
// fps, ball_query, batch_ball_query, dense_ball_query - and two routines the reference runs as
// numba code on the host: grow_proximity (torch_points_kernels/cluster.py:9-37) and instance_iou
// (torch_points_kernels/metrics.py:11-34).
//
// GPU tensors never come here: the Python layer sends them to points_cuda (the HIP kernels) and
// raises when that module is missing.  Nothing in this file is used by the GPU path.
//
// Semantics kept from the reference's CPU path (they differ from its CUDA path):
//   * radius search: hit = d2 < fl(r * r), strict (nanoflann); sorted = nearest first, cut at
//     max_num; unsorted = the hits in random order (std::mt19937 seeded from std::random_device,
//     cpu/src/neighbors.cpp:15-16,70-71), cut at max_num.  Dense layout pads idx with the row's
//     first entry (0 without hits) and dist with -1 (cpu/src/neighbors.cpp:60-105); the packed
//     layout pads both with -1 and returns indices into the packed support array (:226-251).
//   * knn: nearest first; equal distances keep the lower index first (nanoflann leaves that open).
//   * fps: int64 indices, euclidean (not squared) distances, first maximum, and - with
//     random = true, which is what the Python layer passes - a start point drawn from torch's
//     default generator the way the reference draws it: randperm(n)[0] (cpu/src/fps.cpp:6-36).
//   * knn_interpolate / knn_interpolate_grad: sums in index order (cpu/src/interpolate.cpp:6-72).
// Departures, all where the reference misbehaves: a packed cloud without support points has no
// neighbours (the reference searches the previous cloud's tree, cpu/src/neighbors.cpp:196-203);
// queries are assigned to clouds by their batch id, so empty query clouds are fine; index values
// outside the arrays raise instead of reading or writing out of bounds.
#include <torch/extension.h>

#include <ATen/Parallel.h>

#include <algorithm>
#include <cmath>
#include <memory>
#include <random>
#include <tuple>
#include <vector>

#include "cpu/kd_tree.h"

namespace {

using tpk_cpu::KdTree;
using tpk_cpu::Neighbour;

void check_points(const at::Tensor& t, int64_t dims, const char* name)
{
    TORCH_CHECK(!t.is_cuda(), name, " must be a CPU tensor");
    TORCH_CHECK(t.dim() == dims && t.size(dims - 1) == 3, name, " must have shape (", dims == 3 ? "B, " : "", "N, 3)");
    TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kDouble, name, " must be float32 or float64");
}

// The searches also take integer coordinates, as the reference's do (it dispatches over all types:
// cpu/src/ball_query.cpp:25, cpu/src/knn.cpp:20; its own cluster test passes int64 positions).  They are searched as
// float64, which holds them exactly up to 2^53; the squared radius is then cut to an integer, which is what the
// reference's conversion of the float radius to the integer distance type does.
struct Searchable
{
    at::Tensor points;
    bool integral;
};
Searchable searchable(const at::Tensor& t, int64_t dims, const char* name)
{
    TORCH_CHECK(!t.is_cuda(), name, " must be a CPU tensor");
    if (at::isIntegralType(t.scalar_type(), /*includeBool=*/false))
    {
        at::Tensor d = t.to(at::kDouble).contiguous();
        check_points(d, dims, name);
        return {d, true};
    }
    check_points(t, dims, name);
    return {t.contiguous(), false};
}

// One query's row of a radius search: `hits` in their final order, cut and padded to `width`.
template <typename T>
void write_row(std::vector<Neighbour<T>>& hits, bool sorted, std::mt19937& rng, int64_t width, int64_t offset, bool dense_padding,
               int64_t* idx, float* dist)
{
    if (sorted)
        std::sort(hits.begin(), hits.end());
    else
    {
        // (order of discovery depends on the tree: start from ascending indices so that the shuffle is the only source of order)
        std::sort(hits.begin(), hits.end(), [](const Neighbour<T>& a, const Neighbour<T>& b) { return a.index < b.index; });
        std::shuffle(hits.begin(), hits.end(), rng);
    }
    const int64_t kept = std::min<int64_t>(width, static_cast<int64_t>(hits.size()));
    for (int64_t j = 0; j < kept; ++j)
    {
        idx[j] = hits[static_cast<size_t>(j)].index + offset;
        dist[j] = static_cast<float>(hits[static_cast<size_t>(j)].d2);
    }
    const int64_t pad = dense_padding ? (hits.empty() ? 0 : hits[0].index + offset) : -1;
    for (int64_t j = kept; j < width; ++j)
    {
        idx[j] = pad;
        dist[j] = -1.0f;
    }
}

// Radius search of `nq` queries in one cloud of `ns` support points.  max_num > 0: rows of that width;
// otherwise the rows are as wide as the longest list (at least `min_width`).  Returns the width.
template <typename T>
int64_t radius_search(const T* support, int64_t ns, const T* query, int64_t nq, float radius, bool integral, int64_t max_num,
                      bool sorted, int64_t offset, bool dense_padding, int64_t min_width, std::vector<int64_t>& idx,
                      std::vector<float>& dist)
{
    // the reference squares the radius in float and converts to the points' type (cpu/src/neighbors.cpp:18)
    const float r2f = radius * radius;
    const T r2 = integral ? static_cast<T>(std::trunc(r2f)) : static_cast<T>(r2f);
    const KdTree<T> tree(support, ns);
    std::vector<std::vector<Neighbour<T>>> lists(static_cast<size_t>(nq));
    at::parallel_for(0, nq, 64, [&](int64_t q0, int64_t q1) {
        for (int64_t q = q0; q < q1; ++q)
        {
            auto& hits = lists[static_cast<size_t>(q)];
            tree.within(query + 3 * q, r2, [&](int64_t i, T d2) { hits.push_back(Neighbour<T>{d2, i}); });
        }
    });
    int64_t width = max_num;
    if (width <= 0)
    {
        width = min_width;
        for (const auto& l : lists)
            width = std::max<int64_t>(width, static_cast<int64_t>(l.size()));
    }
    idx.assign(static_cast<size_t>(nq * width), 0);
    dist.assign(static_cast<size_t>(nq * width), -1.0f);
    std::random_device device;
    const uint32_t seed = device();
    at::parallel_for(0, nq, 64, [&](int64_t q0, int64_t q1) {
        std::mt19937 rng(seed + static_cast<uint32_t>(q0) * 2654435761u);
        for (int64_t q = q0; q < q1; ++q)
            write_row(lists[static_cast<size_t>(q)], sorted, rng, width, offset, dense_padding, idx.data() + q * width,
                      dist.data() + q * width);
    });
    return width;
}

at::Tensor rows_to_tensor(const std::vector<int64_t>& v, int64_t rows, int64_t width)
{
    at::Tensor t = torch::empty({rows, width}, torch::dtype(torch::kLong));
    std::copy(v.begin(), v.end(), t.data_ptr<int64_t>());
    return t;
}
at::Tensor rows_to_tensor(const std::vector<float>& v, int64_t rows, int64_t width)
{
    at::Tensor t = torch::empty({rows, width}, torch::dtype(torch::kFloat));
    std::copy(v.begin(), v.end(), t.data_ptr<float>());
    return t;
}

void check_mode(int mode)
{
    TORCH_CHECK(mode == 0 || mode == 1, "mode must be 0 (a matrix of neighbours) or 1 (a list of edges)");
}

// mode = 1 of the reference (cpu/src/neighbors.cpp:107-135, :257-291; cpu/src/ball_query.cpp:45-51, :120-126): the
// neighbour matrix as a list of edges (support index, query row) with their squared distances (E, 1), query rows in
// order, a row's neighbours in the order of the matrix.  Unused slots of the matrix hold distance -1.  In the
// one-cloud search a query without neighbours keeps the reference's stand-in (0, -1) as an edge (`keep_empty`); in the
// packed layout such a row contributes nothing.
std::pair<at::Tensor, at::Tensor> matrix_to_edges(const at::Tensor& idx, const at::Tensor& dist, bool keep_empty)
{
    const int64_t rows = idx.size(0), width = idx.size(1);
    const int64_t* pi = idx.data_ptr<int64_t>();
    const float* pd = dist.data_ptr<float>();
    std::vector<int64_t> edges;
    std::vector<float> d2;
    for (int64_t i = 0; i < rows; ++i)
    {
        int64_t used = 0;
        while (used < width && pd[i * width + used] != -1.0f)
            ++used;
        if (used == 0 && keep_empty)
        {
            edges.push_back(0);
            edges.push_back(i);
            d2.push_back(-1.0f);
        }
        for (int64_t j = 0; j < used; ++j)
        {
            edges.push_back(pi[i * width + j]);
            edges.push_back(i);
            d2.push_back(pd[i * width + j]);
        }
    }
    const int64_t count = static_cast<int64_t>(d2.size());
    return {rows_to_tensor(edges, count, 2), rows_to_tensor(d2, count, 1)};
}

// support (N, 3), query (M, 3) of one cloud -> (idx (M, width) int64, dist2 (M, width) float32)
std::pair<at::Tensor, at::Tensor> ball_query(at::Tensor support, at::Tensor query, float radius, int max_num, int mode, bool sorted)
{
    TORCH_CHECK(support.scalar_type() == query.scalar_type(), "support and query must have the same dtype");
    const Searchable s = searchable(support, 2, "support"), q = searchable(query, 2, "query");
    support = s.points;
    query = q.points;
    check_mode(mode);
    std::vector<int64_t> idx;
    std::vector<float> dist;
    int64_t width = 0;
    AT_DISPATCH_FLOATING_TYPES(query.scalar_type(), "ball_query", [&] {
        width = radius_search<scalar_t>(support.data_ptr<scalar_t>(), support.size(0), query.data_ptr<scalar_t>(), query.size(0),
                                        radius, q.integral, max_num, sorted, 0, true, 1, idx, dist);
    });
    const at::Tensor out_idx = rows_to_tensor(idx, query.size(0), width), out_dist = rows_to_tensor(dist, query.size(0), width);
    if (mode == 1)
        return matrix_to_edges(out_idx, out_dist, true);
    return {out_idx, out_dist};
}

// Argument order of the reference (cpu/src/ball_query.cpp:127-146 with the swap at :137): the first tensor holds the
// ball centres (B, M, 3), the second the points searched (B, N, 3).
std::pair<at::Tensor, at::Tensor> dense_ball_query(at::Tensor centres, at::Tensor points, float radius, int max_num, int mode,
                                                   bool sorted)
{
    TORCH_CHECK(centres.dim() == 3 && points.dim() == 3 && centres.size(0) == points.size(0),
                "(B, M, 3) centres and (B, N, 3) points of the same number of clouds expected");
    std::vector<at::Tensor> all_idx, all_dist;
    for (int64_t b = 0; b < centres.size(0); ++b)
    {
        auto one = ball_query(points[b], centres[b], radius, max_num, mode, sorted);
        all_idx.push_back(one.first);
        all_dist.push_back(one.second);
    }
    if (all_idx.empty())
        return {torch::empty({0, centres.size(1), std::max(max_num, 1)}, torch::dtype(torch::kLong)),
                torch::empty({0, centres.size(1), std::max(max_num, 1)}, torch::dtype(torch::kFloat))};
    return {torch::stack(all_idx), torch::stack(all_dist)};
}

// Where every cloud of a sorted batch vector starts: starts[c] .. starts[c + 1].
std::vector<int64_t> cloud_starts(const at::Tensor& batch, int64_t clouds, const char* name)
{
    const int64_t* b = batch.data_ptr<int64_t>();
    const int64_t n = batch.numel();
    std::vector<int64_t> starts(static_cast<size_t>(clouds + 1), 0);
    for (int64_t i = 0; i < n; ++i)
    {
        TORCH_CHECK(b[i] >= 0 && b[i] < clouds && (i == 0 || b[i - 1] <= b[i]), name, " must be sorted and hold ids in [0, ", clouds, ")");
        ++starts[static_cast<size_t>(b[i] + 1)];
    }
    for (int64_t c = 0; c < clouds; ++c)
        starts[static_cast<size_t>(c + 1)] += starts[static_cast<size_t>(c)];
    return starts;
}

// Packed layout (cpu/src/ball_query.cpp:65-124): support (N, 3) with sorted cloud ids support_batch (N,), query (M, 3)
// with query_batch (M,).  Returns indices into `support`, -1 where a row has fewer neighbours.
std::pair<at::Tensor, at::Tensor> batch_ball_query(at::Tensor support, at::Tensor query, at::Tensor support_batch,
                                                   at::Tensor query_batch, float radius, int max_num, int mode, bool sorted)
{
    TORCH_CHECK(support.scalar_type() == query.scalar_type(), "support and query must have the same dtype");
    const Searchable sp = searchable(support, 2, "support"), qp = searchable(query, 2, "query");
    support = sp.points;
    query = qp.points;
    TORCH_CHECK(!support_batch.is_cuda() && !query_batch.is_cuda() && support_batch.scalar_type() == at::kLong &&
                    query_batch.scalar_type() == at::kLong && support_batch.dim() == 1 && query_batch.dim() == 1,
                "batch vectors must be 1-D int64 CPU tensors");
    TORCH_CHECK(support_batch.numel() == support.size(0) && query_batch.numel() == query.size(0),
                "one batch id per point is needed");
    check_mode(mode);
    support_batch = support_batch.contiguous();
    query_batch = query_batch.contiguous();
    const int64_t nq = query.size(0), ns = support.size(0);
    if (nq == 0)
        return {torch::empty({0, mode == 1 ? 2 : std::max(max_num, 0)}, torch::dtype(torch::kLong)),
                torch::empty({0, mode == 1 ? 1 : std::max(max_num, 0)}, torch::dtype(torch::kFloat))};
    const int64_t clouds = query_batch.data_ptr<int64_t>()[nq - 1] + 1;
    TORCH_CHECK(ns > 0 && clouds == support_batch.data_ptr<int64_t>()[ns - 1] + 1,
                "Both batches need to have the same number of samples.");
    const std::vector<int64_t> qs = cloud_starts(query_batch, clouds, "query_batch");
    const std::vector<int64_t> ss = cloud_starts(support_batch, clouds, "support_batch");

    // every cloud on its own, rows as wide as that cloud's search made them; then one matrix of the common width
    std::vector<std::vector<int64_t>> idx(static_cast<size_t>(clouds));
    std::vector<std::vector<float>> dist(static_cast<size_t>(clouds));
    std::vector<int64_t> widths(static_cast<size_t>(clouds), 0);
    int64_t width = std::max(max_num, 0);
    AT_DISPATCH_FLOATING_TYPES(query.scalar_type(), "batch_ball_query", [&] {
        for (int64_t c = 0; c < clouds; ++c)
        {
            const size_t k = static_cast<size_t>(c);
            widths[k] = radius_search<scalar_t>(support.data_ptr<scalar_t>() + 3 * ss[k], ss[k + 1] - ss[k],
                                                query.data_ptr<scalar_t>() + 3 * qs[k], qs[k + 1] - qs[k], radius, qp.integral, max_num,
                                                sorted, ss[k], false, 0, idx[k], dist[k]);
            width = std::max(width, widths[k]);
        }
    });
    at::Tensor out_idx = torch::full({nq, width}, -1, torch::dtype(torch::kLong));
    at::Tensor out_dist = torch::full({nq, width}, -1.0f, torch::dtype(torch::kFloat));
    for (int64_t c = 0; c < clouds; ++c)
    {
        const size_t k = static_cast<size_t>(c);
        for (int64_t q = qs[k]; q < qs[k + 1]; ++q)
        {
            std::copy_n(idx[k].data() + (q - qs[k]) * widths[k], widths[k], out_idx.data_ptr<int64_t>() + q * width);
            std::copy_n(dist[k].data() + (q - qs[k]) * widths[k], widths[k], out_dist.data_ptr<float>() + q * width);
        }
    }
    if (mode == 1)
        return matrix_to_edges(out_idx, out_dist, false);
    return {out_idx, out_dist};
}

// support (B, N, 3), query (B, M, 3) -> (idx (B, M, k) int64, dist2 (B, M, k) float32); cpu/src/knn.cpp:43-62
std::pair<at::Tensor, at::Tensor> dense_knn(at::Tensor support, at::Tensor query, int k)
{
    TORCH_CHECK(support.scalar_type() == query.scalar_type(), "support and query must have the same dtype");
    support = searchable(support, 3, "support").points;
    query = searchable(query, 3, "query").points;
    TORCH_CHECK(support.size(0) == query.size(0), "both tensors must hold the same number of clouds");
    TORCH_CHECK(k >= 0, "k must not be negative");
    TORCH_CHECK(support.size(1) >= k, "Not enough points in support to find " + std::to_string(k) + " neighboors");
    const int64_t b = query.size(0), n = support.size(1), m = query.size(1);
    at::Tensor idx = torch::empty({b, m, k}, torch::dtype(torch::kLong));
    at::Tensor dist = torch::empty({b, m, k}, torch::dtype(torch::kFloat));
    if (k == 0)
        return {idx, dist};
    AT_DISPATCH_FLOATING_TYPES(query.scalar_type(), "dense_knn", [&] {
        for (int64_t c = 0; c < b; ++c)
        {
            const KdTree<scalar_t> tree(support.data_ptr<scalar_t>() + 3 * n * c, n);
            const scalar_t* q = query.data_ptr<scalar_t>() + 3 * m * c;
            int64_t* oi = idx.data_ptr<int64_t>() + c * m * k;
            float* od = dist.data_ptr<float>() + c * m * k;
            at::parallel_for(0, m, 64, [&](int64_t q0, int64_t q1) {
                std::vector<Neighbour<scalar_t>> best(static_cast<size_t>(k));
                for (int64_t i = q0; i < q1; ++i)
                {
                    tree.nearest(q + 3 * i, k, best.data());
                    for (int64_t j = 0; j < k; ++j)
                    {
                        oi[i * k + j] = best[static_cast<size_t>(j)].index;
                        od[i * k + j] = static_cast<float>(best[static_cast<size_t>(j)].d2);
                    }
                }
            });
        }
    });
    return {idx, dist};
}

// points (B, N, 3) -> int64 (B, nsamples); cpu/src/fps.cpp:11-36
at::Tensor fps(at::Tensor points, const int nsamples, bool random)
{
    check_points(points, 3, "points");
    const int64_t b = points.size(0), n = points.size(1);
    TORCH_CHECK(nsamples >= 0 && (nsamples == 0 || n > 0), "cannot sample from an empty cloud");
    points = points.contiguous();
    at::Tensor out = torch::empty({b, nsamples}, torch::dtype(torch::kLong));
    if (nsamples == 0)
        return out;
    // start points first, cloud after cloud: the draws from torch's generator come in the reference's order
    std::vector<int64_t> start(static_cast<size_t>(b), 0);
    if (random)
        for (int64_t c = 0; c < b; ++c)
            start[static_cast<size_t>(c)] = at::randperm(n, torch::dtype(torch::kLong)).data_ptr<int64_t>()[0];
    AT_DISPATCH_FLOATING_TYPES(points.scalar_type(), "fps", [&] {
        const scalar_t* xyz = points.data_ptr<scalar_t>();
        int64_t* o = out.data_ptr<int64_t>();
        at::parallel_for(0, b, 1, [&](int64_t c0, int64_t c1) {
            std::vector<scalar_t> nearest(static_cast<size_t>(n));
            for (int64_t c = c0; c < c1; ++c)
            {
                const scalar_t* p = xyz + 3 * n * c;
                std::fill(nearest.begin(), nearest.end(), std::numeric_limits<scalar_t>::infinity());
                int64_t last = start[static_cast<size_t>(c)];
                o[c * nsamples] = last;
                for (int64_t s = 1; s < nsamples; ++s)
                {
                    const scalar_t* centre = p + 3 * last;
                    scalar_t best = -1;
                    int64_t arg = 0;
                    for (int64_t i = 0; i < n; ++i)
                    {
                        const scalar_t d = std::sqrt(tpk_cpu::squared_distance(p + 3 * i, centre));
                        const scalar_t v = std::min(nearest[static_cast<size_t>(i)], d);
                        nearest[static_cast<size_t>(i)] = v;
                        if (v > best) // first maximum
                        {
                            best = v;
                            arg = i;
                        }
                    }
                    o[c * nsamples + s] = arg;
                    last = arg;
                }
            }
        });
    });
    return out;
}

void check_interpolation(const at::Tensor& values, const at::Tensor& idx, const at::Tensor& weight, const char* name)
{
    TORCH_CHECK(!values.is_cuda() && !idx.is_cuda() && !weight.is_cuda(), name, ": CPU tensors expected");
    TORCH_CHECK(values.dim() == 3 && idx.dim() == 3 && weight.dim() == 3, name, ": 3-D tensors expected");
    TORCH_CHECK(idx.scalar_type() == at::kLong, name, ": idx must be int64");
    TORCH_CHECK(values.scalar_type() == weight.scalar_type(), name, ": values and weights must have the same dtype");
    TORCH_CHECK(idx.sizes() == weight.sizes() && idx.size(0) == values.size(0), name, ": shapes do not match");
}

// features (B, c, m), idx (B, n, K) int64, weight (B, n, K) -> (B, c, n); cpu/src/interpolate.cpp:6-39
at::Tensor knn_interpolate(at::Tensor features, at::Tensor idx, at::Tensor weight)
{
    check_interpolation(features, idx, weight, "knn_interpolate");
    features = features.contiguous();
    idx = idx.contiguous();
    weight = weight.contiguous();
    const int64_t b = features.size(0), c = features.size(1), m = features.size(2), n = idx.size(1), k = idx.size(2);
    TORCH_CHECK(idx.numel() == 0 || (idx.min().item<int64_t>() >= 0 && idx.max().item<int64_t>() < m),
                "knn_interpolate: idx outside the feature rows");
    at::Tensor out = torch::empty({b, c, n}, features.options());
    AT_DISPATCH_FLOATING_TYPES(features.scalar_type(), "knn_interpolate", [&] {
        const scalar_t* f = features.data_ptr<scalar_t>();
        const scalar_t* w = weight.data_ptr<scalar_t>();
        const int64_t* ix = idx.data_ptr<int64_t>();
        scalar_t* o = out.data_ptr<scalar_t>();
        at::parallel_for(0, b * c, 1, [&](int64_t r0, int64_t r1) {
            for (int64_t r = r0; r < r1; ++r)
            {
                const int64_t cloud = r / c;
                const scalar_t* row = f + r * m;
                for (int64_t p = 0; p < n; ++p)
                {
                    const int64_t e = (cloud * n + p) * k;
                    scalar_t acc = 0;
                    for (int64_t t = 0; t < k; ++t)
                        acc += row[ix[e + t]] * w[e + t];
                    o[r * n + p] = acc;
                }
            }
        });
    });
    return out;
}

// grad_out (B, c, n), idx (B, n, K), weight (B, n, K), m -> (B, c, m); cpu/src/interpolate.cpp:41-72
at::Tensor knn_interpolate_grad(at::Tensor grad_out, at::Tensor idx, at::Tensor weight, const int m)
{
    check_interpolation(grad_out, idx, weight, "knn_interpolate_grad");
    grad_out = grad_out.contiguous();
    idx = idx.contiguous();
    weight = weight.contiguous();
    const int64_t b = grad_out.size(0), c = grad_out.size(1), n = idx.size(1), k = idx.size(2);
    TORCH_CHECK(grad_out.size(2) == n, "knn_interpolate_grad: shapes do not match");
    TORCH_CHECK(idx.numel() == 0 || (idx.min().item<int64_t>() >= 0 && idx.max().item<int64_t>() < m),
                "knn_interpolate_grad: idx outside the feature rows");
    at::Tensor out = torch::zeros({b, c, m}, grad_out.options());
    AT_DISPATCH_FLOATING_TYPES(grad_out.scalar_type(), "knn_interpolate_grad", [&] {
        const scalar_t* g = grad_out.data_ptr<scalar_t>();
        const scalar_t* w = weight.data_ptr<scalar_t>();
        const int64_t* ix = idx.data_ptr<int64_t>();
        scalar_t* o = out.data_ptr<scalar_t>();
        // rows are independent; inside a row the terms are added in the order of the columns, as a serial loop adds them
        at::parallel_for(0, b * c, 1, [&](int64_t r0, int64_t r1) {
            for (int64_t r = r0; r < r1; ++r)
            {
                const int64_t cloud = r / c;
                scalar_t* row = o + r * m;
                for (int64_t p = 0; p < n; ++p)
                {
                    const int64_t e = (cloud * n + p) * k;
                    const scalar_t gv = g[r * n + p];
                    for (int64_t t = 0; t < k; ++t)
                        row[ix[e + t]] += gv * w[e + t];
                }
            }
        });
    });
    return out;
}

// neighbours (N, nsample) int64, rows ending at the first -1.  Clusters in the order and with the member order of the
// reference's walk (torch_points_kernels/cluster.py:9-37): points in index order; an unseen point starts a cluster and
// a stack; the last stack entry is taken off, its row read left to right, every unseen neighbour marked, pushed and
// appended.  Returns (members, starts): cluster i = members[starts[i] : starts[i + 1]]; clusters below min_cluster_size
// are dropped.
std::pair<at::Tensor, at::Tensor> grow_proximity(at::Tensor neighbours, int64_t min_cluster_size)
{
    TORCH_CHECK(!neighbours.is_cuda() && neighbours.dim() == 2 && neighbours.scalar_type() == at::kLong,
                "neighbours must be a 2-D int64 CPU tensor");
    neighbours = neighbours.contiguous();
    const int64_t n = neighbours.size(0), width = neighbours.size(1);
    const int64_t* nb = neighbours.data_ptr<int64_t>();
    std::vector<char> seen(static_cast<size_t>(n), 0);
    std::vector<int64_t> members, starts{0}, stack;
    for (int64_t i = 0; i < n; ++i)
    {
        if (seen[static_cast<size_t>(i)])
            continue;
        const size_t first = members.size();
        seen[static_cast<size_t>(i)] = 1;
        stack.assign(1, i);
        members.push_back(i);
        while (!stack.empty())
        {
            const int64_t k = stack.back();
            stack.pop_back();
            for (int64_t j = 0; j < width; ++j)
            {
                const int64_t v = nb[k * width + j];
                if (v == -1)
                    break;
                TORCH_CHECK(v >= 0 && v < n, "neighbour index outside the cloud");
                if (!seen[static_cast<size_t>(v)])
                {
                    seen[static_cast<size_t>(v)] = 1;
                    stack.push_back(v);
                    members.push_back(v);
                }
            }
        }
        if (static_cast<int64_t>(members.size() - first) >= min_cluster_size)
            starts.push_back(static_cast<int64_t>(members.size()));
        else
            members.resize(first);
    }
    at::Tensor m = torch::empty({static_cast<int64_t>(members.size())}, torch::dtype(torch::kLong));
    std::copy(members.begin(), members.end(), m.data_ptr<int64_t>());
    at::Tensor s = torch::empty({static_cast<int64_t>(starts.size())}, torch::dtype(torch::kLong));
    std::copy(starts.begin(), starts.end(), s.data_ptr<int64_t>());
    return {m, s};
}

// IoU of every proposal with the ground-truth instances of its sample (torch_points_kernels/metrics.py:11-34, the
// host routine: intersection / (|proposal| + |instance| - intersection), no epsilon, evaluated in double and stored as
// float32; other columns 0).  All tensors int64: instance_idx (sum of proposal sizes), instance_offsets (P + 1),
// gt_instances (N), gt_instance_sizes (sum of instances), num_gt_instances (samples), batch (N).
at::Tensor instance_iou(at::Tensor instance_idx, at::Tensor instance_offsets, at::Tensor gt_instances,
                        at::Tensor gt_instance_sizes, at::Tensor num_gt_instances, at::Tensor batch)
{
    for (const at::Tensor* t : {&instance_idx, &instance_offsets, &gt_instances, &gt_instance_sizes, &num_gt_instances, &batch})
        TORCH_CHECK(!t->is_cuda() && t->scalar_type() == at::kLong && t->dim() == 1, "1-D int64 CPU tensors expected");
    instance_idx = instance_idx.contiguous();
    instance_offsets = instance_offsets.contiguous();
    gt_instances = gt_instances.contiguous();
    gt_instance_sizes = gt_instance_sizes.contiguous();
    num_gt_instances = num_gt_instances.contiguous();
    batch = batch.contiguous();
    const int64_t proposals = instance_offsets.numel() - 1, points = gt_instances.numel(), samples = num_gt_instances.numel();
    TORCH_CHECK(proposals >= 0 && batch.numel() == points, "shapes do not match");
    const int64_t* count = num_gt_instances.data_ptr<int64_t>();
    std::vector<int64_t> first(static_cast<size_t>(samples + 1), 0);
    for (int64_t s = 0; s < samples; ++s)
    {
        TORCH_CHECK(count[s] >= 0, "negative instance count");
        first[static_cast<size_t>(s + 1)] = first[static_cast<size_t>(s)] + count[s];
    }
    const int64_t columns = first[static_cast<size_t>(samples)];
    TORCH_CHECK(gt_instance_sizes.numel() == columns, "one size per ground-truth instance expected");
    at::Tensor out = torch::zeros({proposals, columns}, torch::dtype(torch::kFloat));
    const int64_t* ii = instance_idx.data_ptr<int64_t>();
    const int64_t* off = instance_offsets.data_ptr<int64_t>();
    const int64_t* gt = gt_instances.data_ptr<int64_t>();
    const int64_t* size = gt_instance_sizes.data_ptr<int64_t>();
    const int64_t* bt = batch.data_ptr<int64_t>();
    float* o = out.data_ptr<float>();
    at::parallel_for(0, proposals, 1, [&](int64_t p0, int64_t p1) {
        std::vector<int64_t> hist;
        for (int64_t p = p0; p < p1; ++p)
        {
            const int64_t lo = off[p], hi = off[p + 1];
            TORCH_CHECK(lo >= 0 && hi >= lo && hi <= instance_idx.numel(), "instance_offsets outside instance_idx");
            if (hi == lo)
                continue;
            TORCH_CHECK(ii[lo] >= 0 && ii[lo] < points, "point index outside the cloud");
            const int64_t sample = bt[ii[lo]];
            TORCH_CHECK(sample >= 0 && sample < samples, "sample id outside num_gt_instances");
            const int64_t instances = count[sample];
            hist.assign(static_cast<size_t>(instances + 1), 0);
            for (int64_t e = lo; e < hi; ++e)
            {
                TORCH_CHECK(ii[e] >= 0 && ii[e] < points, "point index outside the cloud");
                const int64_t id = gt[ii[e]];
                if (id >= 1 && id <= instances)
                    ++hist[static_cast<size_t>(id)];
            }
            for (int64_t id = 1; id <= instances; ++id)
            {
                const int64_t col = first[static_cast<size_t>(sample)] + id - 1;
                const int64_t inter = hist[static_cast<size_t>(id)];
                o[p * columns + col] = static_cast<float>(static_cast<double>(inter) /
                                                          static_cast<double>((hi - lo) + size[col] - inter));
            }
        }
    });
    return out;
}

} // namespace

using namespace pybind11::literals;

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.doc() = "torch_points_kernels operators for CPU tensors (k-d tree searches, sampling, interpolation, region growing, IoU)";
    m.def("dense_knn", &dense_knn, "k nearest neighbours, dense layout", "support"_a, "querry"_a, "k"_a);
    m.def("knn_interpolate", &knn_interpolate, "weighted interpolation", "features"_a, "idx"_a, "weights"_a);
    m.def("knn_interpolate_grad", &knn_interpolate_grad, "gradient of the weighted interpolation", "grad_out"_a, "idx"_a,
          "weights"_a, "m"_a);
    m.def("fps", &fps, "furthest point sampling", "points"_a, "num_samples"_a, "random"_a);
    m.def("ball_query", &ball_query, "radius search in one cloud", "support"_a, "querry"_a, "radius"_a, "max_num"_a = -1,
          "mode"_a = 0, "sorted"_a = false);
    m.def("batch_ball_query", &batch_ball_query, "radius search, packed layout with sorted batch vectors", "support"_a,
          "querry"_a, "query_batch"_a, "support_batch"_a, "radius"_a, "max_num"_a = -1, "mode"_a = 0, "sorted"_a = false);
    m.def("dense_ball_query", &dense_ball_query, "radius search, dense layout", "support"_a, "querry"_a, "radius"_a,
          "max_num"_a = -1, "mode"_a = 0, "sorted"_a = false);
    m.def("grow_proximity", &grow_proximity, "region growing over a neighbour matrix", "neighbours"_a, "min_cluster_size"_a);
    m.def("instance_iou", &instance_iou, "IoU of proposals and ground-truth instances", "instance_idx"_a, "instance_offsets"_a,
          "gt_instances"_a, "gt_instance_sizes"_a, "num_gt_instances"_a, "batch"_a);
}

// k-d tree over one cloud of 3-D points, for the host-side operators that serve CPU tensors:
// radius search and k nearest neighbours.  No torch types here.
//
// Distances are (dx*dx + dy*dy) + dz*dz in the scalar type of the points, every operation
// rounded on its own (the translation unit is compiled -ffp-contract=off) - the same
// expression the reference's nanoflann adaptor accumulates (cpu/include/nanoflann.hpp:291-296,
// L2_Simple_Adaptor) and the GPU kernels of this package evaluate, so the three agree bit for bit.
//
// Pruning is exact in floating point: a subtree on the far side of a splitting plane is skipped
// only when the squared distance to the plane, computed with the same rounded operations, already
// rules its points out; rounding is monotonic, so no point whose computed distance qualifies is
// ever skipped.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <limits>
#include <vector>

namespace tpk_cpu {

template <typename T>
inline T squared_distance(const T* a, const T* b)
{
    const T dx = a[0] - b[0], dy = a[1] - b[1], dz = a[2] - b[2];
    return (dx * dx + dy * dy) + dz * dz;
}

// A neighbour candidate; ordered by distance, equal distances by index.  A distance that is not a number
// (a point or query with NaN, or inf - inf) counts as infinite, so that the order stays total: such
// candidates come last, by index.
template <typename T>
struct Neighbour
{
    T d2;
    int64_t index;
    static T rank(T v) { return std::isnan(v) ? std::numeric_limits<T>::infinity() : v; }
    bool operator<(const Neighbour& o) const
    {
        const T a = rank(d2), b = rank(o.d2);
        return a < b || (a == b && index < o.index);
    }
};

template <typename T>
class KdTree
{
  public:
    static constexpr int LEAF = 12; // points per leaf

    // points: n rows of (x, y, z); the tree keeps its own reordered copy.  Rows with a coordinate that is not
    // finite stay out of the tree (they cannot be ordered along an axis): they follow the tree's points, in
    // index order, no radius search ever reports them, and `nearest` offers them after the tree's points.
    KdTree(const T* points, int64_t n) : n_(n), finite_(0)
    {
        order_.resize(static_cast<size_t>(n));
        for (int64_t i = 0; i < n; ++i)
            if (std::isfinite(points[3 * i]) && std::isfinite(points[3 * i + 1]) && std::isfinite(points[3 * i + 2]))
                order_[static_cast<size_t>(finite_++)] = i;
        int64_t at = finite_;
        for (int64_t i = 0; i < n; ++i)
            if (!(std::isfinite(points[3 * i]) && std::isfinite(points[3 * i + 1]) && std::isfinite(points[3 * i + 2])))
                order_[static_cast<size_t>(at++)] = i;
        if (finite_ > 0)
        {
            nodes_.reserve(static_cast<size_t>(2 * (finite_ / LEAF + 1)));
            build(points, 0, finite_);
        }
        xyz_.resize(static_cast<size_t>(3 * n));
        for (int64_t i = 0; i < n; ++i)
            for (int d = 0; d < 3; ++d)
                xyz_[static_cast<size_t>(3 * i + d)] = points[3 * order_[static_cast<size_t>(i)] + d];
    }

    int64_t size() const { return n_; }

    // Calls visit(index, d2) for every point with d2 < r2 (strict), in no particular order.
    template <typename Visit>
    void within(const T* q, T r2, Visit&& visit) const
    {
        if (finite_ == 0)
            return;
        int stack[64];
        int top = 0;
        stack[top++] = 0;
        while (top > 0)
        {
            const Node& node = nodes_[static_cast<size_t>(stack[--top])];
            if (node.dim < 0)
            {
                for (int64_t i = node.lo; i < node.hi; ++i)
                {
                    const T d2 = squared_distance(q, &xyz_[static_cast<size_t>(3 * i)]);
                    if (d2 < r2)
                        visit(order_[static_cast<size_t>(i)], d2);
                }
                continue;
            }
            const T diff = q[node.dim] - node.split;
            const int near = diff < 0 ? node.left : node.right;
            const int far = diff < 0 ? node.right : node.left;
            if (diff * diff < r2)
                stack[top++] = far;
            stack[top++] = near;
        }
    }

    // The k nearest points by (distance, index), nearest first, into best[0 .. returned).
    // Returns min(k, size()).
    int64_t nearest(const T* q, int64_t k, Neighbour<T>* best) const
    {
        int64_t count = 0;
        if (n_ == 0 || k <= 0)
            return 0;
        struct Pending
        {
            int node;
            T bound; // squared distance to the plane that separates the query from this subtree
        };
        auto offer = [&](const Neighbour<T>& c) {
            if (count == k && !(c < best[k - 1]))
                return;
            int64_t at = count < k ? count++ : k - 1;
            while (at > 0 && c < best[at - 1])
            {
                best[at] = best[at - 1];
                --at;
            }
            best[at] = c;
        };
        Pending stack[64];
        int top = 0;
        if (finite_ > 0)
            stack[top++] = Pending{0, T(0)};
        while (top > 0)
        {
            const Pending p = stack[--top];
            // (an equal bound is still entered: a point at exactly that distance with a lower index would be kept)
            if (count == k && p.bound > best[k - 1].d2)
                continue;
            const Node& node = nodes_[static_cast<size_t>(p.node)];
            if (node.dim < 0)
            {
                for (int64_t i = node.lo; i < node.hi; ++i)
                    offer(Neighbour<T>{squared_distance(q, &xyz_[static_cast<size_t>(3 * i)]), order_[static_cast<size_t>(i)]});
                continue;
            }
            const T diff = q[node.dim] - node.split;
            const int near = diff < 0 ? node.left : node.right;
            const int far = diff < 0 ? node.right : node.left;
            stack[top++] = Pending{far, diff * diff};
            stack[top++] = Pending{near, T(0)};
        }
        for (int64_t i = finite_; i < n_; ++i) // the rows outside the tree
            offer(Neighbour<T>{squared_distance(q, &xyz_[static_cast<size_t>(3 * i)]), order_[static_cast<size_t>(i)]});
        return count;
    }

  private:
    struct Node
    {
        int64_t lo, hi; // leaf: its points in the reordered arrays
        int left, right;
        int dim; // -1: leaf
        T split;
    };

    // Builds the subtree over order_[lo, hi) and returns its node number.  Points left of the split have
    // coordinate <= split, points right of it >= split.  Depth stays below 64: ranges halve.
    int build(const T* points, int64_t lo, int64_t hi)
    {
        const int id = static_cast<int>(nodes_.size());
        nodes_.push_back(Node{lo, hi, -1, -1, -1, T(0)});
        if (hi - lo <= LEAF)
            return id;
        T low[3], high[3];
        for (int d = 0; d < 3; ++d)
        {
            low[d] = std::numeric_limits<T>::infinity();
            high[d] = -std::numeric_limits<T>::infinity();
        }
        for (int64_t i = lo; i < hi; ++i)
            for (int d = 0; d < 3; ++d)
            {
                const T v = points[3 * order_[static_cast<size_t>(i)] + d];
                low[d] = std::min(low[d], v);
                high[d] = std::max(high[d], v);
            }
        int dim = 0;
        for (int d = 1; d < 3; ++d)
            if (high[d] - low[d] > high[dim] - low[dim])
                dim = d;
        if (!(high[dim] - low[dim] > 0)) // all points equal (or not comparable): one leaf, however large
            return id;
        const int64_t mid = lo + (hi - lo) / 2;
        std::nth_element(order_.begin() + lo, order_.begin() + mid, order_.begin() + hi, [&](int64_t a, int64_t b) {
            return points[3 * a + dim] < points[3 * b + dim];
        });
        const T split = points[3 * order_[static_cast<size_t>(mid)] + dim];
        const int left = build(points, lo, mid);
        const int right = build(points, mid, hi);
        Node& node = nodes_[static_cast<size_t>(id)];
        node.left = left;
        node.right = right;
        node.dim = dim;
        node.split = split;
        return id;
    }

    int64_t n_;
    int64_t finite_; // the tree holds the first finite_ positions
    std::vector<int64_t> order_; // position in the tree's arrays -> index in the caller's cloud
    std::vector<T> xyz_;         // the points in tree order
    std::vector<Node> nodes_;
};

} // namespace tpk_cpu

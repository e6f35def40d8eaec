// torch_points_kernels.points_cuda for AMD MI355X: the pybind11 module the Python layer
// imports for tensors on the GPU.  It exports the names and signatures of the reference
// module (cuda/src/bindings.cpp:11-29) for the spatial-search operators, checks and
// allocates tensors the way the reference's host functions do, and hands raw pointers to
// the C ABI of libtpk_hip.so (include/tpk.h) on PyTorch's current HIP stream.  It contains
// no kernels and no CPU implementation: without a GPU tensor it raises.
#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <utility>
#include <vector>

#include "../../include/tpk.h"

namespace {

void check_status(int status, const char* what)
{
    TORCH_CHECK(status == TPK_OK, what, " failed: ", tpk_status_string(status), " (status ",
                status, ")");
}

// The reference's checks (cuda/include/utils.h:5-27) made stricter where it would misread
// memory: exact dtypes instead of "some float" / "some int".
void check_gpu(const at::Tensor& t, const char* name)
{
    TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
}
void check_contiguous(const at::Tensor& t, const char* name)
{
    TORCH_CHECK(t.is_contiguous(), name, " must be a contiguous tensor");
}
void check_f32(const at::Tensor& t, const char* name)
{
    TORCH_CHECK(t.scalar_type() == at::kFloat, name, " must be a float32 tensor");
}
void check_dtype(const at::Tensor& t, at::ScalarType st, const char* name)
{
    TORCH_CHECK(t.scalar_type() == st, name, " must be a ", c10::toString(st), " tensor");
}
void check_same_device(const at::Tensor& a, const at::Tensor& b, const char* names)
{
    TORCH_CHECK(a.device() == b.device(), names, " must be on the same device");
}
void check_points(const at::Tensor& t, int64_t dims, const char* name)
{
    TORCH_CHECK(t.dim() == dims && t.size(dims - 1) == 3, name, " must have shape (",
                dims == 3 ? "B, N, 3)" : "N, 3)");
}
int as_int(int64_t v, const char* name)
{
    TORCH_CHECK(v >= 0 && v <= INT32_MAX, name, " is out of range: ", v);
    return static_cast<int>(v);
}

void* current_stream(const at::Tensor& t)
{
    return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.get_device()).stream());
}

// cuda/src/sampling.cpp:8-25
at::Tensor furthest_point_sampling(at::Tensor points, const int nsamples)
{
    check_contiguous(points, "points");
    check_f32(points, "points");
    check_gpu(points, "points");
    check_points(points, 3, "points");
    TORCH_CHECK(nsamples >= 0, "nsamples must be non-negative");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(points.device());

    at::Tensor output = torch::empty({points.size(0), nsamples},
                                     at::device(points.device()).dtype(at::ScalarType::Int));
    const int b = as_int(points.size(0), "batch size");
    const int n = as_int(points.size(1), "number of points");
    const size_t ws_bytes = tpk_fps_workspace_bytes(b, n);
    at::Tensor ws;
    if (ws_bytes)
        ws = torch::empty({static_cast<int64_t>(ws_bytes)},
                          at::device(points.device()).dtype(at::ScalarType::Byte));
    check_status(tpk_fps_f32(b, n, nsamples, points.data_ptr<float>(),
                             ws_bytes ? ws.data_ptr() : nullptr, ws_bytes,
                             output.data_ptr<int32_t>(), current_stream(points)),
                 "furthest_point_sampling");
    return output;
}

// cuda/src/interpolate.cpp:12-32
std::vector<at::Tensor> three_nn(at::Tensor unknowns, at::Tensor knows)
{
    check_contiguous(unknowns, "unknowns");
    check_contiguous(knows, "knows");
    check_f32(unknowns, "unknowns");
    check_f32(knows, "knows");
    check_gpu(knows, "knows");
    check_gpu(unknowns, "unknowns");
    check_same_device(unknowns, knows, "unknowns and knows");
    check_points(unknowns, 3, "unknowns");
    check_points(knows, 3, "knows");
    TORCH_CHECK(unknowns.size(0) == knows.size(0), "unknowns and knows differ in batch size");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(unknowns.device());

    at::Tensor idx = torch::empty({unknowns.size(0), unknowns.size(1), 3},
                                  at::device(unknowns.device()).dtype(at::ScalarType::Int));
    at::Tensor dist2 = torch::empty({unknowns.size(0), unknowns.size(1), 3},
                                    at::device(unknowns.device()).dtype(at::ScalarType::Float));
    const int b = as_int(unknowns.size(0), "batch size");
    const int n = as_int(unknowns.size(1), "number of unknown points");
    const int m = as_int(knows.size(1), "number of known points");
    const size_t ws_bytes = tpk_three_nn_workspace_bytes(b, n, m);
    at::Tensor ws;
    if (ws_bytes)
        ws = torch::empty({static_cast<int64_t>(ws_bytes)}, unknowns.options().dtype(torch::kUInt8));
    check_status(tpk_three_nn_f32(b, n, m, unknowns.data_ptr<float>(), knows.data_ptr<float>(),
                                  dist2.data_ptr<float>(), idx.data_ptr<int32_t>(),
                                  ws_bytes ? ws.data_ptr() : nullptr, ws_bytes,
                                  current_stream(unknowns)),
                 "three_nn");
    return {dist2, idx};
}

// cpu/src/knn.cpp:43-62 (dense_knn; the reference has it for CPU tensors only)
std::pair<at::Tensor, at::Tensor> dense_knn(at::Tensor support, at::Tensor query, int64_t k)
{
    check_contiguous(support, "support");
    check_contiguous(query, "query");
    check_f32(support, "support");
    check_f32(query, "query");
    check_gpu(support, "support");
    check_gpu(query, "query");
    check_same_device(support, query, "support and query");
    check_points(support, 3, "support");
    check_points(query, 3, "query");
    TORCH_CHECK(support.size(0) == query.size(0), "support and query differ in batch size");
    TORCH_CHECK(k >= 0, "k must not be negative");
    // cpu/src/knn.cpp:12-14
    TORCH_CHECK(support.size(1) >= k, "Not enough points in support to find " + std::to_string(k) + " neighboors");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(support.device());

    at::Tensor idx = torch::empty({query.size(0), query.size(1), k},
                                  at::device(query.device()).dtype(at::ScalarType::Long));
    at::Tensor dist2 = torch::empty({query.size(0), query.size(1), k},
                                    at::device(query.device()).dtype(at::ScalarType::Float));
    const int b = as_int(query.size(0), "batch size");
    const int n = as_int(support.size(1), "number of support points");
    const int m = as_int(query.size(1), "number of query points");
    const size_t ws_bytes = tpk_knn_workspace_bytes(b, n, m);
    at::Tensor ws;
    if (ws_bytes)
        ws = torch::empty({static_cast<int64_t>(ws_bytes)}, query.options().dtype(torch::kUInt8));
    check_status(tpk_knn_f32(b, n, m, as_int(k, "k"), support.data_ptr<float>(), query.data_ptr<float>(),
                             idx.data_ptr<int64_t>(), dist2.data_ptr<float>(),
                             ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, current_stream(query)),
                 "dense_knn");
    return std::make_pair(idx, dist2);
}

// torch_points_kernels/cluster.py:9-37 (_grow_proximity_core; host code in the reference)
// -> (members, starts): clusters one after the other and their offsets (one more than clusters).
std::pair<at::Tensor, at::Tensor> grow_proximity(at::Tensor neighbours, int64_t min_cluster_size,
                                                 bool reference_order)
{
    check_contiguous(neighbours, "neighbours");
    check_dtype(neighbours, at::kLong, "neighbours");
    check_gpu(neighbours, "neighbours");
    TORCH_CHECK(neighbours.dim() == 2, "neighbours must have shape (N, nsample)");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(neighbours.device());
    const int64_t n = neighbours.size(0);
    auto options = at::device(neighbours.device()).dtype(at::ScalarType::Long);
    at::Tensor members = torch::empty({n}, options);
    at::Tensor starts = torch::empty({n + 1}, options);
    int64_t found[2] = {0, 0};
    if (n > 0)
    {
        const size_t ws_bytes = tpk_grow_proximity_workspace_bytes(n, as_int(neighbours.size(1), "nsample"));
        TORCH_CHECK(ws_bytes > 0, "grow_proximity: too many points");
        at::Tensor ws = torch::empty({static_cast<int64_t>(ws_bytes)}, options.dtype(torch::kUInt8));
        check_status(tpk_grow_proximity(n, as_int(neighbours.size(1), "nsample"), neighbours.data_ptr<int64_t>(),
                                        min_cluster_size,
                                        reference_order ? TPK_MEMBERS_AS_REFERENCE : TPK_MEMBERS_BY_INDEX,
                                        members.data_ptr<int64_t>(), starts.data_ptr<int64_t>(), found,
                                        ws.data_ptr(), ws_bytes, current_stream(neighbours)),
                     "grow_proximity");
    }
    if (found[0] == 0)
        return std::make_pair(members.narrow(0, 0, 0), torch::zeros({1}, options));
    return std::make_pair(members.narrow(0, 0, found[1]), starts.narrow(0, 0, found[0] + 1));
}

// cuda/src/interpolate.cpp:34-54
at::Tensor three_interpolate(at::Tensor points, at::Tensor idx, at::Tensor weight)
{
    check_contiguous(points, "points");
    check_contiguous(idx, "idx");
    check_contiguous(weight, "weight");
    check_f32(points, "points");
    check_dtype(idx, at::kInt, "idx");
    check_f32(weight, "weight");
    check_gpu(points, "points");
    check_gpu(idx, "idx");
    check_gpu(weight, "weight");
    check_same_device(points, idx, "points and idx");
    check_same_device(points, weight, "points and weight");
    TORCH_CHECK(points.dim() == 3, "points must have shape (B, c, m)");
    TORCH_CHECK(idx.dim() == 3 && idx.size(2) == 3 && idx.size(0) == points.size(0),
                "idx must have shape (B, n, 3)");
    TORCH_CHECK(weight.sizes() == idx.sizes(), "weight must have the shape of idx");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(points.device());

    at::Tensor output = torch::empty({points.size(0), points.size(1), idx.size(1)},
                                     at::device(points.device()).dtype(at::ScalarType::Float));
    check_status(tpk_three_interpolate_f32(
                     as_int(points.size(0), "batch size"), as_int(points.size(1), "channels"),
                     as_int(points.size(2), "m"), as_int(idx.size(1), "n"),
                     points.data_ptr<float>(), idx.data_ptr<int32_t>(), weight.data_ptr<float>(),
                     output.data_ptr<float>(), current_stream(points)),
                 "three_interpolate");
    return output;
}

// cuda/src/interpolate.cpp:55-76
at::Tensor three_interpolate_grad(at::Tensor grad_out, at::Tensor idx, at::Tensor weight,
                                  const int m)
{
    check_contiguous(grad_out, "grad_out");
    check_contiguous(idx, "idx");
    check_contiguous(weight, "weight");
    check_f32(grad_out, "grad_out");
    check_dtype(idx, at::kInt, "idx");
    check_f32(weight, "weight");
    check_gpu(idx, "idx");
    check_gpu(weight, "weight");
    check_gpu(grad_out, "grad_out");
    check_same_device(grad_out, idx, "grad_out and idx");
    check_same_device(grad_out, weight, "grad_out and weight");
    TORCH_CHECK(grad_out.dim() == 3, "grad_out must have shape (B, c, n)");
    TORCH_CHECK(idx.dim() == 3 && idx.size(2) == 3 && idx.size(0) == grad_out.size(0) &&
                    idx.size(1) == grad_out.size(2),
                "idx must have shape (B, n, 3)");
    TORCH_CHECK(weight.sizes() == idx.sizes(), "weight must have the shape of idx");
    TORCH_CHECK(m >= 0, "m must be non-negative");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(grad_out.device());

    at::Tensor output = torch::empty({grad_out.size(0), grad_out.size(1), m},
                                     at::device(grad_out.device()).dtype(at::ScalarType::Float));
    const int b = as_int(grad_out.size(0), "batch size");
    const int n = as_int(grad_out.size(2), "n");
    const size_t ws_bytes = tpk_three_interpolate_grad_workspace_bytes(b, n, m);
    at::Tensor ws = torch::empty({static_cast<int64_t>(ws_bytes)},
                                 at::device(grad_out.device()).dtype(at::ScalarType::Byte));
    check_status(tpk_three_interpolate_grad_f32(
                     b, as_int(grad_out.size(1), "channels"), n, m, grad_out.data_ptr<float>(),
                     idx.data_ptr<int32_t>(), weight.data_ptr<float>(), output.data_ptr<float>(),
                     ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, current_stream(grad_out)),
                 "three_interpolate_grad");
    return output;
}

// three_interpolate for a caller that will ask for the gradient (autograd is recording): with the forward
// pass the index is inverted into the per-target lists that the backward pass walks (include/tpk.h,
// tpk_three_interpolate_lists_f32), so that the backward pass is the walk alone and several backward passes
// share one inversion.  Returns (output, lists); `lists` is empty where the list path does not serve the shape
// (then three_interpolate_grad is the backward pass).  No counterpart in the reference, whose backward scatters
// with atomics.  (Inverting on a second stream beside the gather was measured: the two event waits between the
// streams cost more than the 18 us they hide - 198 us per call against 52 us one after the other.)
std::pair<at::Tensor, at::Tensor> three_interpolate_recording(at::Tensor points, at::Tensor idx, at::Tensor weight)
{
    check_contiguous(idx, "idx");
    check_contiguous(weight, "weight");
    check_gpu(points, "points");
    check_gpu(idx, "idx");
    check_gpu(weight, "weight");
    check_dtype(idx, at::kInt, "idx");
    check_f32(weight, "weight");
    TORCH_CHECK(points.dim() == 3 && idx.dim() == 3 && idx.size(2) == 3 && weight.sizes() == idx.sizes(),
                "points (B, c, m), idx and weight (B, n, 3) expected");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(points.device());
    const int b = as_int(idx.size(0), "batch size"), n = as_int(idx.size(1), "n"), m = as_int(points.size(2), "m");
    const size_t bytes = tpk_three_interpolate_grad_workspace_bytes(b, n, m);
    if (bytes == 0)
        return {three_interpolate(points, idx, weight), torch::empty({0}, at::device(points.device()).dtype(at::kByte))};
    at::Tensor lists = torch::empty({static_cast<int64_t>(bytes)}, at::device(points.device()).dtype(at::kByte));
    at::Tensor output = three_interpolate(points, idx, weight);
    check_status(tpk_three_interpolate_lists_f32(b, n, m, idx.data_ptr<int32_t>(), weight.data_ptr<float>(), lists.data_ptr(),
                                                 bytes, current_stream(points)),
                 "three_interpolate (lists for the backward pass)");
    return {output, lists};
}

// The backward pass over the lists three_interpolate_recording() returned.
at::Tensor three_interpolate_grad_lists(at::Tensor grad_out, at::Tensor lists, const int m)
{
    check_contiguous(grad_out, "grad_out");
    check_f32(grad_out, "grad_out");
    check_gpu(grad_out, "grad_out");
    check_gpu(lists, "lists");
    check_same_device(grad_out, lists, "grad_out and lists");
    TORCH_CHECK(grad_out.dim() == 3, "grad_out must have shape (B, c, n)");
    TORCH_CHECK(lists.scalar_type() == at::kByte && lists.is_contiguous() && m >= 0, "lists as three_interpolate_recording returned them");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(grad_out.device());
    at::Tensor output = torch::empty({grad_out.size(0), grad_out.size(1), m}, at::device(grad_out.device()).dtype(at::kFloat));
    check_status(tpk_three_interpolate_grad_lists_f32(as_int(grad_out.size(0), "batch size"), as_int(grad_out.size(1), "channels"),
                                                      as_int(grad_out.size(2), "n"), m, grad_out.data_ptr<float>(),
                                                      lists.data_ptr(), static_cast<size_t>(lists.numel()),
                                                      output.data_ptr<float>(), current_stream(grad_out)),
                 "three_interpolate_grad (from lists)");
    return output;
}

// cuda/src/ball_query.cpp:15-36.  Query centres first, as in the reference.
// sorted: the nsample nearest neighbours within the radius, nearest first (what the reference
// computes for CPU tensors with sort=True, cpu/src/ball_query.cpp:127-146).
std::pair<at::Tensor, at::Tensor> ball_query_dense(at::Tensor new_xyz, at::Tensor xyz,
                                                   const float radius, const int nsample, const bool sorted)
{
    check_contiguous(new_xyz, "new_xyz");
    check_contiguous(xyz, "xyz");
    check_f32(new_xyz, "new_xyz");
    check_f32(xyz, "xyz");
    check_gpu(xyz, "xyz");
    check_gpu(new_xyz, "new_xyz");
    check_same_device(xyz, new_xyz, "xyz and new_xyz");
    check_points(new_xyz, 3, "new_xyz");
    check_points(xyz, 3, "xyz");
    TORCH_CHECK(xyz.size(0) == new_xyz.size(0), "xyz and new_xyz differ in batch size");
    TORCH_CHECK(nsample >= 0, "nsample must be non-negative");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(new_xyz.device());

    at::Tensor idx = torch::empty({new_xyz.size(0), new_xyz.size(1), nsample},
                                  at::device(new_xyz.device()).dtype(at::ScalarType::Long));
    at::Tensor dist = torch::empty({new_xyz.size(0), new_xyz.size(1), nsample},
                                   at::device(new_xyz.device()).dtype(at::ScalarType::Float));
    if (sorted)
    {
        const int b = as_int(xyz.size(0), "batch size"), n = as_int(xyz.size(1), "support points");
        const int m = as_int(new_xyz.size(1), "query points");
        const size_t ws_bytes = tpk_ball_query_sorted_dense_workspace_bytes(b, n, m);
        at::Tensor ws;
        if (ws_bytes)
            ws = torch::empty({static_cast<int64_t>(ws_bytes)}, new_xyz.options().dtype(torch::kUInt8));
        check_status(tpk_ball_query_sorted_dense_f32(b, n, m, radius, nsample, new_xyz.data_ptr<float>(),
                                                     xyz.data_ptr<float>(), idx.data_ptr<int64_t>(),
                                                     dist.data_ptr<float>(), ws_bytes ? ws.data_ptr() : nullptr,
                                                     ws_bytes, current_stream(new_xyz)),
                     "ball_query_dense (sorted)");
        return std::make_pair(idx, dist);
    }
    {
        const int b = as_int(xyz.size(0), "batch size"), n = as_int(xyz.size(1), "support points");
        const int m = as_int(new_xyz.size(1), "query points");
        const size_t ws_bytes = tpk_ball_query_dense_workspace_bytes(b, n, m, nsample);
        at::Tensor ws;
        if (ws_bytes)
            ws = torch::empty({static_cast<int64_t>(ws_bytes)}, new_xyz.options().dtype(torch::kUInt8));
        check_status(tpk_ball_query_dense_ws_f32(b, n, m, radius, nsample, new_xyz.data_ptr<float>(), xyz.data_ptr<float>(),
                                                 idx.data_ptr<int64_t>(), dist.data_ptr<float>(),
                                                 ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, current_stream(new_xyz)),
                     "ball_query_dense");
    }
    return std::make_pair(idx, dist);
}

// cuda/src/ball_query.cpp:45-81.  Support first, as in the reference.  The cloud ranges
// are found on the device from the sorted batch vectors; nothing is copied to the host.
std::pair<at::Tensor, at::Tensor> ball_query_partial_dense(at::Tensor x, at::Tensor y,
                                                           at::Tensor batch_x, at::Tensor batch_y,
                                                           const float radius, const int nsample, const bool sorted)
{
    check_contiguous(x, "x");
    check_contiguous(y, "y");
    check_f32(x, "x");
    check_f32(y, "y");
    check_gpu(x, "x");
    check_gpu(y, "y");
    check_gpu(batch_x, "batch_x");
    check_gpu(batch_y, "batch_y");
    check_same_device(x, y, "x and y");
    check_same_device(x, batch_x, "x and batch_x");
    check_same_device(x, batch_y, "x and batch_y");
    check_points(x, 2, "x");
    check_points(y, 2, "y");
    check_dtype(batch_x, at::kLong, "batch_x");
    check_dtype(batch_y, at::kLong, "batch_y");
    TORCH_CHECK(batch_x.dim() == 1 && batch_x.size(0) == x.size(0),
                "batch_x must have one entry per point of x");
    TORCH_CHECK(batch_y.dim() == 1 && batch_y.size(0) == y.size(0),
                "batch_y must have one entry per point of y");
    TORCH_CHECK(nsample >= 0, "nsample must be non-negative");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    batch_x = batch_x.contiguous();
    batch_y = batch_y.contiguous();

    at::Tensor idx =
        torch::empty({y.size(0), nsample}, at::device(y.device()).dtype(at::ScalarType::Long));
    at::Tensor dist =
        torch::empty({y.size(0), nsample}, at::device(y.device()).dtype(at::ScalarType::Float));
    if (sorted)
    {
        // cpu/src/ball_query.cpp:65-124 with sorted = true
        const size_t sorted_ws_bytes = tpk_ball_query_sorted_partial_workspace_bytes(x.size(0), y.size(0));
        at::Tensor sorted_ws;
        if (sorted_ws_bytes)
            sorted_ws = torch::empty({static_cast<int64_t>(sorted_ws_bytes)}, x.options().dtype(torch::kUInt8));
        check_status(tpk_ball_query_sorted_partial_f32(x.size(0), y.size(0), radius, nsample, x.data_ptr<float>(),
                                                       y.data_ptr<float>(), batch_x.data_ptr<int64_t>(),
                                                       batch_y.data_ptr<int64_t>(), idx.data_ptr<int64_t>(),
                                                       dist.data_ptr<float>(),
                                                       sorted_ws_bytes ? sorted_ws.data_ptr() : nullptr, sorted_ws_bytes,
                                                       current_stream(x)),
                     "ball_query_partial_dense (sorted)");
        return std::make_pair(idx, dist);
    }
    const size_t ws_bytes = tpk_ball_query_partial_workspace_bytes(x.size(0), y.size(0), nsample);
    at::Tensor ws;
    if (ws_bytes)
        ws = torch::empty({static_cast<int64_t>(ws_bytes)}, x.options().dtype(torch::kUInt8));
    check_status(tpk_ball_query_partial_f32(x.size(0), y.size(0), radius, nsample,
                                            x.data_ptr<float>(), y.data_ptr<float>(),
                                            batch_x.data_ptr<int64_t>(),
                                            batch_y.data_ptr<int64_t>(), idx.data_ptr<int64_t>(),
                                            dist.data_ptr<float>(), ws_bytes ? ws.data_ptr() : nullptr,
                                            ws_bytes, current_stream(x)),
                 "ball_query_partial_dense");
    return std::make_pair(idx, dist);
}

// cuda/src/metrics.cpp:12-52
at::Tensor instance_iou_cuda(at::Tensor instance_idx, at::Tensor instance_offsets, at::Tensor gt_instances,
                             at::Tensor gt_instance_sizes, at::Tensor num_gt_instances, at::Tensor batch)
{
    const at::Tensor* all[] = {&instance_idx, &instance_offsets, &gt_instances, &gt_instance_sizes, &num_gt_instances, &batch};
    const char* names[] = {"instance_idx", "instance_offsets", "gt_instances", "gt_instance_sizes", "num_gt_instances", "batch"};
    for (int i = 0; i < 6; ++i)
    {
        check_contiguous(*all[i], names[i]);
        check_gpu(*all[i], names[i]);
        check_dtype(*all[i], at::kLong, names[i]);
        check_same_device(*all[i], gt_instances, names[i]);
        TORCH_CHECK(all[i]->dim() == 1, names[i], " must have one dimension");
    }
    TORCH_CHECK(instance_offsets.size(0) >= 1, "instance_offsets must hold at least one entry");
    TORCH_CHECK(batch.size(0) == gt_instances.size(0), "batch and gt_instances differ in length");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(gt_instances.device());
    const int64_t num_proposed_instances = instance_offsets.size(0) - 1;
    // as the reference: the total is read back to size the output
    const int64_t total_gt_instances = num_gt_instances.numel() ? num_gt_instances.sum().item<int64_t>() : 0;
    TORCH_CHECK(gt_instance_sizes.size(0) == total_gt_instances, "gt_instance_sizes must hold one entry per ground-truth instance");
    at::Tensor output = torch::empty({num_proposed_instances, total_gt_instances},
                                     at::device(gt_instances.device()).dtype(at::ScalarType::Float));
    at::Tensor offset_num_gt_instances = at::cat({at::zeros(1, num_gt_instances.options()), num_gt_instances.cumsum(0)}, 0);
    check_status(tpk_instance_iou(total_gt_instances, num_proposed_instances, gt_instances.size(0), num_gt_instances.size(0),
                                  num_gt_instances.data_ptr<int64_t>(), instance_idx.data_ptr<int64_t>(),
                                  instance_offsets.data_ptr<int64_t>(), gt_instances.data_ptr<int64_t>(),
                                  offset_num_gt_instances.data_ptr<int64_t>(), batch.data_ptr<int64_t>(),
                                  gt_instance_sizes.data_ptr<int64_t>(), output.data_ptr<float>(),
                                  current_stream(gt_instances)),
                 "instance_iou_cuda");
    return output;
}

// cuda/src/gridding.cpp:4-12 -> {grid_weights, grid_pt_weights, grid_pt_indexes}
std::vector<at::Tensor> gridding(float min_x, float max_x, float min_y, float max_y, float min_z, float max_z,
                                 at::Tensor ptcloud)
{
    check_gpu(ptcloud, "ptcloud");
    check_contiguous(ptcloud, "ptcloud");
    TORCH_CHECK(ptcloud.scalar_type() == at::kFloat || ptcloud.scalar_type() == at::kDouble,
                "ptcloud must be float32 or float64");
    TORCH_CHECK(ptcloud.dim() == 3 && ptcloud.size(2) == 3, "ptcloud must have shape (B, n_pts, 3)");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(ptcloud.device());
    const int b = as_int(ptcloud.size(0), "batch size"), n = as_int(ptcloud.size(1), "number of points");
    const int64_t len_x = static_cast<int>(max_x - min_x + 1), len_y = static_cast<int>(max_y - min_y + 1);
    const int64_t len_z = static_cast<int>(max_z - min_z + 1);
    TORCH_CHECK(len_x > 0 && len_y > 0 && len_z > 0, "gridding: empty grid");
    at::Tensor grid = torch::empty({b, len_x * len_y * len_z}, ptcloud.options());
    at::Tensor weights = torch::empty({b, n, 8, 3}, ptcloud.options());
    at::Tensor indexes = torch::empty({b, n, 8}, ptcloud.options().dtype(at::kInt));
    if (ptcloud.scalar_type() == at::kFloat)
        check_status(tpk_gridding_f32(b, n, min_x, max_x, min_y, max_y, min_z, max_z, ptcloud.data_ptr<float>(),
                                      grid.data_ptr<float>(), weights.data_ptr<float>(), indexes.data_ptr<int32_t>(),
                                      current_stream(ptcloud)),
                     "gridding");
    else
        check_status(tpk_gridding_f64(b, n, min_x, max_x, min_y, max_y, min_z, max_z, ptcloud.data_ptr<double>(),
                                      grid.data_ptr<double>(), weights.data_ptr<double>(), indexes.data_ptr<int32_t>(),
                                      current_stream(ptcloud)),
                     "gridding");
    return {grid, weights, indexes};
}

// cuda/src/gridding.cpp:14-26
at::Tensor gridding_grad(at::Tensor grid_pt_weights, at::Tensor grid_pt_indexes, at::Tensor grad_grid)
{
    check_gpu(grid_pt_weights, "grid_pt_weights");
    check_gpu(grid_pt_indexes, "grid_pt_indexes");
    check_gpu(grad_grid, "grad_grid");
    check_contiguous(grid_pt_weights, "grid_pt_weights");
    check_contiguous(grid_pt_indexes, "grid_pt_indexes");
    check_contiguous(grad_grid, "grad_grid");
    check_dtype(grid_pt_indexes, at::kInt, "grid_pt_indexes");
    TORCH_CHECK(grid_pt_weights.scalar_type() == at::kFloat || grid_pt_weights.scalar_type() == at::kDouble,
                "grid_pt_weights must be float32 or float64");
    TORCH_CHECK(grad_grid.scalar_type() == grid_pt_weights.scalar_type(), "grad_grid and grid_pt_weights differ in dtype");
    TORCH_CHECK(grid_pt_indexes.dim() == 3 && grid_pt_indexes.size(2) == 8, "grid_pt_indexes must have shape (B, n_pts, 8)");
    TORCH_CHECK(grid_pt_weights.dim() == 4 && grid_pt_weights.size(0) == grid_pt_indexes.size(0) &&
                    grid_pt_weights.size(1) == grid_pt_indexes.size(1) && grid_pt_weights.size(2) == 8 &&
                    grid_pt_weights.size(3) == 3,
                "grid_pt_weights must have shape (B, n_pts, 8, 3)");
    TORCH_CHECK(grad_grid.dim() == 2 && grad_grid.size(0) == grid_pt_indexes.size(0), "grad_grid must have shape (B, n_grid_vertices)");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(grad_grid.device());
    const int b = as_int(grad_grid.size(0), "batch size"), n = as_int(grid_pt_indexes.size(1), "number of points");
    const int vertices = as_int(grad_grid.size(1), "grid vertices");
    at::Tensor grad = torch::empty({b, n, 3}, grid_pt_weights.options());
    if (grid_pt_weights.scalar_type() == at::kFloat)
        check_status(tpk_gridding_grad_f32(b, n, vertices, grid_pt_weights.data_ptr<float>(),
                                           grid_pt_indexes.data_ptr<int32_t>(), grad_grid.data_ptr<float>(),
                                           grad.data_ptr<float>(), current_stream(grad_grid)),
                     "gridding_grad");
    else
        check_status(tpk_gridding_grad_f64(b, n, vertices, grid_pt_weights.data_ptr<double>(),
                                           grid_pt_indexes.data_ptr<int32_t>(), grad_grid.data_ptr<double>(),
                                           grad.data_ptr<double>(), current_stream(grad_grid)),
                     "gridding_grad");
    return grad;
}

// cuda/src/cubic_feature_sampling.cpp:4-16 -> {point_features, grid_pt_indexes}
std::vector<at::Tensor> cubic_feature_sampling(int scale, int neighborhood_size, at::Tensor ptcloud,
                                               at::Tensor cubic_features)
{
    check_gpu(ptcloud, "ptcloud");
    check_gpu(cubic_features, "cubic_features");
    check_contiguous(ptcloud, "ptcloud");
    check_contiguous(cubic_features, "cubic_features");
    check_same_device(ptcloud, cubic_features, "ptcloud and cubic_features");
    TORCH_CHECK(ptcloud.scalar_type() == at::kFloat || ptcloud.scalar_type() == at::kDouble,
                "ptcloud must be float32 or float64");
    TORCH_CHECK(cubic_features.scalar_type() == ptcloud.scalar_type(), "ptcloud and cubic_features differ in dtype");
    TORCH_CHECK(ptcloud.dim() == 3 && ptcloud.size(2) == 3, "ptcloud must have shape (B, n_pts, 3)");
    TORCH_CHECK(cubic_features.dim() == 5 && cubic_features.size(0) == ptcloud.size(0) && cubic_features.size(2) == scale &&
                    cubic_features.size(3) == scale && cubic_features.size(4) == scale,
                "cubic_features must have shape (B, c, scale, scale, scale)");
    TORCH_CHECK(neighborhood_size >= 1 && neighborhood_size <= 64, "neighborhood_size out of range");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(ptcloud.device());
    const int b = as_int(ptcloud.size(0), "batch size"), n = as_int(ptcloud.size(1), "number of points");
    const int channels = as_int(cubic_features.size(1), "channels");
    const int64_t side = 2 * static_cast<int64_t>(neighborhood_size), vertices = side * side * side;
    at::Tensor features = torch::empty({b, n, vertices, channels}, ptcloud.options());
    at::Tensor indexes = torch::empty({b, n, vertices}, ptcloud.options().dtype(at::kInt));
    if (ptcloud.scalar_type() == at::kFloat)
        check_status(tpk_cubic_feature_sampling_f32(b, n, channels, scale, neighborhood_size, ptcloud.data_ptr<float>(),
                                                    cubic_features.data_ptr<float>(), features.data_ptr<float>(),
                                                    indexes.data_ptr<int32_t>(), current_stream(ptcloud)),
                     "cubic_feature_sampling");
    else
        check_status(tpk_cubic_feature_sampling_f64(b, n, channels, scale, neighborhood_size, ptcloud.data_ptr<double>(),
                                                    cubic_features.data_ptr<double>(), features.data_ptr<double>(),
                                                    indexes.data_ptr<int32_t>(), current_stream(ptcloud)),
                     "cubic_feature_sampling");
    return {features, indexes};
}

// cuda/src/cubic_feature_sampling.cpp:18-30 -> {grad_ptcloud, grad_cubic_features}
std::vector<at::Tensor> cubic_feature_sampling_grad(int scale, int neighborhood_size, at::Tensor grad_point_features,
                                                    at::Tensor grid_pt_indexes)
{
    check_gpu(grad_point_features, "grad_point_features");
    check_gpu(grid_pt_indexes, "grid_pt_indexes");
    check_contiguous(grad_point_features, "grad_point_features");
    check_contiguous(grid_pt_indexes, "grid_pt_indexes");
    check_dtype(grid_pt_indexes, at::kInt, "grid_pt_indexes");
    TORCH_CHECK(grad_point_features.scalar_type() == at::kFloat || grad_point_features.scalar_type() == at::kDouble,
                "grad_point_features must be float32 or float64");
    TORCH_CHECK(neighborhood_size >= 1 && neighborhood_size <= 64, "neighborhood_size out of range");
    TORCH_CHECK(scale > 0, "scale must be positive");
    const int64_t side = 2 * static_cast<int64_t>(neighborhood_size), vertices = side * side * side;
    TORCH_CHECK(grid_pt_indexes.dim() == 3 && grid_pt_indexes.size(2) == vertices, "grid_pt_indexes must have shape (B, n_pts, n_vertices)");
    TORCH_CHECK(grad_point_features.dim() == 4 && grad_point_features.size(0) == grid_pt_indexes.size(0) &&
                    grad_point_features.size(1) == grid_pt_indexes.size(1) && grad_point_features.size(2) == vertices,
                "grad_point_features must have shape (B, n_pts, n_vertices, c)");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(grad_point_features.device());
    const int b = as_int(grad_point_features.size(0), "batch size"), n = as_int(grid_pt_indexes.size(1), "number of points");
    const int channels = as_int(grad_point_features.size(3), "channels");
    at::Tensor grad_ptcloud = torch::empty({b, n, 3}, grad_point_features.options());
    at::Tensor grad_cubic = torch::empty({b, channels, scale, scale, scale}, grad_point_features.options());
    if (grad_point_features.scalar_type() == at::kFloat)
        check_status(tpk_cubic_feature_sampling_grad_f32(b, n, channels, scale, neighborhood_size,
                                                         grad_point_features.data_ptr<float>(),
                                                         grid_pt_indexes.data_ptr<int32_t>(), grad_ptcloud.data_ptr<float>(),
                                                         grad_cubic.data_ptr<float>(), current_stream(grad_point_features)),
                     "cubic_feature_sampling_grad");
    else
        check_status(tpk_cubic_feature_sampling_grad_f64(b, n, channels, scale, neighborhood_size,
                                                         grad_point_features.data_ptr<double>(),
                                                         grid_pt_indexes.data_ptr<int32_t>(), grad_ptcloud.data_ptr<double>(),
                                                         grad_cubic.data_ptr<double>(), current_stream(grad_point_features)),
                     "cubic_feature_sampling_grad");
    return {grad_ptcloud, grad_cubic};
}

// No counterpart in the reference's native module: its grouping_operation is
// torch.gather on a repeated index (torch_points_kernels/torchpoints.py:129-146).
at::Tensor grouping_operation(at::Tensor features, at::Tensor idx)
{
    check_contiguous(features, "features");
    check_contiguous(idx, "idx");
    check_f32(features, "features");
    check_dtype(idx, at::kLong, "idx");
    check_gpu(features, "features");
    check_gpu(idx, "idx");
    check_same_device(features, idx, "features and idx");
    TORCH_CHECK(features.dim() == 3, "features must have shape (B, C, N)");
    TORCH_CHECK(idx.dim() == 3 && idx.size(0) == features.size(0),
                "idx must have shape (B, npoint, nsample)");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(features.device());

    at::Tensor out = torch::empty({features.size(0), features.size(1), idx.size(1), idx.size(2)},
                                  at::device(features.device()).dtype(at::ScalarType::Float));
    check_status(tpk_group_f32(as_int(features.size(0), "batch size"),
                               as_int(features.size(1), "channels"), as_int(features.size(2), "N"),
                               as_int(idx.size(1), "npoint"), as_int(idx.size(2), "nsample"),
                               features.data_ptr<float>(), idx.data_ptr<int64_t>(),
                               out.data_ptr<float>(), current_stream(features)),
                 "grouping_operation");
    return out;
}

at::Tensor grouping_operation_grad(at::Tensor grad_out, at::Tensor idx, const int n)
{
    check_contiguous(grad_out, "grad_out");
    check_contiguous(idx, "idx");
    check_f32(grad_out, "grad_out");
    check_dtype(idx, at::kLong, "idx");
    check_gpu(grad_out, "grad_out");
    check_gpu(idx, "idx");
    check_same_device(grad_out, idx, "grad_out and idx");
    TORCH_CHECK(grad_out.dim() == 4, "grad_out must have shape (B, C, npoint, nsample)");
    TORCH_CHECK(idx.dim() == 3 && idx.size(0) == grad_out.size(0) &&
                    idx.size(1) == grad_out.size(2) && idx.size(2) == grad_out.size(3),
                "idx must have shape (B, npoint, nsample)");
    TORCH_CHECK(n >= 0, "n must be non-negative");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(grad_out.device());

    at::Tensor out = torch::empty({grad_out.size(0), grad_out.size(1), n},
                                  at::device(grad_out.device()).dtype(at::ScalarType::Float));
    const int b = as_int(grad_out.size(0), "batch size");
    const int npoint = as_int(idx.size(1), "npoint");
    const int nsample = as_int(idx.size(2), "nsample");
    const size_t ws_bytes = tpk_group_grad_workspace_bytes(b, n, npoint, nsample);
    at::Tensor ws = torch::empty({static_cast<int64_t>(ws_bytes)},
                                 at::device(grad_out.device()).dtype(at::ScalarType::Byte));
    check_status(tpk_group_grad_f32(b, as_int(grad_out.size(1), "channels"), n, npoint, nsample,
                                    grad_out.data_ptr<float>(), idx.data_ptr<int64_t>(),
                                    out.data_ptr<float>(), ws_bytes ? ws.data_ptr() : nullptr,
                                    ws_bytes, current_stream(grad_out)),
                 "grouping_operation_grad");
    return out;
}

// grouping_operation for a caller that will ask for the gradient: as three_interpolate_recording.
std::pair<at::Tensor, at::Tensor> grouping_operation_recording(at::Tensor features, at::Tensor idx)
{
    check_contiguous(idx, "idx");
    check_gpu(features, "features");
    check_gpu(idx, "idx");
    check_dtype(idx, at::kLong, "idx");
    TORCH_CHECK(features.dim() == 3 && idx.dim() == 3, "features (B, C, N) and idx (B, npoint, nsample) expected");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(features.device());
    const int b = as_int(idx.size(0), "batch size"), n = as_int(features.size(2), "N");
    const int npoint = as_int(idx.size(1), "npoint"), nsample = as_int(idx.size(2), "nsample");
    const size_t bytes = tpk_group_grad_workspace_bytes(b, n, npoint, nsample);
    if (bytes == 0)
        return {grouping_operation(features, idx), torch::empty({0}, at::device(features.device()).dtype(at::kByte))};
    at::Tensor lists = torch::empty({static_cast<int64_t>(bytes)}, at::device(features.device()).dtype(at::kByte));
    at::Tensor output = grouping_operation(features, idx);
    check_status(tpk_group_lists(b, n, npoint, nsample, idx.data_ptr<int64_t>(), lists.data_ptr(), bytes, current_stream(features)),
                 "grouping_operation (lists for the backward pass)");
    return {output, lists};
}

at::Tensor grouping_operation_grad_lists(at::Tensor grad_out, at::Tensor lists, const int n)
{
    check_contiguous(grad_out, "grad_out");
    check_f32(grad_out, "grad_out");
    check_gpu(grad_out, "grad_out");
    check_gpu(lists, "lists");
    check_same_device(grad_out, lists, "grad_out and lists");
    TORCH_CHECK(grad_out.dim() == 4, "grad_out must have shape (B, C, npoint, nsample)");
    TORCH_CHECK(lists.scalar_type() == at::kByte && lists.is_contiguous() && n >= 0, "lists as grouping_operation_recording returned them");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(grad_out.device());
    at::Tensor out = torch::empty({grad_out.size(0), grad_out.size(1), n}, at::device(grad_out.device()).dtype(at::kFloat));
    check_status(tpk_group_grad_lists_f32(as_int(grad_out.size(0), "batch size"), as_int(grad_out.size(1), "channels"), n,
                                          as_int(grad_out.size(2), "npoint"), as_int(grad_out.size(3), "nsample"),
                                          grad_out.data_ptr<float>(), lists.data_ptr(), static_cast<size_t>(lists.numel()),
                                          out.data_ptr<float>(), current_stream(grad_out)),
                 "grouping_operation_grad (from lists)");
    return out;
}

// cuda/src/chamfer_dist.cpp:3-6 -> cuda/src/chamfer_dist_gpu.cu:157-184
std::vector<torch::Tensor> chamfer_dist(torch::Tensor xyz1, torch::Tensor xyz2)
{
    check_gpu(xyz1, "xyz1");
    check_gpu(xyz2, "xyz2");
    check_same_device(xyz1, xyz2, "xyz1 and xyz2");
    check_points(xyz1, 3, "xyz1");
    check_points(xyz2, 3, "xyz2");
    TORCH_CHECK(xyz1.size(0) == xyz2.size(0), "xyz1 and xyz2 differ in batch size");
    TORCH_CHECK(xyz1.scalar_type() == xyz2.scalar_type(), "xyz1 and xyz2 differ in dtype");
    TORCH_CHECK(xyz1.scalar_type() == at::kFloat || xyz1.scalar_type() == at::kDouble,
                "chamfer_dist supports float32 and float64");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(xyz1.device());
    xyz1 = xyz1.contiguous();
    xyz2 = xyz2.contiguous();

    const int b = as_int(xyz1.size(0), "batch size");
    const int n = as_int(xyz1.size(1), "points of xyz1");
    const int m = as_int(xyz2.size(1), "points of xyz2");
    auto fopt = xyz1.options();
    auto iopt = xyz1.options().dtype(torch::kInt);
    torch::Tensor dist1 = torch::empty({b, n}, fopt);
    torch::Tensor dist2 = torch::empty({b, m}, fopt);
    torch::Tensor idx1 = torch::empty({b, n}, iopt);
    torch::Tensor idx2 = torch::empty({b, m}, iopt);
    void* s = current_stream(xyz1);
    if (xyz1.scalar_type() == at::kFloat)
    {
        const size_t ws_bytes = tpk_chamfer_fwd_workspace_bytes(b, n, m);
        torch::Tensor ws;
        if (ws_bytes)
            ws = torch::empty({static_cast<int64_t>(ws_bytes)}, xyz1.options().dtype(torch::kUInt8));
        check_status(tpk_chamfer_fwd_f32(b, n, m, xyz1.data_ptr<float>(), xyz2.data_ptr<float>(),
                                         dist1.data_ptr<float>(), dist2.data_ptr<float>(),
                                         idx1.data_ptr<int32_t>(), idx2.data_ptr<int32_t>(),
                                         ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, s),
                     "chamfer_dist");
    }
    else
        check_status(tpk_chamfer_fwd_f64(b, n, m, xyz1.data_ptr<double>(),
                                         xyz2.data_ptr<double>(), dist1.data_ptr<double>(),
                                         dist2.data_ptr<double>(), idx1.data_ptr<int32_t>(),
                                         idx2.data_ptr<int32_t>(), s),
                     "chamfer_dist");
    return {dist1, dist2, idx1, idx2};
}

// cuda/src/chamfer_dist.cpp:8-13 -> cuda/src/chamfer_dist_gpu.cu:215-245
std::vector<torch::Tensor> chamfer_dist_grad(torch::Tensor xyz1, torch::Tensor xyz2,
                                             torch::Tensor idx1, torch::Tensor idx2,
                                             torch::Tensor grad_dist1, torch::Tensor grad_dist2)
{
    check_gpu(xyz1, "xyz1");
    check_gpu(xyz2, "xyz2");
    check_gpu(idx1, "idx1");
    check_gpu(idx2, "idx2");
    check_gpu(grad_dist1, "grad_dist1");
    check_gpu(grad_dist2, "grad_dist2");
    check_points(xyz1, 3, "xyz1");
    check_points(xyz2, 3, "xyz2");
    check_dtype(idx1, at::kInt, "idx1");
    check_dtype(idx2, at::kInt, "idx2");
    TORCH_CHECK(xyz1.scalar_type() == xyz2.scalar_type() &&
                    xyz1.scalar_type() == grad_dist1.scalar_type() &&
                    xyz1.scalar_type() == grad_dist2.scalar_type(),
                "clouds and gradients differ in dtype");
    TORCH_CHECK(xyz1.scalar_type() == at::kFloat || xyz1.scalar_type() == at::kDouble,
                "chamfer_dist_grad supports float32 and float64");
    const int b = as_int(xyz1.size(0), "batch size");
    const int n = as_int(xyz1.size(1), "points of xyz1");
    const int m = as_int(xyz2.size(1), "points of xyz2");
    TORCH_CHECK(xyz2.size(0) == b && idx1.numel() == static_cast<int64_t>(b) * n &&
                    idx2.numel() == static_cast<int64_t>(b) * m &&
                    grad_dist1.numel() == idx1.numel() && grad_dist2.numel() == idx2.numel(),
                "shapes of clouds, indices and gradients do not match");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(xyz1.device());
    xyz1 = xyz1.contiguous();
    xyz2 = xyz2.contiguous();
    idx1 = idx1.contiguous();
    idx2 = idx2.contiguous();
    grad_dist1 = grad_dist1.contiguous();
    grad_dist2 = grad_dist2.contiguous();

    torch::Tensor grad_xyz1 = torch::empty_like(xyz1);
    torch::Tensor grad_xyz2 = torch::empty_like(xyz2);
    const size_t ws_bytes = tpk_chamfer_bwd_workspace_bytes(b, n, m);
    torch::Tensor ws = torch::empty({static_cast<int64_t>(ws_bytes)}, xyz1.options().dtype(torch::kByte));
    void* wsp = ws_bytes ? ws.data_ptr() : nullptr;
    void* s = current_stream(xyz1);
    if (xyz1.scalar_type() == at::kFloat)
        check_status(tpk_chamfer_bwd_f32(b, n, m, xyz1.data_ptr<float>(), xyz2.data_ptr<float>(),
                                         idx1.data_ptr<int32_t>(), idx2.data_ptr<int32_t>(),
                                         grad_dist1.data_ptr<float>(),
                                         grad_dist2.data_ptr<float>(),
                                         grad_xyz1.data_ptr<float>(),
                                         grad_xyz2.data_ptr<float>(), wsp, ws_bytes, s),
                     "chamfer_dist_grad");
    else
        check_status(tpk_chamfer_bwd_f64(b, n, m, xyz1.data_ptr<double>(),
                                         xyz2.data_ptr<double>(), idx1.data_ptr<int32_t>(),
                                         idx2.data_ptr<int32_t>(), grad_dist1.data_ptr<double>(),
                                         grad_dist2.data_ptr<double>(),
                                         grad_xyz1.data_ptr<double>(),
                                         grad_xyz2.data_ptr<double>(), wsp, ws_bytes, s),
                     "chamfer_dist_grad");
    return {grad_xyz1, grad_xyz2};
}

} // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("furthest_point_sampling", &furthest_point_sampling);
    m.def("three_nn", &three_nn);
    m.def("dense_knn", &dense_knn);
    m.def("grow_proximity", &grow_proximity);
    m.def("instance_iou_cuda", &instance_iou_cuda);
    m.def("gridding", &gridding);
    m.def("gridding_grad", &gridding_grad);
    m.def("cubic_feature_sampling", &cubic_feature_sampling);
    m.def("cubic_feature_sampling_grad", &cubic_feature_sampling_grad);
    m.def("three_interpolate", &three_interpolate);
    m.def("three_interpolate_grad", &three_interpolate_grad);
    m.def("three_interpolate_recording", &three_interpolate_recording);
    m.def("three_interpolate_grad_lists", &three_interpolate_grad_lists);
    m.def("ball_query_dense", &ball_query_dense, pybind11::arg("new_xyz"), pybind11::arg("xyz"), pybind11::arg("radius"),
          pybind11::arg("nsample"), pybind11::arg("sorted") = false);
    m.def("ball_query_partial_dense", &ball_query_partial_dense, pybind11::arg("x"), pybind11::arg("y"),
          pybind11::arg("batch_x"), pybind11::arg("batch_y"), pybind11::arg("radius"), pybind11::arg("nsample"),
          pybind11::arg("sorted") = false);
    m.def("grouping_operation", &grouping_operation);
    m.def("grouping_operation_grad", &grouping_operation_grad);
    m.def("grouping_operation_recording", &grouping_operation_recording);
    m.def("grouping_operation_grad_lists", &grouping_operation_grad_lists);
    m.def("chamfer_dist", &chamfer_dist);
    m.def("chamfer_dist_grad", &chamfer_dist_grad);
    m.def("tpk_version", &tpk_version);
}

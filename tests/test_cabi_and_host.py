"""CPU-only checks of the drop-in boundary: the C-ABI library exports what include/tpk.h
declares, the Python layer mirrors the reference's error behaviour, and nothing falls back
to a CPU implementation."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tpk.h")
LIB = os.path.join(ROOT, "torch-points-kernels_amd", "torch_points_kernels", "libtpk_hip.so")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tpk_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_symbols()
    for want in (
        "tpk_fps_f32", "tpk_fps_workspace_bytes", "tpk_ball_query_dense_f32", "tpk_ball_query_dense_workspace_bytes", "tpk_ball_query_dense_ws_f32", "tpk_ball_query_partial_workspace_bytes", "tpk_ball_query_partial_f32",
        "tpk_three_nn_workspace_bytes", "tpk_three_nn_f32", "tpk_knn_workspace_bytes", "tpk_knn_f32", "tpk_three_interpolate_f32", "tpk_three_interpolate_grad_f32", "tpk_group_f32",
        "tpk_three_interpolate_lists_f32", "tpk_three_interpolate_grad_lists_f32", "tpk_group_lists", "tpk_group_grad_lists_f32",
        "tpk_group_grad_f32", "tpk_chamfer_fwd_workspace_bytes", "tpk_chamfer_fwd_f32", "tpk_chamfer_fwd_f64", "tpk_chamfer_bwd_f32",
        "tpk_chamfer_bwd_f64", "tpk_grow_proximity_workspace_bytes", "tpk_grow_proximity", "tpk_instance_iou", "tpk_gridding_f32", "tpk_gridding_f64", "tpk_gridding_grad_f32",
        "tpk_gridding_grad_f64", "tpk_cubic_feature_sampling_f32", "tpk_cubic_feature_sampling_f64",
        "tpk_cubic_feature_sampling_grad_f32", "tpk_cubic_feature_sampling_grad_f64", "tpk_ball_query_sorted_dense_workspace_bytes",
        "tpk_ball_query_sorted_dense_f32", "tpk_ball_query_sorted_partial_workspace_bytes", "tpk_ball_query_sorted_partial_f32", "tpk_status_string", "tpk_version",
    ):
        assert want in names


def test_counting_build_exports_the_same_abi_plus_its_reader():
    """libtpk_hip_counting.so (measurement only) carries the whole C ABI and tpk_work_read_reset; the
    shipping library carries no counter."""
    path = LIB.replace("libtpk_hip.so", "libtpk_hip_counting.so")
    assert os.path.exists(path), "libtpk_hip_counting.so is not built (run torch-points-kernels_amd/build.py)"
    lib = ctypes.CDLL(path)
    for name in _declared_symbols() + ["tpk_work_read_reset"]:
        assert hasattr(lib, name), name
    assert not hasattr(ctypes.CDLL(LIB), "tpk_work_read_reset")
    text = open(os.path.join(ROOT, "include", "tpk_counting.h")).read()
    assert "tpk_work_read_reset" in text


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "libtpk_hip.so is not built (run torch-points-kernels_amd/build.py)"
    lib = ctypes.CDLL(LIB)
    for name in _declared_symbols():
        assert hasattr(lib, name), name
    lib.tpk_status_string.restype = ctypes.c_char_p
    assert lib.tpk_status_string(0) == b"ok"
    assert b"invalid" in lib.tpk_status_string(-1)
    assert lib.tpk_version() >= 100
    lib.tpk_fps_workspace_bytes.restype = ctypes.c_size_t
    assert lib.tpk_fps_workspace_bytes(4, 16384) == 0
    # 16385..163840 points: records (16 B), boxes (160 B per cell of 64) and minima (4 B) of whole windows of 16384
    # and, for the coarse order in front: a record (16 B) and a place (4 B) per point, and per chunk of 16384 points
    # of the batch two clouds' spans (16 B), boxes (48 B) and counts (2 x 4096 x 4 B), every array a multiple of 256 B
    up = lambda v: (v + 255) // 256 * 256
    chunks = (4 * 50000 + 16383) // 16384
    coarse = up(4 * 50000 * 16) + up(4 * 50000 * 4) + up(chunks * 16) + up(chunks * 48) + up(chunks * 2 * 4096 * 4)
    assert lib.tpk_fps_workspace_bytes(4, 50000) == 4 * 4 * 256 * (64 * 16 + 160 + 64 * 4) + coarse
    assert lib.tpk_fps_workspace_bytes(2, 200000) == 2 * 200000 * 4  # larger: the minima only
    # searches over curve-ordered cells: 16 bytes per point padded to cells of 64, 160 bytes per cell;
    # 0 = the shape is served by the all-pairs scan, no workspace wanted
    for name in ("tpk_three_nn_workspace_bytes", "tpk_chamfer_fwd_workspace_bytes", "tpk_knn_workspace_bytes"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_size_t
        assert fn(2, 100, 100) == 0 and fn(2, 200000, 1000) == 0 and fn(0, 1000, 1000) == 0
        # (the Chamfer search also keeps the cells of every window in the order it hands them out: 4 bytes per cell)
        order = ((11, 4), (15, 4)) if "chamfer" in name else ()
        want = sum(-(-2 * c * nbytes // 256) * 256 for c, nbytes in ((11, 1024), (15, 1024), (11, 160), (15, 160)) + order)
        # (three_nn: one word per cloud at the end, for the clouds that a kernel in front has not answered)
        flags = 256 if "three_nn" in name else 0
        assert fn(2, 700, 900) == want + flags
        # clouds above 16384 points: whole windows of 16384 points (256 cells each)
        order = ((512, 4), (15, 4)) if "chamfer" in name else ()
        want = sum(-(-2 * c * nbytes // 256) * 256 for c, nbytes in ((512, 1024), (15, 1024), (512, 160), (15, 160)) + order)
        assert fn(2, 20000, 900) == want + flags
    up = lambda v: -(-v // 256) * 256
    # sorted ball query (b, support points, queries): only the support points are ordered when one wavefront serves a
    # query (up to 64 neighbours); the size also covers the k-nearest lists that serve more neighbours
    fn = lib.tpk_ball_query_sorted_dense_workspace_bytes
    fn.restype = ctypes.c_size_t
    cells = lambda n: -(-n // 64) if n <= 16384 else -(-n // 16384) * 256
    # records (1024 B per cell of 64), cell boxes (160 B), boxes of runs of 16 cells (32 B)
    support_only = lambda b, n: up(b * cells(n) * 1024) + up(b * cells(n) * 160) + up(b * -(-cells(n) // 16) * 32)
    assert fn(2, 100, 5000) == 0 and fn(0, 1000, 1000) == 0
    assert fn(2, 4096, 100) == support_only(2, 4096)
    assert fn(2, 200000, 1000) == support_only(2, 200000)
    assert fn(2, 700, 900) == sum(-(-2 * c * nbytes // 256) * 256 for c, nbytes in ((11, 1024), (15, 1024), (11, 160), (15, 160)))
    # list-based backward passes, per cloud part (a part = up to 32768 columns): 16 regions (16 B each), the first
    # target of 16 x 64 lanes (4 B each), and entry slots for every index entry, one empty entry per target, the
    # rounding to rows of 64 and the gaps between the 16 regions (8 B weighted, 4 B plain)
    slots = lambda m, total: -(-(total + m) // 64) * 64 + 128 * 16 + 64
    lists = lambda parts, m, total, size: up(parts * 16 * 16) + up(parts * 16 * 64 * 4) + up(parts * slots(m, total) * size)
    lib.tpk_three_interpolate_grad_workspace_bytes.restype = ctypes.c_size_t
    assert lib.tpk_three_interpolate_grad_workspace_bytes(2, 1000, 100) == lists(2, 100, 3000, 8)
    # 20000 columns: one part of 20000 columns (rows go one at a time)
    assert lib.tpk_three_interpolate_grad_workspace_bytes(1, 20000, 64) == lists(1, 64, 60000, 8)
    # 40000 columns: two parts of 32768 columns
    assert lib.tpk_three_interpolate_grad_workspace_bytes(1, 40000, 64) == lists(2, 64, 3 * 32768, 8)
    lib.tpk_group_grad_workspace_bytes.restype = ctypes.c_size_t
    assert lib.tpk_group_grad_workspace_bytes(3, 70, 16, 8) == lists(3, 70, 128, 4)
    lib.tpk_chamfer_bwd_workspace_bytes.restype = ctypes.c_size_t
    # the Chamfer backward keeps its chains in LDS: no workspace
    assert lib.tpk_chamfer_bwd_workspace_bytes(2, 300, 515) == 0
    assert lib.tpk_chamfer_bwd_workspace_bytes(0, 300, 515) == 0
    lib.tpk_ball_query_partial_workspace_bytes.restype = ctypes.c_size_t
    lib.tpk_ball_query_partial_workspace_bytes.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
    assert lib.tpk_ball_query_partial_workspace_bytes(8191, 100, 16) == 0
    assert lib.tpk_ball_query_partial_workspace_bytes(40000, 100, 0) == 0
    windows = 5  # 40000 support points in windows of 8192 (arrays of at most 64 such windows)
    assert lib.tpk_ball_query_partial_workspace_bytes(40000, 100, 16) == windows * (8192 * 16 + 4096 * 4) + 256 + 1024  # + the queries' cloud rows, 8 bytes each
    windows = 37  # 600000 support points: windows of 16384
    assert lib.tpk_ball_query_partial_workspace_bytes(600000, 100, 16) == windows * (16384 * 16 + 4096 * 4) + 1280 + 1024


def test_argument_errors_are_reported_without_a_gpu():
    lib = ctypes.CDLL(LIB)
    null = ctypes.c_void_p(0)
    # negative sizes / missing pointers are rejected before anything is launched
    assert lib.tpk_three_nn_f32(-1, 4, 4, null, null, null, null, null) == -1
    assert lib.tpk_three_nn_f32(1, 4, 4, null, null, null, null, null) == -1
    assert lib.tpk_ball_query_dense_f32(1, 4, 4, ctypes.c_float(0.1), -3, null, null, null, null, null) == -1
    assert lib.tpk_fps_f32(1, 4, 2, null, null, ctypes.c_size_t(0), null, null) == -1
    # empty problems succeed trivially
    assert lib.tpk_three_nn_f32(0, 4, 4, null, null, null, null, null) == 0
    found = (ctypes.c_int64 * 2)(5, 5)
    grow = lib.tpk_grow_proximity
    grow.argtypes = [ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int] + [ctypes.c_void_p] * 4 + [
        ctypes.c_size_t, ctypes.c_void_p]
    assert grow(0, 16, None, 1, 0, None, None, found, None, 0, None) == 0 and list(found) == [0, 0]
    assert grow(-1, 16, None, 1, 0, None, None, found, None, 0, None) == -1
    assert grow(5, 16, None, 1, 0, None, None, found, None, 0, None) == -1  # no arrays
    assert grow(0, 16, None, 1, 7, None, None, found, None, 0, None) == -1  # unknown member order
    assert grow(0, 16, None, 1, 0, None, None, None, None, 0, None) == -1  # nowhere to report the counts
    assert lib.tpk_group_f32(0, 1, 1, 1, 1, null, null, null, null) == 0


def test_python_api_errors_match_the_reference(tpk):
    x = torch.zeros(2, 10, 3)
    # reference torchpoints.py:32-33
    with pytest.raises(ValueError):
        tpk.furthest_point_sample(x, 11)
    # reference torchpoints.py:57-58
    with pytest.raises(ValueError):
        tpk.three_nn(torch.zeros(1, 2, 3), x[:1])
    # reference torchpoints.py:201-218
    with pytest.raises(Exception, match="mode should be defined"):
        tpk.ball_query(0.1, 4, x, x, mode=None)
    with pytest.raises(Exception, match="should be provided"):
        tpk.ball_query(0.1, 4, x[0], x[0], mode="partial_dense")
    with pytest.raises(Exception, match="should not be provided"):
        tpk.ball_query(0.1, 4, x, x, mode="dense", batch_x=torch.zeros(10).long())
    with pytest.raises(Exception, match="unrecognized mode"):
        tpk.ball_query(0.1, 4, x, x, mode="sparse")
    with pytest.raises(AssertionError):
        tpk.ball_query(0.1, 4, x[0], x[0], mode="DENSE")
    with pytest.raises(AssertionError):
        tpk.ball_query(0.1, 4, x[0], x[0], mode="PARTIAL_DENSE", batch_x=torch.zeros(3).long(),
                       batch_y=torch.zeros(10).long())
    # reference chamfer_dist.py:43-44 and :10-11
    from torch_points_kernels.chamfer_dist import ChamferFunction, chamfer_dist

    with pytest.raises(ValueError):
        chamfer_dist(torch.zeros(4, 3), torch.zeros(1, 4, 3))
    with pytest.raises(NotImplementedError):
        ChamferFunction.apply(x, x)


def test_tensors_are_served_by_the_module_of_their_device(tpk, monkeypatch):
    """CPU tensors go to points_cpu, never to the HIP extension; and a GPU tensor whose extension is missing raises
    instead of being served by the host module (checked by making the loader fail: the dispatch looks at is_cuda only)."""
    from torch_points_kernels import _native, torchpoints

    x = torch.rand(1, 16, 3)
    idx, dist = tpk.ball_query(0.5, 4, x, x, sort=True)
    assert idx.dtype == torch.int64 and not idx.is_cuda and idx[0, :, 0].tolist() == list(range(16))
    assert tpk.furthest_point_sample(x, 4).dtype == torch.int64  # the reference's CPU convention
    assert tpk.three_nn(x, x)[1].dtype == torch.int64

    class FakeGpuTensor:
        is_cuda = True
        shape = (1, 16, 3)

    def missing():
        raise ImportError("points_cuda is not built")

    monkeypatch.setattr(torchpoints, "native", missing)
    monkeypatch.setattr(torchpoints, "host", lambda: pytest.fail("a GPU tensor must not reach the host module"))
    with pytest.raises(ImportError):
        tpk.furthest_point_sample(FakeGpuTensor(), 4)
    with pytest.raises(ImportError):
        torchpoints.ball_query_dense(0.5, 4, FakeGpuTensor(), FakeGpuTensor())
    with pytest.raises(ImportError):
        torchpoints.ball_query_partial_dense(0.5, 4, FakeGpuTensor(), FakeGpuTensor(), None, None)
    assert _native.native is not missing


def test_gpu_only_operators_raise_for_cpu_tensors_and_bad_shapes(tpk):
    from torch_points_kernels.cluster import grow_proximity, region_grow
    from torch_points_kernels.cubic_feature_sampling import cubic_feature_sampling
    from torch_points_kernels.gridding import gridding
    from torch_points_kernels.metrics import instance_iou

    pos = torch.rand(20, 3)
    batch = torch.zeros(20, dtype=torch.long)
    with pytest.raises(AssertionError):
        region_grow(pos, torch.zeros(20, 1, dtype=torch.long), batch)  # reference cluster.py:71
    with pytest.raises(ValueError):
        grow_proximity(pos, batch, member_order="sorted")
    # the operators the reference has no CPU path for refuse CPU tensors (reference: chamfer_dist.py:10-11; its
    # gridding.py and cubic_feature_sampling.py call the CUDA module unconditionally)
    with pytest.raises(NotImplementedError):
        gridding(torch.rand(1, 10, 3), 4)
    with pytest.raises(NotImplementedError):
        cubic_feature_sampling(torch.rand(1, 10, 3), torch.rand(1, 2, 4, 4, 4))
    # reference gridding.py:50-51, cubic_feature_sampling.py:53-54
    with pytest.raises(ValueError):
        gridding(torch.rand(10, 3), 4)
    with pytest.raises(ValueError):
        cubic_feature_sampling(torch.rand(10, 3), torch.rand(1, 2, 4, 4, 4))
    with pytest.raises(NotImplementedError):
        gridding(torch.rand(1, 10, 3), 4)
    with pytest.raises(NotImplementedError):
        cubic_feature_sampling(torch.rand(1, 10, 3), torch.rand(1, 2, 4, 4, 4))


def test_product_package_does_not_reference_the_oracle():
    pkg = os.path.join(ROOT, "torch-points-kernels_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.sep + "build" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_bench_line_is_short_and_parses():
    """bench.py prints ONE line; a harness that keeps only the end of the output must still find all of it.
    Built here from canned numbers (no GPU): 18 operators with long workload texts and notes."""
    import json

    import bench

    prose = "x" * 900
    roof_f = {"bound": "mfma", "achieved": 0.578912345, "peak": 157.3, "unit": "TFLOP/s", "frac": 0.0036801234,
              "traffic": 3779123.0, "executed_pairs": 86222336, "algorithmic_pairs": 1073479680,
              "algorithmic_rate": 7.2081234, "algorithmic_speedup": 12.45, "note": prose,
              "valu": {"valu_busy_pct": 4.3, "valu_lane_utilisation_pct": 75.8, "source": prose, "measured_at_commit": "abc"}}
    roof_b = {"bound": "hbm", "achieved": 2394.123456, "peak": 8000.0, "unit": "GB/s", "frac": 0.299265432,
              "traffic": 242912345.0, "traffic_source": prose, "traffic_measured_at_commit": "abc", "note": prose}
    cpu = {"value": 5894.123456, "unit": "ms/batch", "cores": 16, "kind": "reference", "sample": prose}
    fps = {"wall_ms": 1.4968812345, "kernel_ms": 1.489371234, "roofline": roof_f, "cpu_baseline": cpu}
    full = bench.headline_object(fps, 20, 3, "AMD Instinct MI355X")
    full["ops"] = {}
    for i, name in enumerate(bench.OPS_ORDER):
        e = {"workload": prose, "metric": "queries/s", "value": 1.23456789e9, "kernel_ms": 0.0123456789, "wall_ms": 0.02,
             "roofline": dict(roof_f if i % 2 else roof_b), "algorithmic_bytes": 174063616, "pairs": 1 << 30,
             "cpu_baseline": dict(cpu, unit="queries/s")}
        if i % 3 == 0:
            e["all_pairs_kernel"] = {"what": prose, "kernel_ms": 1.116123, "wall_ms": 1.2, "roofline": dict(roof_f)}
        full["ops"][name] = e
    text = bench.compact_line(full, bench.DETAIL_FILE)
    assert "\n" not in text and len(text) < 4096, len(text)
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["value"] == line["ms_per_step"] == 1.49688
    assert set(line["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"}
    assert line["roofline"]["bound"] in ("hbm", "mfma") and "note" not in line["roofline"]
    assert set(line["cpu_baseline"]) == {"value", "unit", "cores", "kind", "sample"} and line["cpu_baseline"]["cores"] == 16
    assert list(line["ops"]) == list(bench.OPS_ORDER) and "ops_dropped" not in line
    assert line["ops"]["three_interpolate_bwd"]["ms"] == 0.01235
    # a line that would be too long sheds the operators outside the BASELINE configurations first
    short = json.loads(bench.compact_line(full, bench.DETAIL_FILE, limit=2600))
    assert short["ops_dropped"] > 0 and "ball_query_dense" in short["ops"] and "roofline" in short

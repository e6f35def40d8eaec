"""Loader of the native module (points_cuda.so, built in-tree by ../build.py).

There is no CPU implementation behind this package: an operator called with a tensor that
is not on the GPU raises, and so does every operator when the native module has not been
built.  Nothing here falls back to PyTorch ops.
"""
import importlib

_module = None


def native():
    global _module
    if _module is None:
        try:
            _module = importlib.import_module("torch_points_kernels.points_cuda")
        except ImportError as e:  # pragma: no cover - depends on the build
            raise ImportError(
                "torch_points_kernels.points_cuda (the HIP extension) is not built or cannot be "
                "loaded; run `python build.py` in torch-points-kernels_amd/. Original error: %s" % e
            ) from e
    return _module


def require_gpu(tensor, op):
    if not tensor.is_cuda:
        raise NotImplementedError(
            "%s: this build implements the GPU (HIP) path only; got a tensor on %s" % (op, tensor.device)
        )

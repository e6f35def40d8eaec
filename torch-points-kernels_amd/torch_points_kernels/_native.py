"""Loaders of the two native modules (built in-tree by ../build.py).

points_cuda: the HIP kernels behind the C ABI; serves tensors on the GPU.
points_cpu:  host C++ (k-d tree searches, sampling, interpolation); serves tensors in host memory,
             as the reference's module of that name does.

A tensor is served by the module of its own device, never by the other one: a GPU tensor whose
extension is missing raises ImportError, it does not fall back to the host.  Nothing here falls
back to PyTorch ops either.
"""
import importlib

_modules = {}


def _load(name, what):
    mod = _modules.get(name)
    if mod is None:
        try:
            mod = importlib.import_module("torch_points_kernels." + name)
        except ImportError as e:  # pragma: no cover - depends on the build
            raise ImportError(
                "torch_points_kernels.%s (%s) is not built or cannot be loaded; run `python build.py` in "
                "torch-points-kernels_amd/. Original error: %s" % (name, what, e)
            ) from e
        _modules[name] = mod
    return mod


def native():
    """The HIP extension."""
    return _load("points_cuda", "the HIP extension")


def host():
    """The module for CPU tensors."""
    return _load("points_cpu", "the module for CPU tensors")


def require_gpu(tensor, op):
    if not tensor.is_cuda:
        raise NotImplementedError("%s has no CPU implementation; got a tensor on %s" % (op, tensor.device))

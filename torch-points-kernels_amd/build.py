"""Build the native parts in-tree, for gfx950 only.

  csrc/*.hip          -> torch_points_kernels/libtpk_hip.so   (HIP kernels + C ABI, no torch)
  csrc/points_cuda.cpp -> torch_points_kernels/points_cuda.so  (pybind11 module over the C ABI)
  csrc/points_cpu.cpp  -> torch_points_kernels/points_cpu.so   (operators for CPU tensors; host code only, no HIP)
  csrc/*.hip          -> torch_points_kernels/libtpk_hip_counting.so: the same library with the
                         distance scans compiled -DTPK_COUNT_WORK (they count the pair
                         evaluations they execute; include/tpk_counting.h).  Measurement only:
                         the package never loads it.

Run as ``python build.py`` (add ``--force`` to rebuild everything).  hipcc cross-compiles, so
no GPU is needed to build.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
PKG = os.path.join(HERE, "torch_points_kernels")
OBJ = os.path.join(HERE, "build")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# -ffp-contract=off: products and sums round separately (integer outputs depend on it).
# -packed-fp32-ops: packed fp32 VALU instructions are not to be generated.
# -simplifycfg-sink-common=false: keeps the arms of wave-uniform branches that pick one element
#   of a register-resident array from being merged into one indexed access, which would move
#   the whole array to scratch memory (fps.hip).
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-simplifycfg-sink-common=false",
    "-Wall", "-Wno-unused-function", "-I" + INCLUDE,
]


def _newer(target, deps):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


# Translation units that hold distance scans (and the counters' reader): compiled a second time
# with -DTPK_COUNT_WORK for the counting library; the other objects are shared.
COUNTING_UNITS = ("status", "ball_query", "three_nn", "chamfer", "nn_grid", "fps")


def build_kernels(force=False):
    os.makedirs(OBJ, exist_ok=True)
    headers = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(INCLUDE, "*.h"))
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    lib = os.path.join(PKG, "libtpk_hip.so")
    counting_lib = os.path.join(PKG, "libtpk_hip_counting.so")
    jobs = []
    objs = []
    counting_objs = []
    for src in sources:
        unit = os.path.basename(src)[:-4]
        obj = os.path.join(OBJ, unit + ".o")
        objs.append(obj)
        if force or not _newer(obj, [src] + headers):
            jobs.append([HIPCC] + HIP_FLAGS + ["-c", src, "-o", obj])
        if unit in COUNTING_UNITS:
            obj = os.path.join(OBJ, unit + ".counting.o")
            if force or not _newer(obj, [src] + headers):
                jobs.append([HIPCC] + HIP_FLAGS + ["-DTPK_COUNT_WORK", "-c", src, "-o", obj])
        counting_objs.append(obj)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for out in ex.map(_run, jobs):
            if out.strip():
                print(out)
    if force or jobs or not _newer(lib, objs):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    if force or jobs or not _newer(counting_lib, counting_objs):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", counting_lib] + counting_objs)
    return lib


def build_extension(force=False):
    import torch
    from torch.utils import cpp_extension

    src = os.path.join(CSRC, "points_cuda.cpp")
    out = os.path.join(PKG, "points_cuda.so")
    deps = [src, os.path.join(INCLUDE, "tpk.h")]
    if not force and _newer(out, deps):
        return out
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=points_cuda",
           "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in cpp_extension.include_paths() + [sysconfig.get_paths()["include"],
                                                 os.path.join(ROCM, "include"), INCLUDE]:
        cmd.append("-I" + inc)
    cmd += [src, "-o", out,
            "-L" + PKG, "-ltpk_hip", "-Wl,-rpath,$ORIGIN",
            "-L" + torch_lib, "-Wl,-rpath," + torch_lib,
            "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            "-L" + os.path.join(ROCM, "lib"), "-Wl,-rpath," + os.path.join(ROCM, "lib"),
            "-lamdhip64"]
    _run(cmd)
    return out


def build_cpu_extension(force=False):
    """The module that serves CPU tensors: plain host C++ (g++), linked against torch only."""
    import torch
    from torch.utils import cpp_extension

    src = os.path.join(CSRC, "points_cpu.cpp")
    out = os.path.join(PKG, "points_cpu.so")
    deps = [src] + glob.glob(os.path.join(CSRC, "cpu", "*.h"))
    if not force and _newer(out, deps):
        return out
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    # -ffp-contract=off: distances round every operation on its own, as in the GPU kernels
    cmd = ["g++", "-O3", "-std=c++17", "-fPIC", "-shared", "-w", "-fopenmp", "-ffp-contract=off",
           "-DTORCH_EXTENSION_NAME=points_cpu", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-I" + CSRC]
    for inc in cpp_extension.include_paths(device_type="cpu") + [sysconfig.get_paths()["include"]]:
        cmd.append("-I" + inc)
    cmd += [src, "-o", out, "-L" + torch_lib, "-Wl,-rpath," + torch_lib,
            "-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python"]
    _run(cmd)
    return out


def build(force=False):
    lib = build_kernels(force)
    ext = build_extension(force)
    build_cpu_extension(force)
    return lib, ext


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))

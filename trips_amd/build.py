"""Builds libtrips_splat.so (HIP kernels + C ABI) in-tree for gfx950 with hipcc."""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtrips_splat.so")
SOURCES = ["trips_splat_abi.hip", "splat_forward.hip", "splat_backward.hip", "misc_kernels.hip", "unet_forward.hip",
           "unet_backward.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # packed FP32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


HEADERS = ["splat_internal.h", "trips_math.h", "row16.h", "unet_common.h", os.path.join("..", "..", "include", "trips_splat.h"),
           os.path.join("..", "..", "include", "trips_unet.h")]


def build(verbose=False, incremental=False):
    """One hipcc process per translation unit, side by side, then one link. `incremental` skips units whose object
    is newer than the unit and every header (a convenience while editing; the default compiles everything)."""
    objdir = os.path.join(CSRC, "_obj")
    os.makedirs(objdir, exist_ok=True)
    newest_header = max(os.path.getmtime(os.path.join(CSRC, h)) for h in HEADERS)
    procs, objs = [], []
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), newest_header):
            continue
        cmd = [hipcc()] + FLAGS + ["-c", path, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd)))
    for cmd, pr in procs:
        if pr.wait() != 0:
            raise subprocess.CalledProcessError(pr.returncode, cmd)
    link = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    return LIB


SHIM_DIR = os.path.join(CSRC, "torch_shim")
SHIM_LIB = os.path.join(HERE, "_trips_torch.so")


def build_torch_shim(verbose=False):
    """Builds the libtorch host side (PointRender / NeuralRenderInfo / MyAdam in C++) with a pybind11 test driver.
    Plain g++: the shim holds no device code, it only calls the C ABI of libtrips_splat.so."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce
    tlib = ce.library_paths()[0]
    inc = [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include"]
    abi_flag = f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"
    flags = (["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-variable", abi_flag, "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
              "-DTORCH_EXTENSION_NAME=_trips_torch", "-DTORCH_API_INCLUDE_EXTENSION_H"] + inc)
    sources = ("trips_torch.cpp", "trips_unet_torch.cpp", "trips_scene_io.cpp", "trips_torch_py.cpp")
    objdir = os.path.join(SHIM_DIR, "_obj")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    for f in sources:  # one compiler process per translation unit, side by side
        obj = os.path.join(objdir, f.replace(".cpp", ".o"))
        cmd = ["g++"] + flags + ["-c", os.path.join(SHIM_DIR, f), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, obj, subprocess.Popen(cmd)))
    for cmd, obj, pr in procs:
        if pr.wait() != 0:
            raise subprocess.CalledProcessError(pr.returncode, cmd)
    link = (["g++", "-shared"] + [obj for _, obj, _ in procs] +
            [f"-L{tlib}", f"-L{HERE}", "-ltrips_splat", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
             "-ltorch_python", f"-Wl,-rpath,{tlib}", "-Wl,-rpath,$ORIGIN", "-o", SHIM_LIB])
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    return SHIM_LIB


if __name__ == "__main__":
    build(verbose=True, incremental="--incremental" in sys.argv)
    print(LIB)
    if "--shim" in sys.argv:
        print(build_torch_shim(verbose=True))

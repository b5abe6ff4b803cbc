"""Builds hingetreefortorch_amd/libhingetree_hip.so from csrc/*.hip with hipcc for gfx950 (cross-compiles without a GPU)
and, on top of it, the native host module hingetreefortorch_amd/_hingetree_host.so from csrc_host/hingetree_host.cpp
with the host compiler against the installed torch headers.

    python -m hingetreefortorch_amd.build

The objects go to hingetreefortorch_amd/build/, the two libraries next to this file (in-tree, git-ignored).
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libhingetree_hip.so")

SOURCES = ["capi.hip", "forest_forward.hip", "forest_backward.hip", "forest_maps.hip", "conv.hip", "projection.hip", "mix_f64.hip", "expand.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",       # margin = x - thr and |margin| * w must round like the reference's CPU code
    "-munsafe-fp-atomics",     # hardware fp32/fp64 atomic add instead of compare-and-swap loops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the HIP library cannot be built")


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc()] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, obj, proc.returncode, proc.stdout


def build_library(verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        for src, obj, rc, log in pool.map(_compile, SOURCES):
            text = "\n".join(l for l in log.splitlines() if "packed-fp32-ops" not in l)
            if verbose and text.strip():
                print(text)
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src}:\n{log}")
            objs.append(obj)
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


HOST_SRC = os.path.join(HERE, "csrc_host", "hingetree_host.cpp")
HOST_PATH = os.path.join(HERE, "_hingetree_host.so")


def build_host(verbose=True):
    """The pybind11 / ATen host module (the compiled counterpart of hingetree_cpp.py's forest / fern / convolution
    operators). Needs libhingetree_hip.so, which it links."""
    import sysconfig

    import torch

    torch_dir = os.path.dirname(torch.__file__)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cxx = os.environ.get("CXX") or shutil.which("g++") or "g++"
    tmp = HOST_PATH + ".tmp"
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_hingetree_host",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch.compiled_with_cxx11_abi()),
           "-I" + os.path.join(torch_dir, "include"),
           "-I" + os.path.join(torch_dir, "include", "torch", "csrc", "api", "include"),
           "-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(rocm, "include"),
           HOST_SRC, "-o", tmp,
           "-L" + os.path.join(torch_dir, "lib"), "-Wl,-rpath," + os.path.join(torch_dir, "lib"),
           "-L" + HERE, "-Wl,-rpath,$ORIGIN", "-lhingetree_hip",
           "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building the native host module failed:\n{proc.stdout}")
    if verbose and proc.stdout.strip():
        print(proc.stdout)
    os.replace(tmp, HOST_PATH)
    return HOST_PATH


if __name__ == "__main__":
    print(build_library())
    print(build_host())
    sys.exit(0)

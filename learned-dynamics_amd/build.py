"""Build libmanagan_hip.so (the C-ABI library) for gfx950 with hipcc, and managan_torch_ext.so, the
thin PyTorch C++ binding of it (host code only: csrc/torch_binding.cpp, compiled with g++ against
torch's headers and linked to the library next to it).

Run as `python learned-dynamics_amd/build.py` or call build().  hipcc
cross-compiles without a GPU.  Objects go to csrc/_obj, the libraries next to
this file so they travel with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB = os.path.join(HERE, "libmanagan_hip.so")
EXT = os.path.join(HERE, "managan_torch_ext.so")

COMMON = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-I", INCLUDE, "-I", CSRC,
    # packed fp32 instructions are switched off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]
# Per-file extra flags.  The neighbour search must reproduce an exact fp32
# recipe, so nothing in it may be contracted into FMAs behind its back.
EXTRA = {
    "neighbour_grid.hip": ["-ffp-contract=off"],
}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj_dir = os.path.join(CSRC, "_obj")
    os.makedirs(obj_dir, exist_ok=True)
    obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
    cmd = ["hipcc", "-c", os.path.join(CSRC, src), "-o", obj] + COMMON + EXTRA.get(src, [])
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    noise = ("is not a recognized feature for this target", "warning generated", "warnings generated")
    warnings = [l for l in r.stderr.splitlines() if l.strip() and not any(n in l for n in noise)]
    return obj, "\n".join(warnings)


def build(verbose=False, jobs=4):
    srcs = sources()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, srcs))
    objs = [o for o, _ in results]
    if verbose:
        for s, (_, w) in zip(srcs, results):
            if w:
                print(f"[{s}]\n{w}", file=sys.stderr)
    cmd = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    build_torch_binding()
    return LIB


def build_torch_binding():
    """managan_torch_ext.so: pybind11 module over torch's C++ API and the C ABI.  Plain host C++: no device code, so
    the host compiler builds it; it finds libmanagan_hip.so beside itself ($ORIGIN)."""
    import sysconfig

    import torch
    tdir = os.path.dirname(torch.__file__)
    cmd = ["g++", "-O2", "-fPIC", "-shared", "-std=c++17", "-Wall", "-Wno-unused-function",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=managan_torch_ext",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I", INCLUDE, "-I", os.path.join(tdir, "include"),
           "-I", os.path.join(tdir, "include", "torch", "csrc", "api", "include"), "-I", "/opt/rocm/include",
           "-I", sysconfig.get_paths()["include"],
           os.path.join(CSRC, "torch_binding.cpp"), "-o", EXT,
           "-L", os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
           "-L", HERE, "-l:libmanagan_hip.so", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"g++ failed on torch_binding.cpp:\n{r.stdout}\n{r.stderr}")
    return EXT


if __name__ == "__main__":
    print(build(verbose=True))

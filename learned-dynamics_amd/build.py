"""Build libmanagan_hip.so (the C-ABI library) for gfx950 with hipcc.

Run as `python learned-dynamics_amd/build.py` or call build().  hipcc
cross-compiles without a GPU.  Objects go to csrc/_obj, the library next to
this file so it travels with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB = os.path.join(HERE, "libmanagan_hip.so")

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
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))

"""CPU oracle for the equivariant message-passing hot path.

TEST INFRASTRUCTURE ONLY.  Only tests, the smoke check and the benchmark's
cpu_baseline leg may import this package; the product package never does.

Modules:
  neighbour  ctypes front end of neighbour_oracle.c (periodic cell-list radius graph)
  products   the 13 Cartesian tensor products, tensor_linear, TensorProdBare/TensorProds
  layers     Graph gather/scatter, radial encodings, PaiNN Message/Update, Bee Messages/SelfTensProds
"""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(force: bool = False) -> str:
    """Compile the C part of the oracle with gcc; returns the library path."""
    lib = os.path.join(_HERE, "_build", "libneighbour_oracle.so")
    if force or not os.path.exists(lib):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return lib

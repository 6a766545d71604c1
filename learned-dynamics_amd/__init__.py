"""MI355X (gfx950) implementation of the equivariant message-passing hot path
of pb1729/learned-dynamics: periodic neighbour search, Cartesian tensor
products + channel-mixing linears, edge->node segment sums.

The directory name contains a hyphen, so import it with
    importlib.import_module("learned-dynamics_amd")

Layout
  csrc/                      HIP kernels and the extern "C" entry points (libmanagan_hip.so);
                             torch_binding.cpp: the PyTorch C++ binding (managan_torch_ext.so)
  _lib.py, ops.py            ctypes binding and torch-facing operators
  graph_layers.py            Graph, radius_graph, edges_read*, edges_reduce_src, boxwrap
  tensor_products.py         TensLinear, TensorProdBare, TensorProds, norms, tens_sigmoid
  codegen_tensor_products.py Bee, Cow0, Cow1 autograd functions
  painn.py, bee_layers.py    PaiNN Message/Update/Block and Bee Messages/SelfTensProds
  shims/                     modules named like the reference's extensions
                             (neighbour_grid_cuda, tensor_ops_cuda, codegen_tensops_cuda, torch_scatter)
"""
import os
import sys

from . import _lib

_SHIMS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "shims")


def install_shims():
    """Make `import neighbour_grid_cuda`, `tensor_ops_cuda`, `codegen_tensops_cuda`, `polymer_sims_cuda`
    and `torch_scatter` resolve to this package's HIP implementations."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for path in (root, _SHIMS):
        if path not in sys.path:
            sys.path.insert(0, path)

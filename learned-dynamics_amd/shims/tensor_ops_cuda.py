"""Drop-in for the reference's `tensor_ops_cuda` extension
(extensions/tensor_ops/tensor_ops.cpp:173-182): differentiable tensor_linear.

Two routes to the same contraction.  Problems of a few thousand rows, where the time is the host's, go through the
package's PyTorch C++ binding (csrc/torch_binding.cpp: fp32 matrix-core kernel, a few microseconds of host time per
call); large ones go through the Python operator, which keeps pre-split weight planes and row bounds between calls
and runs the wide linears on the split-fp16 matrix path."""
import importlib

_tp = importlib.import_module("learned-dynamics_amd.tensor_products")
_ext = importlib.import_module("learned-dynamics_amd._lib").load_torch_ext()

SMALL_ROWS = 8192          # rows x components at or below which the C++ route is taken


def tensor_linear(inds, W, x):
    if x.is_cuda and x.numel() <= SMALL_ROWS * max(1, W.shape[-1]):
        return _ext.tensor_linear(inds, W, x)
    return _tp.tensor_linear(inds, W, x)

"""Drop-in for the reference's `tensor_ops_cuda` extension
(extensions/tensor_ops/tensor_ops.cpp:173-182): differentiable tensor_linear."""
import importlib

_tp = importlib.import_module("learned-dynamics_amd.tensor_products")


def tensor_linear(inds, W, x):
    return _tp.tensor_linear(inds, W, x)

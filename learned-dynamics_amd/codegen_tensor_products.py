"""Bee / Cow0 / Cow1 autograd functions, mirroring
managan/codegen_tensor_products.py:64-101 of the reference on top of the HIP
kernels (forward and both backward passes)."""
import torch

from . import ops


def _c(ts):
    return [t.contiguous() for t in ts]


class Bee(torch.autograd.Function):
    @staticmethod
    def forward(ctx, l_0, l_1, l_2, r_0, r_1, r_2):
        ctx.save_for_backward(l_0, l_1, l_2, r_0, r_1, r_2)
        return tuple(ops.bee_fwd(l_0, l_1, l_2, r_0, r_1, r_2))

    @staticmethod
    def backward(ctx, *dys):
        l_0, l_1, l_2, r_0, r_1, r_2 = ctx.saved_tensors
        dys = _c(dys)
        dl = ops.bee_bwl(r_0, r_1, r_2, *dys)
        dr = ops.bee_bwr(l_0, l_1, l_2, *dys)
        return (*dl, *dr)


class Cow0(torch.autograd.Function):
    @staticmethod
    def forward(ctx, l_0, l_1, r_0, r_1):
        ctx.save_for_backward(l_0, l_1, r_0, r_1)
        return tuple(ops.cow_o0_fwd(l_0, l_1, r_0, r_1))

    @staticmethod
    def backward(ctx, *dys):
        l_0, l_1, r_0, r_1 = ctx.saved_tensors
        dys = _c(dys)
        return (*ops.cow_o0_bwl(r_0, r_1, *dys), *ops.cow_o0_bwr(l_0, l_1, *dys))


class Cow1(torch.autograd.Function):
    @staticmethod
    def forward(ctx, l_0, l_1, r_0, r_1):
        ctx.save_for_backward(l_0, l_1, r_0, r_1)
        return tuple(ops.cow_o1_fwd(l_0, l_1, r_0, r_1))

    @staticmethod
    def backward(ctx, *dys):
        l_0, l_1, r_0, r_1 = ctx.saved_tensors
        dys = _c(dys)
        return (*ops.cow_o1_bwl(r_0, r_1, *dys), *ops.cow_o1_bwr(l_0, l_1, *dys))

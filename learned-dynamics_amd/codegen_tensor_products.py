"""Ant16 / Bee / Cow0 / Cow1 autograd functions, mirroring
managan/codegen_tensor_products.py:19-101 of the reference on top of the HIP
kernels (Bee, Cow: forward and both backward passes; Ant16: forward)."""
import torch

from . import ops


def _c(ts):
    return [t.contiguous() for t in ts]


class Ant16(torch.autograd.Function):
    """managan/codegen_tensor_products.py:19-61.  Forward only: the legacy architectures that use it
    run inference here; differentiating through it raises."""

    @staticmethod
    def forward(ctx, x_0, x_1, x_2,
                P_000, left_000, P_110, left_110, P_220, left_220,
                P_011, left_011, P_101, left_101, P_121, left_121, P_211, left_211, P_111, left_111,
                P_022, left_022, P_202, left_202, P_112, left_112, P_222, left_222, P_212, left_212):
        y_0, = ops.ant16_o0(x_0, x_1, x_2, P_000, left_000, P_110, left_110, P_220, left_220)
        y_1, = ops.ant16_o1(x_0, x_1, x_2, P_011, left_011, P_101, left_101, P_121, left_121, P_211, left_211)
        y_2, = ops.ant16_o2(x_0, x_1, x_2, P_022, left_022, P_202, left_202, P_112, left_112, P_222, left_222)
        y_1c, y_2c = ops.ant16_oc(x_1, x_2, P_111, left_111, P_212, left_212)
        return y_0, y_1 + y_1c, y_2 + y_2c

    @staticmethod
    def backward(ctx, *dys):
        raise NotImplementedError("Ant16: backward is not implemented (inference only)")


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

"""Ant16 / Bee / Cow0 / Cow1 autograd functions, mirroring
managan/codegen_tensor_products.py:19-101 of the reference on top of the HIP
kernels (forward and all backward passes of Bee, Cow and Ant16)."""
import torch

from . import ant16_backward as a16
from . import ops


def _c(ts):
    return [t.contiguous() for t in ts]


_ANT16_LABELS = ("000", "110", "220", "011", "101", "121", "211", "111", "022", "202", "112", "222", "212")


class Ant16(torch.autograd.Function):
    """managan/codegen_tensor_products.py:19-61.  Arguments after x_0, x_1, x_2 are (P, left) pairs in
    the order 000 110 220 011 101 121 211 111 022 202 112 222 212; gradients come back in that order."""

    @staticmethod
    def forward(ctx, x_0, x_1, x_2,
                P_000, left_000, P_110, left_110, P_220, left_220,
                P_011, left_011, P_101, left_101, P_121, left_121, P_211, left_211, P_111, left_111,
                P_022, left_022, P_202, left_202, P_112, left_112, P_222, left_222, P_212, left_212):
        ctx.save_for_backward(x_0, x_1, x_2,
                              P_000, left_000, P_110, left_110, P_220, left_220,
                              P_011, left_011, P_101, left_101, P_121, left_121, P_211, left_211, P_111, left_111,
                              P_022, left_022, P_202, left_202, P_112, left_112, P_222, left_222, P_212, left_212)
        y_0, = ops.ant16_o0(x_0, x_1, x_2, P_000, left_000, P_110, left_110, P_220, left_220)
        y_1, = ops.ant16_o1(x_0, x_1, x_2, P_011, left_011, P_101, left_101, P_121, left_121, P_211, left_211)
        y_2, = ops.ant16_o2(x_0, x_1, x_2, P_022, left_022, P_202, left_202, P_112, left_112, P_222, left_222)
        y_1c, y_2c = ops.ant16_oc(x_1, x_2, P_111, left_111, P_212, left_212)
        return y_0, y_1 + y_1c, y_2 + y_2c

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dy_0, dy_1, dy_2):
        xs = ctx.saved_tensors[:3]
        pairs = ctx.saved_tensors[3:]
        dys = tuple(d.contiguous() for d in (dy_0, dy_1, dy_2))
        needs = ctx.needs_input_grad
        terms = [(lab, pairs[2 * k], pairs[2 * k + 1]) for k, lab in enumerate(_ANT16_LABELS)]
        # one launch per rank of x, over every product type that reads that rank
        dxs = a16.grad_x_all(dys, [t for t in terms if needs[int(t[0][1])]])
        grads = []
        for k, (lab, P, left) in enumerate(terms):
            dy, x = dys[int(lab[2])], xs[int(lab[1])]
            grads.append(a16.grad_P(lab, dy, left, x) if needs[3 + 2 * k] else None)
            grads.append(a16.grad_left(lab, dy, P, x) if needs[4 + 2 * k] else None)
        return (*dxs, *grads)


class Bee(torch.autograd.Function):
    """The 13 products y = P(l, r) (managan/codegen_tensor_products.py:64-75).  P is bilinear, so the three kernels
    (forward, gradient for l, gradient for r) are each other's derivatives:
        <g, BWL(r, dy)> = <P(g, r), dy>,   <g, BWR(l, dy)> = <P(l, g), dy>.
    The backward passes are written with the autograd functions below, which makes Bee differentiable any number of
    times (the meanflow loss takes a Jacobian-vector product with create_graph=True)."""

    @staticmethod
    def forward(ctx, l_0, l_1, l_2, r_0, r_1, r_2):
        ctx.save_for_backward(l_0, l_1, l_2, r_0, r_1, r_2)
        ctx.save_for_forward(l_0, l_1, l_2, r_0, r_1, r_2)
        return tuple(ops.bee_fwd(*_c((l_0, l_1, l_2, r_0, r_1, r_2))))

    @staticmethod
    def jvp(ctx, *tangents):
        """Forward mode: P(l_t, r) + P(l, r_t) (an operand without a tangent arrives as zeros)."""
        l_0, l_1, l_2, r_0, r_1, r_2 = ctx.saved_tensors
        left, right = Bee.apply(*tangents[:3], r_0, r_1, r_2), Bee.apply(l_0, l_1, l_2, *tangents[3:])
        return tuple(a + b for a, b in zip(left, right))

    @staticmethod
    def backward(ctx, *dys):
        l_0, l_1, l_2, r_0, r_1, r_2 = ctx.saved_tensors
        dl = _BeeGradLeft.apply(r_0, r_1, r_2, *dys) if any(ctx.needs_input_grad[:3]) else (None, None, None)
        dr = _BeeGradRight.apply(l_0, l_1, l_2, *dys) if any(ctx.needs_input_grad[3:]) else (None, None, None)
        return (*dl, *dr)


class _BeeGradLeft(torch.autograd.Function):
    """(r, dy) -> dl = BWL(r, dy) (bee_bwl_cuda)."""

    @staticmethod
    def forward(ctx, r_0, r_1, r_2, *dys):
        ctx.save_for_backward(r_0, r_1, r_2, *dys)
        return tuple(ops.bee_bwl(*_c((r_0, r_1, r_2)), *_c(dys)))

    @staticmethod
    def backward(ctx, g_0, g_1, g_2):
        r_0, r_1, r_2, *dys = ctx.saved_tensors
        d_r = _BeeGradRight.apply(g_0, g_1, g_2, *dys) if any(ctx.needs_input_grad[:3]) else (None, None, None)
        d_dy = Bee.apply(g_0, g_1, g_2, r_0, r_1, r_2) if any(ctx.needs_input_grad[3:]) else (None,) * 13
        return (*d_r, *d_dy)


class _BeeGradRight(torch.autograd.Function):
    """(l, dy) -> dr = BWR(l, dy) (bee_bwr_cuda)."""

    @staticmethod
    def forward(ctx, l_0, l_1, l_2, *dys):
        ctx.save_for_backward(l_0, l_1, l_2, *dys)
        return tuple(ops.bee_bwr(*_c((l_0, l_1, l_2)), *_c(dys)))

    @staticmethod
    def backward(ctx, g_0, g_1, g_2):
        l_0, l_1, l_2, *dys = ctx.saved_tensors
        d_l = _BeeGradLeft.apply(g_0, g_1, g_2, *dys) if any(ctx.needs_input_grad[:3]) else (None, None, None)
        d_dy = Bee.apply(l_0, l_1, l_2, g_0, g_1, g_2) if any(ctx.needs_input_grad[3:]) else (None,) * 13
        return (*d_l, *d_dy)


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

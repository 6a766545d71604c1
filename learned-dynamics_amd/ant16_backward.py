"""The three backward families of Ant16 (ant16_o{0,1,2,c}_{backward,backleft,wtsback}_cuda,
extensions/codegen_tensops/codegen_tensops.cpp:669-821,892-1070,1142-1325,1374-1517; used by
managan/codegen_tensor_products.py:35-61) on the HIP kernels.

For one product type with coupling tensor T (entries 0, +1, -1; one Levi-Civita factor for the chiral
types) the forward is  y[b,o,O] = sum_{l,i,L,X} P[o,l,i] T[L,X,O] left[b,l,L] x[b,i,X], and
    dx[b,i,X]    = sum_{o,l,L,O} P[o,l,i] T[L,X,O] left[b,l,L] dy[b,o,O]       ("backward")
    dleft[b,l,L] = sum_{o,i,X,O} P[o,l,i] T[L,X,O] x[b,i,X] dy[b,o,O]          ("backleft")
    dP[o,l,i]    = sum_{b,L,X,O} T[L,X,O] left[b,l,L] x[b,i,X] dy[b,o,O]       ("wtsback")
The first two run on the forward kernel with the roles of the channel axes of P permuted, the third is a
contraction over rows with an ordered (deterministic) reduction.

These are raw kernels, not autograd functions: Ant16 is differentiable ONCE, as the reference's is (its backward
also calls kernels); codegen_tensor_products.Ant16.backward is marked once_differentiable, so a second derivative
(a double backward, or jvp(create_graph=True) followed by backward) raises instead of silently treating these
gradients as constants.  Bee, the linears and the PaiNN layers are differentiable to any order."""
import torch

from . import ops

FAMILIES = {"o0": ("000", "110", "220"), "o1": ("011", "101", "121", "211"), "o2": ("022", "202", "112", "222")}


def grad_x(label, dy, P, left):
    """dx of one product type: (batch, dim_r, (3,)^rank_r)."""
    dys = [None, None, None]
    dys[int(label[2])] = dy
    return ops.ant16_grad_x(int(label[1]), dys, [(label, P, left)])


def grad_left(label, dy, P, x):
    """dleft of one product type: (batch, dim_l, (3,)^rank_l)."""
    return ops.ant16_grad_left(label, P, x, dy)


def grad_P(label, dy, left, x):
    """dP of one product type: (dim_o, dim_l, dim_r)."""
    return ops.ant16_grad_weight(label, left, x, dy)


def grad_x_all(dys, terms):
    """[dx_0, dx_1, dx_2] summed over terms = [(label, P, left)]; one launch per rank of x.  A rank no term
    reads comes back as None."""
    out = [None, None, None]
    for r in range(3):
        mine = [t for t in terms if int(t[0][1]) == r]
        if mine:
            out[r] = ops.ant16_grad_x(r, dys, mine)
    return out


def backward(family, dy, *P_left):
    """ant16_<family>_backward_cuda(dy, P_a, left_a, P_b, left_b, ...) -> [dx_0, dx_1, dx_2]."""
    labels = FAMILIES[family]
    dys = [None, None, None]
    dys[int(family[1])] = dy
    return grad_x_all(dys, [(lab, P_left[2 * k], P_left[2 * k + 1]) for k, lab in enumerate(labels)])


def backleft(family, x_0, x_1, x_2, dy, *Ps):
    """ant16_<family>_backleft_cuda(x_0, x_1, x_2, dy, P_a, P_b, ...) -> [dleft_a, dleft_b, ...]."""
    xs = (x_0, x_1, x_2)
    return [grad_left(lab, dy, P, xs[int(lab[1])]) for lab, P in zip(FAMILIES[family], Ps)]


def wtsback(family, x_0, x_1, x_2, dy, *lefts):
    """ant16_<family>_wtsback_cuda(x_0, x_1, x_2, dy, left_a, left_b, ...) -> [dP_a, dP_b, ...]."""
    xs = (x_0, x_1, x_2)
    return [grad_P(lab, dy, left, xs[int(lab[1])]) for lab, left in zip(FAMILIES[family], lefts)]


def oc_backward(dy_1, dy_2, P_111, left_111, P_212, left_212):
    """-> [dx_1, dx_2]; both chiral products take x_1 on the right, so dx_2 is zero
    (shape (batch, dim_2, 3, 3) with dim_2 the channel count of dy_2, as the reference returns it)."""
    dx_1 = ops.ant16_grad_x(1, [None, dy_1, dy_2], [("111", P_111, left_111), ("212", P_212, left_212)])
    return [dx_1, torch.zeros_like(dy_2)]


def oc_backleft(x_1, x_2, dy_1, dy_2, P_111, P_212):
    return [grad_left("111", dy_1, P_111, x_1), grad_left("212", dy_2, P_212, x_1)]


def oc_wtsback(x_1, x_2, dy_1, dy_2, left_111, left_212):
    return [grad_P("111", dy_1, left_111, x_1), grad_P("212", dy_2, left_212, x_1)]


# The reference's generated example with nine product types of mixed output rank (fused_tensor_prods_example{,_backward,
# _backleft,_wtsback}_cuda: extensions/codegen_tensops/do_codegen.py:4-7, codegen_tensops.cpp:158-608, bound at
# :1981-1984; exercised by extensions/codegen_tensops/test.py:29-39).  Same contraction as Ant16, so the same kernels:
# one forward launch per output rank, one gradient launch per rank of x, one per left / P.
EXAMPLE = ("000", "011", "101", "110", "220", "222", "211", "111", "212")


def example_forward(x_0, x_1, x_2, *P_left):
    """fused_tensor_prods_example_cuda(x_0, x_1, x_2, P_000, left_000, P_011, left_011, ...) -> [y_0, y_1, y_2]."""
    terms = [(lab, P_left[2 * k], P_left[2 * k + 1]) for k, lab in enumerate(EXAMPLE)]
    return [ops._ant16(rank, x_0, x_1, x_2, [t for t in terms if int(t[0][2]) == rank]) for rank in range(3)]


def example_backward(dy_0, dy_1, dy_2, *P_left):
    """fused_tensor_prods_example_backward_cuda(dy_0, dy_1, dy_2, P_000, left_000, ...) -> [dx_0, dx_1, dx_2]."""
    return grad_x_all([dy_0, dy_1, dy_2], [(lab, P_left[2 * k], P_left[2 * k + 1]) for k, lab in enumerate(EXAMPLE)])


def example_backleft(x_0, x_1, x_2, dy_0, dy_1, dy_2, *Ps):
    """fused_tensor_prods_example_backleft_cuda(x_0, x_1, x_2, dy_0, dy_1, dy_2, P_000, P_011, ...) -> nine dleft."""
    xs, dys = (x_0, x_1, x_2), (dy_0, dy_1, dy_2)
    return [grad_left(lab, dys[int(lab[2])], P, xs[int(lab[1])]) for lab, P in zip(EXAMPLE, Ps)]


def example_wtsback(x_0, x_1, x_2, dy_0, dy_1, dy_2, *lefts):
    """fused_tensor_prods_example_wtsback_cuda(x_0, x_1, x_2, dy_0, dy_1, dy_2, left_000, left_011, ...) -> nine dP."""
    xs, dys = (x_0, x_1, x_2), (dy_0, dy_1, dy_2)
    return [grad_P(lab, dys[int(lab[2])], left, xs[int(lab[1])]) for lab, left in zip(EXAMPLE, lefts)]

"""The three backward families of Ant16 (ant16_o{0,1,2,c}_{backward,backleft,wtsback}_cuda,
extensions/codegen_tensops/codegen_tensops.cpp:669-821,892-1070,1142-1325,1374-1517; used by
managan/codegen_tensor_products.py:35-61), as contractions on the device.

For one product type with coupling tensor T (entries 0, +1, -1; one Levi-Civita factor for the chiral
types) the forward is  y[b,o,O] = sum_{l,i,L,X} P[o,l,i] T[L,X,O] left[b,l,L] x[b,i,X], and
    dx[b,i,X]    = sum_{o,l,L,O} P[o,l,i] T[L,X,O] left[b,l,L] dy[b,o,O]       ("backward")
    dleft[b,l,L] = sum_{o,i,X,O} P[o,l,i] T[L,X,O] x[b,i,X] dy[b,o,O]          ("backleft")
    dP[o,l,i]    = sum_{b,L,X,O} T[L,X,O] left[b,l,L] x[b,i,X] dy[b,o,O]       ("wtsback")
Each is evaluated as two pairwise contractions (a GEMM over the channel axes through rocBLAS, then the
small component contraction), so the largest temporary is (batch, dim_l, dim_r, 3^rank_o).  These run
as library GEMMs, not hand-written kernels: the legacy architectures that train through Ant16 are not
on the measured path.  Being compositions of differentiable torch operations they can be
differentiated again."""
import torch

# component subscripts of (left, right operand, output) per product type; contracted indices trail,
# kept left indices come before kept right ones; the chiral types carry one Levi-Civita factor
_SUBSCRIPTS = {
    "000": ("", "", "", None), "110": ("x", "x", "", None), "220": ("xy", "xy", "", None),
    "011": ("", "x", "x", None), "101": ("x", "", "x", None), "121": ("x", "yx", "y", None),
    "211": ("xy", "y", "x", None), "111": ("x", "y", "z", "xyz"),
    "022": ("", "xy", "xy", None), "202": ("xy", "", "xy", None), "112": ("x", "y", "xy", None),
    "222": ("xy", "zy", "xz", None), "212": ("xy", "z", "xw", "yzw"),
}
FAMILIES = {"o0": ("000", "110", "220"), "o1": ("011", "101", "121", "211"), "o2": ("022", "202", "112", "222")}

_eps_cache = {}


def _levi_civita(device, dtype):
    key = (str(device), dtype)
    if key not in _eps_cache:
        e = torch.zeros(3, 3, 3, dtype=dtype)
        for i, j, k in ((0, 1, 2), (1, 2, 0), (2, 0, 1)):
            e[i, j, k] = 1.0
            e[i, k, j] = -1.0
        _eps_cache[key] = e.to(device)
    return _eps_cache[key]


def _contract(spec, *operands, eps_sub=None):
    if eps_sub is not None:
        lhs, rhs = spec.split("->")
        return torch.einsum(f"{lhs},{eps_sub}->{rhs}", *operands, _levi_civita(operands[0].device, operands[0].dtype))
    return torch.einsum(spec, *operands)


def grad_x(label, dy, P, left):
    """dx of one product type: (batch, dim_r, (3,)^rank_r)."""
    L, X, O, eps = _SUBSCRIPTS[label]
    g = torch.einsum(f"bo{O},oli->bli{O}", dy, P)
    return _contract(f"bli{O},bl{L}->bi{X}", g, left, eps_sub=eps)


def grad_left(label, dy, P, x):
    """dleft of one product type: (batch, dim_l, (3,)^rank_l)."""
    L, X, O, eps = _SUBSCRIPTS[label]
    g = torch.einsum(f"bo{O},oli->bli{O}", dy, P)
    return _contract(f"bli{O},bi{X}->bl{L}", g, x, eps_sub=eps)


def grad_P(label, dy, left, x):
    """dP of one product type: (dim_o, dim_l, dim_r)."""
    L, X, O, eps = _SUBSCRIPTS[label]
    q = _contract(f"bl{L},bi{X}->bli{O}", left, x, eps_sub=eps)
    return torch.einsum(f"bo{O},bli{O}->oli", dy, q)


def _x_of(label, xs):
    return xs[int(label[1])]


def backward(family, dy, *P_left):
    """ant16_<family>_backward_cuda(dy, P_a, left_a, P_b, left_b, ...) -> [dx_0, dx_1, dx_2]."""
    labels = FAMILIES[family]
    out = [None, None, None]
    for k, lab in enumerate(labels):
        d = grad_x(lab, dy, P_left[2 * k], P_left[2 * k + 1])
        r = int(lab[1])
        out[r] = d if out[r] is None else out[r] + d
    return out


def backleft(family, x_0, x_1, x_2, dy, *Ps):
    """ant16_<family>_backleft_cuda(x_0, x_1, x_2, dy, P_a, P_b, ...) -> [dleft_a, dleft_b, ...]."""
    xs = (x_0, x_1, x_2)
    return [grad_left(lab, dy, P, _x_of(lab, xs)) for lab, P in zip(FAMILIES[family], Ps)]


def wtsback(family, x_0, x_1, x_2, dy, *lefts):
    """ant16_<family>_wtsback_cuda(x_0, x_1, x_2, dy, left_a, left_b, ...) -> [dP_a, dP_b, ...]."""
    xs = (x_0, x_1, x_2)
    return [grad_P(lab, dy, left, _x_of(lab, xs)) for lab, left in zip(FAMILIES[family], lefts)]


def oc_backward(dy_1, dy_2, P_111, left_111, P_212, left_212):
    """-> [dx_1, dx_2]; both chiral products take x_1 on the right, so dx_2 is zero
    (shape (batch, dim_2, 3, 3) with dim_2 the channel count of dy_2, as the reference returns it)."""
    dx_1 = grad_x("111", dy_1, P_111, left_111) + grad_x("212", dy_2, P_212, left_212)
    return [dx_1, torch.zeros_like(dy_2)]


def oc_backleft(x_1, x_2, dy_1, dy_2, P_111, P_212):
    return [grad_left("111", dy_1, P_111, x_1), grad_left("212", dy_2, P_212, x_1)]


def oc_wtsback(x_1, x_2, dy_1, dy_2, left_111, left_212):
    return [grad_P("111", dy_1, left_111, x_1), grad_P("212", dy_2, left_212, x_1)]

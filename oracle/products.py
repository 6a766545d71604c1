"""TEST INFRASTRUCTURE ONLY — CPU restatement (PyTorch, any float dtype) of the
Cartesian tensor products and the per-irrep channel-mixing linear.

Follows (relative to the reference checkout):
  managan/codegen_tensor_products.py:235-249   the 13 products behind Bee (einsum forms)
  managan/codegen_tensor_products.py:279-288   Cow0 (000,110) and Cow1 (011,101,111)
  managan/codegen_tensor_products.py:112-133   Ant16: weights P[o,l,r] folded into each product
  managan/tensor_products.py:41-43             Levi-Civita symbol
  managan/tensor_products.py:91-106            TensorProdBare: contracted indices trail both operands
  managan/tensor_products.py:109-121           TensorProds = lin_o(prod(lin_l(x_l), lin_r(x_r)))
  extensions/tensor_ops/test.py:9-15           tensor_linear == einsum("OI, ...Iijk -> ...Oijk")

Layout of every operand: (rows, chan[, 3[, 3]]), component index fastest.
Pinned by tests/test_oracle_products.py against library routines (cross,
matmul, trace), an explicit-loop evaluation on tiny inputs and SO(3)
equivariance under the reference's fixed rotation matrix.
"""
import itertools
import torch

BEE_ORDER = ("000", "110", "220", "011", "101", "121", "211",
             "022", "202", "112", "222", "111", "212")
COW0_ORDER = ("000", "110")
COW1_ORDER = ("011", "101", "111")

# label -> einsum over (left, right[, epsilon]); b = row, c = channel
_FORMS = {
    "000": "bc,bc->bc",
    "110": "bcx,bcx->bc",
    "220": "bcxy,bcxy->bc",
    "011": "bc,bcx->bcx",
    "101": "bcx,bc->bcx",
    "121": "bcx,bcyx->bcy",
    "211": "bcxy,bcy->bcx",
    "022": "bc,bcxy->bcxy",
    "202": "bcxy,bc->bcxy",
    "112": "bcx,bcy->bcxy",
    "222": "bcxy,bczy->bcxz",
    "111": "bcx,bcy,xyz->bcz",
    "212": "bcxy,bcz,yzw->bcxw",
}
CHIRAL = ("111", "212")


def levi_civita(dtype=torch.float32):
    eps = torch.zeros(3, 3, 3, dtype=dtype)
    for i, j, k in itertools.permutations(range(3)):
        # sign of the permutation (i,j,k)
        eps[i, j, k] = ((i - j) * (j - k) * (k - i)) / 2.0
    return eps


def product(label, left, right):
    """One of the 13 products; left has rank label[0], right rank label[1], result rank label[2]."""
    if label in CHIRAL:
        return torch.einsum(_FORMS[label], left, right, levi_civita(left.dtype))
    return torch.einsum(_FORMS[label], left, right)


def _by_rank(label, t0, t1, t2, side):
    return (t0, t1, t2)[int(label[side])]


def bee(l_0, l_1, l_2, r_0, r_1, r_2):
    return tuple(product(lab, _by_rank(lab, l_0, l_1, l_2, 0), _by_rank(lab, r_0, r_1, r_2, 1))
                 for lab in BEE_ORDER)


def cow0(l_0, l_1, r_0, r_1):
    return tuple(product(lab, _by_rank(lab, l_0, l_1, None, 0), _by_rank(lab, r_0, r_1, None, 1))
                 for lab in COW0_ORDER)


def cow1(l_0, l_1, r_0, r_1):
    return tuple(product(lab, _by_rank(lab, l_0, l_1, None, 0), _by_rank(lab, r_0, r_1, None, 1))
                 for lab in COW1_ORDER)


def tensor_linear(inds, W, x):
    """y[..., o, t] = sum_i W[o, i] x[..., i, t]; t runs over the 3**inds trailing components."""
    shape = x.shape
    lead = shape[:len(shape) - inds - 1]
    dim_in = shape[len(lead)]
    assert dim_in == W.shape[1]
    x2 = x.reshape(-1, dim_in, 3 ** inds)
    y2 = torch.matmul(W, x2)
    return y2.reshape(*lead, W.shape[0], *([3] * inds))


def tensor_prod_bare(inds_l, inds_r, inds_o, x_l, x_r):
    """Contract the trailing indices of both operands; kept left indices first, then kept right."""
    assert (inds_l + inds_r - inds_o) % 2 == 0, "parity mismatch"
    k = (inds_l + inds_r - inds_o) // 2
    assert 0 <= k <= min(inds_l, inds_r)
    letters = "ijklmn"
    keep_l = letters[:inds_l - k]
    keep_r = letters[inds_l - k:inds_l - k + inds_r - k]
    con = "uvw"[:k]
    return torch.einsum(f"...{keep_l}{con},...{keep_r}{con}->...{keep_l}{keep_r}", x_l, x_r)


def tensor_prods(inds_l, inds_r, inds_o, W_l, W_r, W_o, x_l, x_r):
    a = tensor_linear(inds_l, W_l, x_l)
    b = tensor_linear(inds_r, W_r, x_r)
    return tensor_linear(inds_o, W_o, tensor_prod_bare(inds_l, inds_r, inds_o, a, b))


# ---------------------------------------------------------------------------
# Ant16: y_o = sum over labels with output rank o of  sum_{l,i} P[o,l,i] prod(left[l], x[i])
# ---------------------------------------------------------------------------
_ANT_FORMS = {
    "000": "bl,br,olr->bo",
    "110": "blx,brx,olr->bo",
    "220": "blxy,brxy,olr->bo",
    "011": "bl,brx,olr->box",
    "101": "blx,br,olr->box",
    "121": "blx,bryx,olr->boy",
    "211": "blxy,bry,olr->box",
    "022": "bl,brxy,olr->boxy",
    "202": "blxy,br,olr->boxy",
    "112": "blx,bry,olr->boxy",
    "222": "blxy,brzy,olr->boxz",
    "111": "blx,bry,olr,xyz->boz",
    "212": "blxy,brz,olr,yzw->boxw",
}


def ant16(x_0, x_1, x_2, P, left):
    """P, left: dicts label -> tensor.  Returns (y_0, y_1, y_2)."""
    xs = (x_0, x_1, x_2)
    out = [None, None, None]
    for lab in BEE_ORDER:
        xr = xs[int(lab[1])]
        if lab in CHIRAL:
            p = torch.einsum(_ANT_FORMS[lab], left[lab], xr, P[lab], levi_civita(xr.dtype))
        else:
            p = torch.einsum(_ANT_FORMS[lab], left[lab], xr, P[lab])
        o = int(lab[2])
        out[o] = p if out[o] is None else out[o] + p
    return tuple(out)


# ---------------------------------------------------------------------------
# Backward of the 13 products, by autograd on the restatement (used as the
# oracle for bee_bwl/bwr and cow_*_bwl/bwr).
# ---------------------------------------------------------------------------
def products_backward(order, lefts, rights, dys):
    """lefts/rights: tuples indexed by rank (None for unused ranks); dys in `order`.
    Returns (dl by rank, dr by rank) with zeros for ranks that receive no gradient."""
    ls = [None if t is None else t.detach().clone().requires_grad_(True) for t in lefts]
    rs = [None if t is None else t.detach().clone().requires_grad_(True) for t in rights]
    total = 0.0
    for lab, dy in zip(order, dys):
        y = product(lab, ls[int(lab[0])], rs[int(lab[1])])
        total = total + (y * dy).sum()
    leaves = [t for t in ls + rs if t is not None]
    grads = torch.autograd.grad(total, leaves, allow_unused=True)
    it = iter(grads)
    dl = [None if t is None else next(it) for t in ls]
    dr = [None if t is None else next(it) for t in rs]
    dl = [None if t is None else (torch.zeros_like(t) if g is None else g) for t, g in zip(ls, dl)]
    dr = [None if t is None else (torch.zeros_like(t) if g is None else g) for t, g in zip(rs, dr)]
    return dl, dr

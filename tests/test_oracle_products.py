"""Pins oracle/products.py with checks that do not restate its formulas:
library routines (cross, matmul, trace), explicit loops on tiny inputs, SO(3)
equivariance under the reference's fixed rotation (managan/symmetries.py:54-57),
and autograd consistency of the backward helper."""
import itertools

import pytest
import os

import torch

from conftest import load_golden
from oracle import products as OP

ROT = torch.tensor(load_golden("symmetry_checks")["rotation"], dtype=torch.float64)


def _rand(rows, chan, rank, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(rows, chan, *([3] * rank), generator=g, dtype=dtype)


def _ops(seed=0, rows=4, chan=5):
    l = [_rand(rows, chan, k, seed + k) for k in range(3)]
    r = [_rand(rows, chan, k, seed + 10 + k) for k in range(3)]
    return l, r


def test_levi_civita():
    eps = OP.levi_civita(torch.float64)
    assert eps[0, 1, 2] == 1 and eps[1, 2, 0] == 1 and eps[2, 0, 1] == 1
    assert eps[0, 2, 1] == -1 and eps[2, 1, 0] == -1 and eps[1, 0, 2] == -1
    assert eps.abs().sum() == 6
    # determinant identity: eps_ijk R_ia R_jb R_kc = det(R) eps_abc, det(ROT) ~ +1
    lhs = torch.einsum("ijk,ia,jb,kc->abc", eps, ROT, ROT, ROT)
    assert torch.allclose(lhs, torch.linalg.det(ROT) * eps, atol=1e-12)


def test_products_against_library_routines():
    (l0, l1, l2), (r0, r1, r2) = _ops()
    y = dict(zip(OP.BEE_ORDER, OP.bee(l0, l1, l2, r0, r1, r2)))
    assert torch.allclose(y["000"], l0 * r0)
    assert torch.allclose(y["110"], (l1 * r1).sum(-1))
    assert torch.allclose(y["220"], (l2 @ r2.transpose(-1, -2)).diagonal(dim1=-2, dim2=-1).sum(-1))
    assert torch.allclose(y["011"], l0[..., None] * r1)
    assert torch.allclose(y["101"], l1 * r0[..., None])
    assert torch.allclose(y["121"], (r2 @ l1[..., None])[..., 0])          # y_y = sum_x r_yx l_x
    assert torch.allclose(y["211"], (l2 @ r1[..., None])[..., 0])          # y_x = sum_y l_xy r_y
    assert torch.allclose(y["022"], l0[..., None, None] * r2)
    assert torch.allclose(y["202"], l2 * r0[..., None, None])
    assert torch.allclose(y["112"], l1[..., :, None] * r1[..., None, :])   # full outer product
    assert torch.allclose(y["222"], l2 @ r2.transpose(-1, -2))             # L R^T
    assert torch.allclose(y["111"], torch.linalg.cross(l1, r1))
    assert torch.allclose(y["212"], torch.linalg.cross(l2, r1[..., None, :].expand_as(l2)))  # rows of L cross r


def test_products_explicit_loops_tiny():
    (l0, l1, l2), (r0, r1, r2) = _ops(seed=3, rows=1, chan=2)
    y = dict(zip(OP.BEE_ORDER, OP.bee(l0, l1, l2, r0, r1, r2)))
    eps = OP.levi_civita(torch.float64)
    for c in range(2):
        L1, L2, R1, R2 = l1[0, c], l2[0, c], r1[0, c], r2[0, c]
        for a in range(3):
            assert abs(y["121"][0, c, a] - sum(L1[x] * R2[a, x] for x in range(3))) < 1e-12
            assert abs(y["211"][0, c, a] - sum(L2[a, b] * R1[b] for b in range(3))) < 1e-12
            assert abs(y["111"][0, c, a] - sum(eps[x, yy, a] * L1[x] * R1[yy]
                                               for x in range(3) for yy in range(3))) < 1e-12
            for w in range(3):
                assert abs(y["222"][0, c, a, w] - sum(L2[a, b] * R2[w, b] for b in range(3))) < 1e-12
                assert abs(y["212"][0, c, a, w] - sum(eps[b, z, w] * L2[a, b] * R1[z]
                                                      for b in range(3) for z in range(3))) < 1e-12


def _rotate(t, rank, R):
    if rank == 0:
        return t
    if rank == 1:
        return torch.einsum("...i,ij->...j", t, R)
    return torch.einsum("...ij,ia,jb->...ab", t, R, R)


def test_products_are_rotation_equivariant():
    """Proper rotation: also the two chiral products (one Levi-Civita each) must co-rotate."""
    q, _ = torch.linalg.qr(ROT)            # the printed matrix is orthogonal to 4 digits only
    R = q * torch.sign(torch.linalg.det(q))
    assert torch.allclose(R.abs(), ROT.abs(), atol=2e-3)
    (l0, l1, l2), (r0, r1, r2) = _ops(seed=5)
    y = OP.bee(l0, l1, l2, r0, r1, r2)
    ls = [_rotate(t, k, R) for k, t in enumerate((l0, l1, l2))]
    rs = [_rotate(t, k, R) for k, t in enumerate((r0, r1, r2))]
    y_rot_in = OP.bee(*ls, *rs)
    for lab, a, b in zip(OP.BEE_ORDER, y, y_rot_in):
        assert torch.allclose(_rotate(a, int(lab[2]), R), b, atol=1e-10), lab


def test_cow_subsets_match_bee():
    (l0, l1, l2), (r0, r1, r2) = _ops(seed=6)
    y = dict(zip(OP.BEE_ORDER, OP.bee(l0, l1, l2, r0, r1, r2)))
    for lab, t in zip(OP.COW0_ORDER, OP.cow0(l0, l1, r0, r1)):
        assert torch.equal(t, y[lab])
    for lab, t in zip(OP.COW1_ORDER, OP.cow1(l0, l1, r0, r1)):
        assert torch.equal(t, y[lab])


@pytest.mark.parametrize("lro", [(0, 0, 0), (1, 1, 0), (2, 2, 0), (0, 1, 1), (1, 0, 1), (1, 2, 1), (2, 1, 1),
                                 (0, 2, 2), (2, 0, 2), (1, 1, 2), (2, 2, 2)])
def test_tensor_prod_bare_equals_labelled_product(lro):
    il, ir, io = lro
    x_l, x_r = _rand(3, 4, il, 7), _rand(3, 4, ir, 8)
    lab = f"{il}{ir}{io}"
    assert torch.allclose(OP.tensor_prod_bare(il, ir, io, x_l, x_r), OP.product(lab, x_l, x_r))


def test_tensor_prod_bare_rejects_chiral():
    x = _rand(3, 4, 1, 7)
    with pytest.raises(AssertionError, match="parity"):
        OP.tensor_prod_bare(1, 1, 1, x, x)


def test_tensor_linear_is_matmul_per_component():
    g = torch.Generator().manual_seed(9)
    W = torch.randn(21, 11, generator=g, dtype=torch.float64)
    for inds in range(3):
        x = torch.randn(2, 5, 11, *([3] * inds), generator=g, dtype=torch.float64)
        y = OP.tensor_linear(inds, W, x)
        letters = "ijk"[:inds]
        assert torch.allclose(y, torch.einsum(f"OI,...I{letters}->...O{letters}", W, x))
        # component by component: an ordinary matrix-vector product
        flat_x = x.reshape(10, 11, -1)
        flat_y = y.reshape(10, 21, -1)
        for t in range(3 ** inds):
            assert torch.allclose(flat_y[:, :, t], flat_x[:, :, t] @ W.T)


def test_ant16_reduces_to_bee_for_diagonal_weights():
    """With dim_l = dim_r = dim_o = C and P[o,l,r] = delta_ol delta_or, Ant16 is the sum of the Bee products."""
    C = 4
    (l0, l1, l2), (r0, r1, r2) = _ops(seed=12, rows=3, chan=C)
    eye = torch.zeros(C, C, C, dtype=torch.float64)
    for c in range(C):
        eye[c, c, c] = 1.0
    P = {lab: eye for lab in OP.BEE_ORDER}
    left = {lab: (l0, l1, l2)[int(lab[0])] for lab in OP.BEE_ORDER}
    y0, y1, y2 = OP.ant16(r0, r1, r2, P, left)
    prods = dict(zip(OP.BEE_ORDER, OP.bee(l0, l1, l2, r0, r1, r2)))
    assert torch.allclose(y0, prods["000"] + prods["110"] + prods["220"])
    assert torch.allclose(y1, prods["011"] + prods["101"] + prods["121"] + prods["211"] + prods["111"])
    assert torch.allclose(y2, prods["022"] + prods["202"] + prods["112"] + prods["222"] + prods["212"])


def test_ant16_against_explicit_loops():
    """P[o, l, r] pairs channel l of `left` with channel r of x (and not the other way round): explicit
    loops over (b, o, l, r) around the single-channel products, on sizes where every axis differs."""
    g = torch.Generator().manual_seed(21)
    batch, dims, dl = 2, (3, 4, 2), 5
    x = [torch.randn(batch, dims[k], *([3] * k), generator=g, dtype=torch.float64) for k in range(3)]
    P = {lab: torch.randn(dims[int(lab[2])], dl, dims[int(lab[1])], generator=g, dtype=torch.float64)
         for lab in OP.BEE_ORDER}
    left = {lab: torch.randn(batch, dl, *([3] * int(lab[0])), generator=g, dtype=torch.float64)
            for lab in OP.BEE_ORDER}
    ys = OP.ant16(x[0], x[1], x[2], P, left)
    want = [torch.zeros_like(y) for y in ys]
    for lab in OP.BEE_ORDER:
        rl, rr, ro = int(lab[0]), int(lab[1]), int(lab[2])
        for b in range(batch):
            for o in range(dims[ro]):
                for l in range(dl):
                    for r in range(dims[rr]):
                        # product() takes (rows, chan, ...) operands: one row, one channel
                        prod = OP.product(lab, left[lab][b:b + 1, l:l + 1], x[rr][b:b + 1, r:r + 1])[0, 0]
                        want[ro][b, o] += P[lab][o, l, r] * prod
    for y, w in zip(ys, want):
        assert torch.allclose(y, w)


def test_backward_helper_matches_finite_differences():
    (l0, l1, l2), (r0, r1, r2) = _ops(seed=13, rows=2, chan=2)
    g = torch.Generator().manual_seed(14)
    dys = [torch.randn(2, 2, *([3] * int(lab[2])), generator=g, dtype=torch.float64) for lab in OP.BEE_ORDER]
    dl, dr = OP.products_backward(OP.BEE_ORDER, (l0, l1, l2), (r0, r1, r2), dys)

    def loss(ls, rs):
        return sum((y * dy).sum() for y, dy in zip(OP.bee(*ls, *rs), dys))

    h = 1e-6
    for k, t in enumerate((l0, l1, l2)):
        flat = t.reshape(-1)
        for j in (0, flat.numel() - 1):
            tp = t.clone().reshape(-1); tp[j] += h
            tm = t.clone().reshape(-1); tm[j] -= h
            ls_p = [l0, l1, l2]; ls_p[k] = tp.reshape(t.shape)
            ls_m = [l0, l1, l2]; ls_m[k] = tm.reshape(t.shape)
            fd = (loss(ls_p, (r0, r1, r2)) - loss(ls_m, (r0, r1, r2))) / (2 * h)
            assert abs(fd - dl[k].reshape(-1)[j]) < 1e-6


def _coupling_generator():
    import importlib.util
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "learned-dynamics_amd", "csrc",
                        "gen_ant16_coupling.py")
    spec = importlib.util.spec_from_file_location("gen_ant16_coupling", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod, path


def test_ant16_coupling_table_against_the_products_and_their_derivatives():
    """The term lists the Ant16 kernels are generated from (forward, gradient for x, gradient for left), evaluated
    here on random operands, against the oracle's product of each type and autograd through it; and the committed
    table is what the generator writes."""
    gen, path = _coupling_generator()
    tab = gen.table()
    assert gen.LABELS == tuple(OP.BEE_ORDER)

    def apply(mode, k, n_out, a, b):
        out = torch.zeros(n_out, dtype=torch.float64)
        for c in range(n_out):
            for e in tab[mode][k][c]:
                out[c] += (-1.0 if e & 256 else 1.0) * a.reshape(-1)[e & 15] * b.reshape(-1)[(e >> 4) & 15]
        return out

    g = torch.Generator().manual_seed(5)
    for k, lab in enumerate(OP.BEE_ORDER):
        rl, rr, ro = (int(c) for c in lab)
        l = torch.randn(1, 1, *([3] * rl), generator=g, dtype=torch.float64, requires_grad=True)
        r = torch.randn(1, 1, *([3] * rr), generator=g, dtype=torch.float64, requires_grad=True)
        y = OP.product(lab, l, r)
        dy = torch.randn(y.shape, generator=g, dtype=torch.float64)
        gl, gr = torch.autograd.grad((y * dy).sum(), (l, r))
        assert torch.allclose(apply(0, k, 3 ** ro, l.detach(), r.detach()), y.detach().reshape(-1), atol=1e-14)
        assert torch.allclose(apply(1, k, 3 ** rr, l.detach(), dy), gr.reshape(-1), atol=1e-14)
        assert torch.allclose(apply(2, k, 3 ** rl, r.detach(), dy), gl.reshape(-1), atol=1e-14)
    committed = open(os.path.join(os.path.dirname(path), "ant16_coupling.inc")).read()
    import tempfile, shutil
    with tempfile.TemporaryDirectory() as tmp:
        shutil.copy(path, tmp)
        mod_path = os.path.join(tmp, "gen_ant16_coupling.py")
        import importlib.util
        spec = importlib.util.spec_from_file_location("gen_tmp", mod_path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        assert open(mod.main()).read() == committed

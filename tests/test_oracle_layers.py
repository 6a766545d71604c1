"""Pins oracle/layers.py with checks that do not restate its formulas: library
routines (scipy Jacobi polynomials, torch GroupNorm), closed forms, special
cases, SO(3) equivariance under the reference's rotation, brute-force loops."""
import math

import numpy as np
import pytest
import torch

from conftest import load_golden
from oracle import layers as OL
from oracle import products as OP

ROT = torch.tensor(load_golden("symmetry_checks")["rotation"], dtype=torch.float64)   # managan/symmetries.py:54-57
Q, _ = torch.linalg.qr(ROT)
ROT = Q * torch.sign(torch.linalg.det(Q))            # exact rotation next to the printed one


def test_jacobi_matrix_against_scipy():
    from scipy.special import eval_jacobi
    A = OL.jacobi_matrix(8, torch.float64)
    z = np.linspace(0.0, 1.0, 41)
    for i in range(8):
        poly = sum(A[i, j].item() * z ** j for j in range(9))
        assert np.allclose(poly, eval_jacobi(i, 1, 0, 2 * z - 1), atol=1e-9)
    assert float(A[:, 8].abs().max()) == 0.0          # degree < 8
    assert float(A.abs().max()) < 2 ** 24             # exactly representable in fp32


def test_radial_encode_8_properties_and_fp32_conditioning():
    g = torch.Generator().manual_seed(0)
    r = torch.randn(2000, 3, generator=g, dtype=torch.float64) * 3
    enc = OL.radial_encode_8(r, 6.0)
    z = r.norm(dim=-1) / 6.0
    assert torch.all(enc[z >= 1.0] == 0)                                  # relu(1 - z) cutoff
    assert torch.allclose(enc[:, 0], torch.relu(1 - z))                    # P_0 = 1
    assert torch.allclose(enc[:, 1], (3 * z - 1) * torch.relu(1 - z))      # P_1^{(1,0)}(t) = (3t+1)/2, t = 2z-1
    # the literal fp32 evaluation (what the reference runs) is ill-conditioned: it differs from the
    # exact value by far more than fp32 epsilon, which is why the device evaluates in fp64
    enc32 = OL.radial_encode_8(r.float(), 6.0).double()
    err = (enc32 - enc).abs().max().item()
    assert 1e-6 < err < 5e-2, err


def test_radial_encode_painn_closed_form():
    r = torch.tensor([[3.0, 4.0, 0.0], [0.0, 0.0, 2.0]], dtype=torch.float64)
    n, rmax = 7, 8.0
    enc = OL.radial_encode_painn(r, n, rmax)
    assert enc.shape == (2, 7)
    d = torch.tensor([5.0, 2.0], dtype=torch.float64)
    ks = [math.pi / rmax * (1 + m // 2) for m in range(4)]                 # hn = 4: frequencies 1,1,2,2
    expect = torch.stack([torch.cos(ks[0] * d), torch.cos(ks[1] * d), torch.cos(ks[2] * d), torch.cos(ks[3] * d),
                          torch.sin(ks[0] * d), torch.sin(ks[1] * d), torch.sin(ks[2] * d)], dim=-1)
    assert torch.allclose(enc, expect)


def test_sq_radial_encode_zeros_special_values_and_scalar_loop():
    """archs/diffuser_atoms14.py:32-48.  Column m is sin(c_m h)(sqrt(1/2) - h) with h = sqrt(1 + |r|^2 / rmax^2) and
    c_m = (pi / sqrt 2) exp(m n^-0.7): it vanishes where c_m h is a multiple of pi, which pins c_m and the
    normalisation of the length without restating the product."""
    n, rmax = 4, 7.0
    D = torch.float64
    # r = 0: h = 1, value sin(c_m) (sqrt(1/2) - 1)
    at0 = OL.sq_radial_encode(torch.zeros(1, 3, dtype=D), n, rmax)[0]
    for m in range(n):
        c = math.pi / math.sqrt(2.0) * math.exp(m * n ** -0.7)
        assert abs(float(at0[m]) - math.sin(c) * (math.sqrt(0.5) - 1.0)) < 1e-14
    # |r| = rmax: h = sqrt 2, c_0 h = pi, so column 0 vanishes; |r| = sqrt(7) rmax: h = 2 sqrt 2, c_0 h = 2 pi
    for length in (rmax, math.sqrt(7.0) * rmax):
        e = OL.sq_radial_encode(torch.tensor([[0.0, length, 0.0]], dtype=D), n, rmax)[0]
        assert abs(float(e[0])) < 1e-13
        assert abs(float(e[1])) > 1e-2                       # the other columns do not vanish there
    # column m vanishes at h = k sqrt(2) exp(-m n^-0.7) for integer k (taken where h >= 1)
    for m, k in ((1, 2), (2, 2), (3, 3), (3, 4)):
        h = k * math.sqrt(2.0) * math.exp(-m * n ** -0.7)
        assert h > 1.0
        length = rmax * math.sqrt(h * h - 1.0)
        e = OL.sq_radial_encode(torch.tensor([[length, 0.0, 0.0]], dtype=D), n, rmax)[0]
        assert abs(float(e[m])) < 1e-12, (m, k, float(e[m]))
    # the envelope alone: where sin(c_m h) = +-1 the value is +-(sqrt(1/2) - h); c_0 h = pi / 2 needs h < 1, so take
    # c_0 h = 3 pi / 2: h = 3 / sqrt 2
    h = 3.0 / math.sqrt(2.0)
    e = OL.sq_radial_encode(torch.tensor([[0.0, 0.0, rmax * math.sqrt(h * h - 1.0)]], dtype=D), n, rmax)[0]
    assert abs(float(e[0]) - (-1.0) * (math.sqrt(0.5) - h)) < 1e-13
    # a scalar loop over (edge, column) on leading dims of different sizes
    g = torch.Generator().manual_seed(5)
    r = torch.randn(3, 5, 3, generator=g, dtype=D) * 4
    enc = OL.sq_radial_encode(r, 6, 5.5)
    assert enc.shape == (3, 5, 6)
    for a in range(3):
        for b in range(5):
            x, y, z = (float(v) for v in r[a, b])
            h = math.sqrt(1.0 + (x * x + y * y + z * z) / (5.5 * 5.5))
            for m in range(6):
                c = math.pi / math.sqrt(2.0) * math.exp(m * 6 ** -0.7)
                assert abs(float(enc[a, b, m]) - math.sin(c * h) * (math.sqrt(0.5) - h)) < 1e-12


def test_radial_encode_edge_special_values_and_scalar_loop():
    """archs/diffuser_atoms5.py:25-30.  x = |r|^2 / rmax (the reference divides the squared length by rmax, not by
    rmax^2): all columns are 1 at r = 0, 0 from |r|^2 = rmax on, and cos(m pi / 2) 3/4 at |r|^2 = rmax / 4."""
    n, rmax = 6, 7.0
    D = torch.float64
    assert torch.equal(OL.radial_encode_edge(torch.zeros(2, 3, dtype=D), n, rmax), torch.ones(2, n, dtype=D))
    edge = torch.tensor([[math.sqrt(rmax), 0.0, 0.0], [0.0, 1.5 * math.sqrt(rmax), 0.0], [0.0, 0.0, rmax]], dtype=D)
    at_zero = OL.radial_encode_edge(edge, n, rmax)
    assert float(at_zero.abs().max()) < 1e-15              # |r|^2 >= rmax; with rmax^2 in the quotient none would vanish
    inside = OL.radial_encode_edge(torch.tensor([[0.0, 0.99 * math.sqrt(rmax), 0.0]], dtype=D), n, rmax)
    assert float(inside[0, 0]) > 1e-3                      # cos(0) (1 - 0.98): open just inside the envelope's zero
    quarter = OL.radial_encode_edge(torch.tensor([[0.0, 0.0, 0.5 * math.sqrt(rmax)]], dtype=D), n, rmax)[0]
    want = torch.tensor([1.0, 0.0, -1.0, 0.0, 1.0, 0.0], dtype=D) * 0.75
    assert float((quarter - want).abs().max()) < 1e-15
    g = torch.Generator().manual_seed(6)
    r = torch.randn(4, 3, 3, generator=g, dtype=D)
    enc = OL.radial_encode_edge(r, 5, 3.0)
    assert enc.shape == (4, 3, 5)
    for a in range(4):
        for b in range(3):
            x, y, z = (float(v) for v in r[a, b])
            xs = (x * x + y * y + z * z) / 3.0
            for m in range(5):
                assert abs(float(enc[a, b, m]) - math.cos(m * math.pi * math.sqrt(xs)) * max(0.0, 1.0 - xs)) < 1e-13


def test_tens_sigmoid_norm_and_direction():
    x = torch.randn(5, 4, 3, 3, dtype=torch.float64)
    y = OL.tens_sigmoid(2, x)
    nx, ny = x.flatten(-2).norm(dim=-1), y.flatten(-2).norm(dim=-1)
    assert torch.allclose(ny, nx / torch.sqrt(1 + nx ** 2))
    assert torch.allclose(y / ny[..., None, None], x / nx[..., None, None])


def test_scal_group_norm_equals_torch_group_norm():
    """With the nodes moved into the 'spatial' axis, torch's GroupNorm is the same reduction."""
    x = torch.randn(3, 50, 16, dtype=torch.float64)
    gamma, beta = torch.randn(16, dtype=torch.float64), torch.randn(16, dtype=torch.float64)
    ours = OL.scal_group_norm(x, 4, gamma, beta, 1.0)
    ref = torch.nn.functional.group_norm(x.transpose(1, 2), 4, gamma, beta, eps=1.0).transpose(1, 2)
    assert torch.allclose(ours, ref, atol=1e-12)


def test_tens_group_norm_brute_force():
    x = torch.randn(2, 7, 8, 3, dtype=torch.float64)
    gamma = torch.randn(8, 1, dtype=torch.float64)
    out = OL.tens_group_norm(1, x, 4, gamma, 1e-5)
    for b in range(2):
        for g in range(4):
            blk = x[b, :, 2 * g:2 * g + 2]                       # nodes x 2 channels x 3
            m2 = (blk ** 2).sum(-1).mean()
            expect = gamma[2 * g:2 * g + 2] * blk / torch.sqrt(1e-5 + m2)
            assert torch.allclose(out[b, :, 2 * g:2 * g + 2], expect)


def test_scatter_gather_brute_force():
    src = torch.tensor([0, 0, 2, 2, 2, 5])
    dst = torch.tensor([1, 2, 0, 5, 3, 2])
    x = torch.randn(1, 6, 3, dtype=torch.float64)
    gathered = OL.edges_read_dst(dst, x, 1, 6)
    out = OL.edges_reduce_src(src, gathered, 1, 6)
    expect = torch.zeros(6, 3, dtype=torch.float64)
    for s, d in zip(src.tolist(), dst.tolist()):
        expect[s] += x[0, d]
    assert torch.allclose(out[0], expect)


def _rand_mlp(din, dout, g, leaky=False):
    w = {"W1": torch.randn(dout if not leaky else 2 * din, din, generator=g, dtype=torch.float64) * 0.2}
    h = w["W1"].shape[0]
    w["b1"] = torch.randn(h, generator=g, dtype=torch.float64) * 0.1
    w["W2"] = torch.randn(h, h, generator=g, dtype=torch.float64) * 0.2
    w["b2"] = torch.randn(h, generator=g, dtype=torch.float64) * 0.1
    w["W3"] = torch.randn(dout, h, generator=g, dtype=torch.float64) * 0.2
    w["b3"] = torch.randn(dout, generator=g, dtype=torch.float64) * 0.1
    if leaky:
        w["W_direct"] = torch.randn(dout, din, generator=g, dtype=torch.float64) * 0.2
    return w


def _ring_graph(N):
    src = torch.arange(N).repeat_interleave(2)
    dst = torch.stack([(torch.arange(N) + 1) % N, (torch.arange(N) - 1) % N], 1).reshape(-1)
    return src, dst


def test_painn_message_single_edge_closed_form_and_equivariance():
    g = torch.Generator().manual_seed(3)
    n = 4
    w_dist, w_actv = _rand_mlp(n, 4 * n, g), _rand_mlp(n, 4 * n, g)
    N = 6
    src, dst = _ring_graph(N)
    pos = torch.randn(N, 3, generator=g, dtype=torch.float64)
    r_ij = pos[dst] - pos[src]
    x_a = torch.randn(1, N, n, generator=g, dtype=torch.float64)
    x_v = torch.randn(1, N, n, 3, generator=g, dtype=torch.float64)
    da, dv = OL.painn_message(src, dst, 1, N, x_a, x_v, r_ij, w_dist, w_actv, 5.0, n)
    # node 0 by hand from its two edges
    ea, ev = torch.zeros(n, dtype=torch.float64), torch.zeros(n, 3, dtype=torch.float64)
    for e in (0, 1):
        j = int(dst[e])
        filt = OL.mlp_silu(OL.radial_encode_painn(r_ij[e:e + 1], n, 5.0), w_dist)[0]
        p = filt * OL.mlp_silu(x_a[0, j:j + 1], w_actv)[0]
        u = r_ij[e] / torch.sqrt(0.1 + (r_ij[e] ** 2).sum())
        v = x_v[0, j]
        ev += v * p[:n, None] + torch.linalg.cross(v, u.expand(n, 3)) * p[n:2 * n, None] + u[None] * p[2 * n:3 * n, None]
        ea += p[3 * n:]
    assert torch.allclose(da[0, 0], ea) and torch.allclose(dv[0, 0], ev)
    # rotate inputs: scalars invariant, vectors co-rotate (the cross product needs a proper rotation)
    da_r, dv_r = OL.painn_message(src, dst, 1, N, x_a, x_v @ ROT, r_ij @ ROT, w_dist, w_actv, 5.0, n)
    assert torch.allclose(da_r, da, atol=1e-10) and torch.allclose(dv_r, dv @ ROT, atol=1e-10)


def test_painn_update_equivariance_and_squash_bound():
    g = torch.Generator().manual_seed(4)
    n = 8
    w = {"W_l": torch.randn(n, n, generator=g, dtype=torch.float64), "W_r": torch.randn(n, n, generator=g, dtype=torch.float64),
         "W_v": torch.randn(n, n, generator=g, dtype=torch.float64), "mlp": _rand_mlp(2 * n, 3 * n, g),
         "gn_gamma": torch.randn(n, generator=g, dtype=torch.float64), "gn_beta": torch.randn(n, generator=g, dtype=torch.float64)}
    x_a = torch.randn(2, 9, n, generator=g, dtype=torch.float64)
    x_v = torch.randn(2, 9, n, 3, generator=g, dtype=torch.float64)
    a, v = OL.painn_update(x_a, x_v, w, n)
    a_r, v_r = OL.painn_update(x_a, x_v @ ROT, w, n)
    assert torch.allclose(a_r, a, atol=1e-10) and torch.allclose(v_r, v @ ROT, atol=1e-10)
    assert torch.all(v.norm(dim=-1) < 1.0)                      # v / sqrt(1 + |v|^2)


def _rot(t, rank):
    if rank == 0:
        return t
    if rank == 1:
        return torch.einsum("...i,ij->...j", t, ROT)
    return torch.einsum("...ij,ia,jb->...ab", t, ROT, ROT)


def test_bee_messages_and_self_products_equivariance():
    g = torch.Generator().manual_seed(5)
    dim_a, dim_v, dim_d, chan, N = 6, 5, 4, 7, 8
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * 0.5
    Y = {lab: rn((dim_a, dim_v, dim_d)[int(lab[2])], chan) for lab in OP.BEE_ORDER}
    w = {"L0": rn(chan, dim_a), "L1": rn(chan, dim_v), "L2": rn(chan, dim_d), "Y": Y, "enc_W": rn(chan, 8),
         "enc_b": rn(chan), "mlp_a": _rand_mlp(dim_a, dim_a, g, leaky=True)}
    src, dst = _ring_graph(N)
    pos = rn(N, 3) * 4
    r_ij = pos[dst] - pos[src]
    x = [rn(1, N, dim_a), rn(1, N, dim_v, 3), rn(1, N, dim_d, 3, 3)]
    out = OL.bee_messages(src, dst, 1, N, r_ij, *x, w, 6.0)
    out_r = OL.bee_messages(src, dst, 1, N, r_ij @ ROT, *[_rot(t, k) for k, t in enumerate(x)], w, 6.0)
    for k in range(3):
        assert torch.allclose(out_r[k], _rot(out[k], k), atol=1e-10)
    ws = {k: rn(chan, d) for k, d in (("L0", dim_a), ("R0", dim_a), ("L1", dim_v), ("R1", dim_v), ("L2", dim_d), ("R2", dim_d))}
    ws.update(Y=Y, gn_a=rn(dim_a), gn_v=rn(dim_v, 1), gn_d=rn(dim_d, 1, 1))
    so = OL.self_tens_prods(*x, ws, groups=1)
    so_r = OL.self_tens_prods(*[_rot(t, k) for k, t in enumerate(x)], ws, groups=1)
    for k in range(3):
        assert torch.allclose(so_r[k], _rot(so[k], k), atol=1e-10)


def test_bee_messages_reduces_to_scalar_message_when_vectors_vanish():
    """With x_v = x_d = 0 only product 000 feeds the scalar output: B_a = 0.1 sum_j (u + mlp(u)),
    u = Y_000 (L0 x_a[j] * phi_a)."""
    g = torch.Generator().manual_seed(6)
    dim_a, chan, N = 5, 6, 7
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * 0.5
    Y = {lab: rn((dim_a, 3, 2)[int(lab[2])], chan) for lab in OP.BEE_ORDER}
    w = {"L0": rn(chan, dim_a), "L1": rn(chan, 3), "L2": rn(chan, 2), "Y": Y, "enc_W": rn(chan, 8), "enc_b": rn(chan),
         "mlp_a": _rand_mlp(dim_a, dim_a, g, leaky=True)}
    src, dst = _ring_graph(N)
    r_ij = rn(2 * N, 3) * 3
    x_a = rn(1, N, dim_a)
    B_a, B_v, B_d = OL.bee_messages(src, dst, 1, N, r_ij, x_a, torch.zeros(1, N, 3, 3, dtype=torch.float64),
                                    torch.zeros(1, N, 2, 3, 3, dtype=torch.float64), w, 6.0)
    phi = torch.nn.functional.linear(OL.radial_encode_8(r_ij, 6.0), w["enc_W"], w["enc_b"])
    u = ((x_a[0] @ w["L0"].T)[dst] * phi) @ Y["000"].T
    expect = torch.zeros(N, dim_a, dtype=torch.float64).index_add_(0, src, u + OL.mlp_leaky(u, w["mlp_a"]))
    assert torch.allclose(B_a[0], 0.1 * expect)


def test_displacement_tensors_closed_form_and_equivariance():
    """One edge per node along a known direction: A_a = phi, A_v = phi u, A_d = phi u u^T with
    u = s r / sqrt(1 + |s r|^2), s = 7 / r0, written out by hand; identity read-outs.  Then a ring graph under the
    reference's rotation: rank-k outputs rotate as rank-k tensors, and the sums are explicit loops over edges."""
    g = torch.Generator().manual_seed(8)
    dim_a, dim_v, dim_d, N, r0 = 5, 5, 5, 6, 6.0
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * 0.5
    w = {"lin_W": rn(dim_a, 8), "lin_b": rn(dim_a), "mlp": _rand_mlp(dim_a, dim_a, g, leaky=True),
         "readout_v": torch.eye(dim_a, dtype=torch.float64), "readout_d": torch.eye(dim_a, dtype=torch.float64)}
    src = torch.arange(N)
    r_ij = torch.zeros(N, 3, dtype=torch.float64)
    r_ij[:, 0] = torch.linspace(0.5, 5.5, N)                 # along x
    A_a, A_v, A_d = OL.displacement_tensors(src, 1, N, r_ij, w, r0)
    z = r_ij[:, 0] / r0
    enc = OL.radial_encode_8(r_ij, r0)
    assert torch.allclose(enc[:, 0], 1 - z) and torch.allclose(enc[:, 1], (3 * z - 1) * (1 - z))   # P0 = 1, P1 = 3z - 1
    phi = OL.mlp_leaky(enc @ w["lin_W"].T + w["lin_b"], w["mlp"])
    s = 7.0 / r0
    ux = s * r_ij[:, 0] / torch.sqrt(1 + (s * r_ij[:, 0]) ** 2)
    assert torch.allclose(A_a[0], phi)
    assert torch.allclose(A_v[0, :, :, 0], phi * ux[:, None]) and not bool(A_v[0, :, :, 1:].any())
    assert torch.allclose(A_d[0, :, :, 0, 0], phi * (ux ** 2)[:, None])
    assert not bool(A_d[0, :, :, 1:, :].any()) and not bool(A_d[0, :, :, :, 1:].any())
    # ring graph: explicit loops, read-outs mixing channels, rotation
    w["readout_v"], w["readout_d"] = rn(3, dim_a), rn(2, dim_a)
    src, dst = _ring_graph(N)
    pos = rn(N, 3) * 4
    r_ij = pos[dst] - pos[src]
    out = OL.displacement_tensors(src, 1, N, r_ij, w, r0)
    phi = OL.mlp_leaky(OL.radial_encode_8(r_ij, r0) @ w["lin_W"].T + w["lin_b"], w["mlp"])
    u = OL.tens_sigmoid(1, r_ij * s)
    A_v = torch.zeros(N, dim_a, 3, dtype=torch.float64)
    A_d = torch.zeros(N, dim_a, 3, 3, dtype=torch.float64)
    for e in range(2 * N):
        for c in range(dim_a):
            A_v[src[e], c] += phi[e, c] * u[e]
            A_d[src[e], c] += phi[e, c] * torch.outer(u[e], u[e])
    assert torch.allclose(out[1][0], torch.einsum("oc,ncx->nox", w["readout_v"], A_v))
    assert torch.allclose(out[2][0], torch.einsum("oc,ncxy->noxy", w["readout_d"], A_d))
    out_r = OL.displacement_tensors(src, 1, N, r_ij @ ROT, w, r0)
    for k in range(3):
        assert torch.allclose(out_r[k], _rot(out[k], k), atol=1e-10)


"""Pins the layer-level functions of the CPU oracle (oracle/layers.py) with statements of the reference's
formulas that share no code with it: scalar Python loops over (node / edge, channel, component) on sizes where
every axis differs, and block tests (all but one slice of an intermediate switched off, then a geometric property of
the output that only the right slice assignment has).

  archs/meanflow_painn8.py:63-75     Update.forward    -> OL.painn_update
  archs/meanflow_painn8.py:85-100    Message.forward   -> OL.painn_message
  archs/diffuser_atoms15.py:52-57    apply_tens_prod_submodules
  archs/diffuser_atoms15.py:75-95    SelfTensProds.forward -> OL.self_tens_prods
  archs/diffuser_atoms15.py:238-253  Messages.forward  -> OL.bee_messages

A swapped slice of y, |r| taken from lin_l, an l <-> r or L <-> R mix-up, a transposed phi_d or a psi sum over the
wrong labels each fail at least one assertion here (the mutation tests at the end of the file show it)."""
import math

import pytest
import torch

from oracle import layers as OL
from oracle import products as OP

F64 = torch.float64


def _rn(g, *shape, scale=1.0):
    return torch.randn(*shape, generator=g, dtype=F64) * scale


def _silu(x):
    return x / (1.0 + math.exp(-x))


def _leaky(x):
    return x if x > 0 else 0.1 * x


def _linear_scalar(W, b, x):
    """y[o] = sum_i W[o][i] x[i] + b[o] on Python lists."""
    return [sum(W[o][i] * x[i] for i in range(len(x))) + (b[o] if b is not None else 0.0) for o in range(len(W))]


def _mlp3_scalar(w, x, act):
    h = [act(v) for v in _linear_scalar(w["W1"].tolist(), w["b1"].tolist(), x)]
    h = [act(v) for v in _linear_scalar(w["W2"].tolist(), w["b2"].tolist(), h)]
    return _linear_scalar(w["W3"].tolist(), w["b3"].tolist(), h)


def _rand_mlp(din, dout, g, direct=False):
    w = {"W1": _rn(g, dout, din, scale=0.4), "b1": _rn(g, dout, scale=0.2), "W2": _rn(g, dout, dout, scale=0.4),
         "b2": _rn(g, dout, scale=0.2), "W3": _rn(g, dout, dout, scale=0.4), "b3": _rn(g, dout, scale=0.2)}
    if direct:
        w["W_direct"] = _rn(g, dout, din, scale=0.4)
    return w


def _eps(i, j, k):
    return (i - j) * (j - k) * (k - i) // 2


# ------------------------------------------------------------------------------------------------- Update
def _update_scalar(x_a, x_v, w, n):
    """archs/meanflow_painn8.py:63-75 as loops.  x_a (B,N,n), x_v (B,N,n,3) nested lists."""
    B, N = len(x_a), len(x_a[0])
    Wl, Wr, Wv = w["W_l"].tolist(), w["W_r"].tolist(), w["W_v"].tolist()
    gamma, beta = w["gn_gamma"].tolist(), w["gn_beta"].tolist()
    groups, per = 4, n // 4
    lin = lambda W, b_, i_, o, x: sum(W[o][c] * x_v[b_][i_][c][x] for c in range(n))
    out_a = [[[0.0] * n for _ in range(N)] for _ in range(B)]
    out_v = [[[[0.0] * 3 for _ in range(n)] for _ in range(N)] for _ in range(B)]
    pre_norm = [[[0.0] * n for _ in range(N)] for _ in range(B)]
    y_all = [[None] * N for _ in range(B)]
    for b in range(B):
        for i in range(N):
            l = [[lin(Wl, b, i, o, x) for x in range(3)] for o in range(n)]
            r = [[lin(Wr, b, i, o, x) for x in range(3)] for o in range(n)]
            v = [[lin(Wv, b, i, o, x) for x in range(3)] for o in range(n)]
            ip = [sum(l[o][x] * r[o][x] for x in range(3)) for o in range(n)]
            r_norm = [math.sqrt(sum(r[o][x] ** 2 for x in range(3))) for o in range(n)]      # |lin_r(x_v)|, not lin_l
            y = _mlp3_scalar(w["mlp"], list(x_a[b][i]) + r_norm, _silu)                      # cat order: x_a first
            y_all[b][i] = y
            for o in range(n):
                vv = [v[o][x] * y[o] for x in range(3)]                                       # slice [0, n)
                s = math.sqrt(1.0 + sum(t * t for t in vv))
                out_v[b][i][o] = [t / s for t in vv]
                pre_norm[b][i][o] = ip[o] * y[n + o]                                           # slice [n, 2n)
    for b in range(B):                                  # ScalGroupNorm(n, 4, epsilon=1): statistics over (nodes, chan/4)
        for gidx in range(groups):
            vals = [pre_norm[b][i][gidx * per + k] for i in range(N) for k in range(per)]
            mean = sum(vals) / len(vals)
            var = sum((t - mean) ** 2 for t in vals) / len(vals)
            for i in range(N):
                for k in range(per):
                    o = gidx * per + k
                    normed = beta[o] + gamma[o] * (pre_norm[b][i][o] - mean) / math.sqrt(1.0 + var)
                    out_a[b][i][o] = normed + y_all[b][i][2 * n + o]                           # slice [2n, 3n)
    return torch.tensor(out_a, dtype=F64), torch.tensor(out_v, dtype=F64)


def _update_inputs(seed=4, n=8, B=2, N=3):
    g = torch.Generator().manual_seed(seed)
    w = {"W_l": _rn(g, n, n, scale=0.5), "W_r": _rn(g, n, n, scale=0.5), "W_v": _rn(g, n, n, scale=0.5),
         "mlp": _rand_mlp(2 * n, 3 * n, g), "gn_gamma": _rn(g, n), "gn_beta": _rn(g, n)}
    return w, _rn(g, B, N, n), _rn(g, B, N, n, 3), n


def test_painn_update_against_scalar_loops():
    w, x_a, x_v, n = _update_inputs()
    a, v = OL.painn_update(x_a, x_v, w, n)
    ea, ev = _update_scalar(x_a.tolist(), x_v.tolist(), w, n)
    assert torch.allclose(a, ea, rtol=1e-12, atol=1e-12)
    assert torch.allclose(v, ev, rtol=1e-12, atol=1e-12)


def test_painn_update_slices_of_y_by_switching_blocks_off():
    """Last layer of the MLP with only one block of n output rows alive.  Block 0 scales lin_v(x_v); block 1
    multiplies the inner product before the norm; block 2 is added after it."""
    w, x_a, x_v, n = _update_inputs(seed=5)

    def only(block, base=None):
        base = w if base is None else base
        keep = torch.zeros(3 * n, 1, dtype=F64)
        keep[block * n:(block + 1) * n] = 1.0
        ww = dict(base, mlp=dict(base["mlp"], W3=base["mlp"]["W3"] * keep, b3=base["mlp"]["b3"] * keep[:, 0]))
        return OL.painn_update(x_a, x_v, ww, n)

    beta = w["gn_beta"]
    a0, v0 = only(0)
    assert v0.abs().max() > 1e-3 and torch.allclose(a0, beta.expand_as(a0))           # y[n:] = 0: GN(0) + 0 = beta
    a1, v1 = only(1)
    assert not v1.any() and not torch.allclose(a1, beta.expand_as(a1))
    # with gamma = 1, beta = 0 the output of block 1 alone is a group-normalised quantity: zero mean per (box, group)
    a1n, _ = only(1, dict(w, gn_gamma=torch.ones(n, dtype=F64), gn_beta=torch.zeros(n, dtype=F64)))
    assert torch.allclose(a1n.reshape(2, 3, 4, n // 4).mean(dim=(1, 3)), torch.zeros(2, 4, dtype=F64), atol=1e-12)
    a2, v2 = only(2)
    assert not v2.any()
    y = OL.mlp_silu(torch.cat([x_a, torch.linalg.vector_norm(OP.tensor_linear(1, w["W_r"], x_v), dim=-1)], -1), w["mlp"])
    assert torch.allclose(a2, beta + y[..., 2 * n:])
    # |r| comes from lin_r: with W_r = 0 the MLP sees zeros there and the inner product vanishes; with W_l = 0 only the
    # inner product vanishes
    a_r0, v_r0 = OL.painn_update(x_a, x_v, dict(w, W_r=torch.zeros(n, n, dtype=F64)), n)
    y_r0 = OL.mlp_silu(torch.cat([x_a, torch.zeros_like(x_a)], -1), w["mlp"])
    assert torch.allclose(a_r0, beta + y_r0[..., 2 * n:])
    a_l0, _ = OL.painn_update(x_a, x_v, dict(w, W_l=torch.zeros(n, n, dtype=F64)), n)
    assert torch.allclose(a_l0, beta + y[..., 2 * n:]) and not torch.allclose(a_l0, a_r0)


# ------------------------------------------------------------------------------------------------ Message
def _radial_scalar(d, n_rbf, r0):
    hn = (n_rbf + 1) // 2
    k = [(math.pi / r0) * (1 + m // 2) for m in range(hn)]
    return [math.cos(k[m] * d) for m in range(hn)] + [math.sin(k[m] * d) for m in range(n_rbf - hn)]


def _message_scalar(src, dst, N, x_a, x_v, r_ij, w_dist, w_actv, r0, n, n_rbf, epsilon=0.1):
    """archs/meanflow_painn8.py:85-100 as loops over (edge, channel, component); cross(v, u) written out."""
    out_a = [[0.0] * n for _ in range(N)]
    out_v = [[[0.0] * 3 for _ in range(n)] for _ in range(N)]
    for e in range(len(src)):
        i, j = src[e], dst[e]
        r = r_ij[e]
        d = math.sqrt(r[0] ** 2 + r[1] ** 2 + r[2] ** 2)
        filt = _mlp3_scalar(w_dist, _radial_scalar(d, n_rbf, r0), _silu)
        actv = _mlp3_scalar(w_actv, list(x_a[j]), _silu)
        p = [filt[k] * actv[k] for k in range(4 * n)]
        s = math.sqrt(epsilon + d * d)
        u = [r[0] / s, r[1] / s, r[2] / s]
        for c in range(n):
            v = x_v[j][c]
            cross = [v[1] * u[2] - v[2] * u[1], v[2] * u[0] - v[0] * u[2], v[0] * u[1] - v[1] * u[0]]
            for x in range(3):
                out_v[i][c][x] += v[x] * p[c] + cross[x] * p[n + c] + u[x] * p[2 * n + c]
            out_a[i][c] += p[3 * n + c]
    return torch.tensor(out_a, dtype=F64), torch.tensor(out_v, dtype=F64)


def _message_inputs(seed, n=3, n_rbf=5, N=5):
    g = torch.Generator().manual_seed(seed)
    src = torch.tensor([0, 0, 1, 2, 2, 2, 4])                      # node 3 has no edge; rows of 2, 1, 3, 0, 1 edges
    dst = torch.tensor([1, 4, 0, 0, 1, 3, 2])
    return (src, dst, _rn(g, 1, N, n), _rn(g, 1, N, n, 3), _rn(g, len(src), 3, scale=2.0),
            _rand_mlp(n_rbf, 4 * n, g), _rand_mlp(n, 4 * n, g), n, n_rbf, N)


def test_painn_message_against_scalar_loops():
    src, dst, x_a, x_v, r_ij, w_dist, w_actv, n, n_rbf, N = _message_inputs(11)
    da, dv = OL.painn_message(src, dst, 1, N, x_a, x_v, r_ij, w_dist, w_actv, 5.0, n, n_rbf)
    ea, ev = _message_scalar(src.tolist(), dst.tolist(), N, x_a[0].tolist(), x_v[0].tolist(), r_ij.tolist(), w_dist,
                             w_actv, 5.0, n, n_rbf)
    assert torch.allclose(da[0], ea, rtol=1e-12, atol=1e-12) and torch.allclose(dv[0], ev, rtol=1e-12, atol=1e-12)
    assert not da[0, 3].any() and not dv[0, 3].any()


def test_painn_message_slices_of_the_filter_by_switching_blocks_off():
    """Filter MLP with only one block of n output rows alive, on a graph with ONE edge per node, so that each
    node's output is a single edge's message and its geometry can be read off: block 0 gives a vector parallel to
    x_v[j]; block 1 one perpendicular to both x_v[j] and the edge, with the orientation of x_v[j] x u; block 2 one
    parallel to the edge; block 3 feeds only the scalar output."""
    g = torch.Generator().manual_seed(12)
    n, n_rbf, N = 3, 4, 4
    src, dst = torch.arange(N), torch.tensor([2, 3, 1, 0])
    x_a, x_v, r_ij = _rn(g, 1, N, n), _rn(g, 1, N, n, 3), _rn(g, N, 3, scale=2.0)
    w_dist, w_actv = _rand_mlp(n_rbf, 4 * n, g), _rand_mlp(n, 4 * n, g)

    def only(block):
        keep = torch.zeros(4 * n, 1, dtype=F64)
        keep[block * n:(block + 1) * n] = 1.0
        wd = dict(w_dist, W3=w_dist["W3"] * keep, b3=w_dist["b3"] * keep[:, 0])
        return OL.painn_message(src, dst, 1, N, x_a, x_v, r_ij, wd, w_actv, 5.0, n, n_rbf)

    p = OL.mlp_silu(OL.radial_encode_painn(r_ij, n_rbf, 5.0), w_dist) * OL.mlp_silu(x_a[0][dst], w_actv)   # (E, 4n)
    u = r_ij / torch.sqrt(0.1 + (r_ij ** 2).sum(-1, keepdim=True))
    vj = x_v[0][dst]
    a, v = only(0)
    assert not a.any() and torch.allclose(v[0], vj * p[:, 0:n, None])
    a, v = only(1)
    assert not a.any()
    assert torch.allclose((v[0] * vj).sum(-1), torch.zeros(N, n, dtype=F64), atol=1e-12)
    assert torch.allclose((v[0] * u[:, None]).sum(-1), torch.zeros(N, n, dtype=F64), atol=1e-12)
    for e in range(N):
        for c in range(n):      # orientation and size: triple product (v_j, u, out) = |v_j x u|^2 p
            vx = vj[e, c].tolist()
            ux = u[e].tolist()
            cr = [vx[1] * ux[2] - vx[2] * ux[1], vx[2] * ux[0] - vx[0] * ux[2], vx[0] * ux[1] - vx[1] * ux[0]]
            want = [t * float(p[e, n + c]) for t in cr]
            assert torch.allclose(v[0, e, c], torch.tensor(want, dtype=F64), atol=1e-12)
    a, v = only(2)
    assert not a.any() and torch.allclose(v[0], u[:, None, :] * p[:, 2 * n:3 * n, None])
    a, v = only(3)
    assert not v.any() and torch.allclose(a[0], p[:, 3 * n:])


# ------------------------------------------------------------------------------- the 13 products as loops
def _product_scalar(lab, l, r):
    """One (row, channel) element of product `lab` (ranks of left, right, output); contracted indices are the
    trailing ones of both operands, kept left indices come first in the output (extensions/codegen_tensops/
    codegen.py:281-350).  l, r: float | list[3] | list[3][3]."""
    R = range(3)
    if lab == "000": return l * r
    if lab == "110": return sum(l[x] * r[x] for x in R)
    if lab == "220": return sum(l[x][y] * r[x][y] for x in R for y in R)
    if lab == "011": return [l * r[x] for x in R]
    if lab == "101": return [l[x] * r for x in R]
    if lab == "121": return [sum(l[x] * r[y][x] for x in R) for y in R]
    if lab == "211": return [sum(l[x][y] * r[y] for y in R) for x in R]
    if lab == "022": return [[l * r[x][y] for y in R] for x in R]
    if lab == "202": return [[l[x][y] * r for y in R] for x in R]
    if lab == "112": return [[l[x] * r[y] for y in R] for x in R]
    if lab == "222": return [[sum(l[x][y] * r[z][y] for y in R) for z in R] for x in R]
    if lab == "111": return [sum(_eps(x, y, z) * l[x] * r[y] for x in R for y in R) for z in R]
    if lab == "212": return [[sum(_eps(y, z, w) * l[x][y] * r[z] for y in R for z in R) for w in R] for x in R]
    raise KeyError(lab)


def test_scalar_products_agree_with_the_oracle_products():
    g = torch.Generator().manual_seed(13)
    rows, chan = 2, 3
    l = [_rn(g, rows, chan), _rn(g, rows, chan, 3), _rn(g, rows, chan, 3, 3)]
    r = [_rn(g, rows, chan), _rn(g, rows, chan, 3), _rn(g, rows, chan, 3, 3)]
    for lab, got in zip(OP.BEE_ORDER, OP.bee(*l, *r)):
        ll, rr = l[int(lab[0])], r[int(lab[1])]
        want = [[_product_scalar(lab, ll[b, c].tolist(), rr[b, c].tolist()) for c in range(chan)] for b in range(rows)]
        assert torch.allclose(got, torch.tensor(want, dtype=F64), rtol=1e-13, atol=1e-13), lab


def _tens_linear_scalar(W, x, rank):
    """y[o, comps] = sum_c W[o][c] x[c, comps] on nested lists."""
    if rank == 0:
        return [sum(W[o][c] * x[c] for c in range(len(x))) for o in range(len(W))]
    if rank == 1:
        return [[sum(W[o][c] * x[c][a] for c in range(len(x))) for a in range(3)] for o in range(len(W))]
    return [[[sum(W[o][c] * x[c][a][b] for c in range(len(x))) for b in range(3)] for a in range(3)] for o in range(len(W))]


def _apply_Y_scalar(Y, l, r, chan):
    """psi_k = sum over the labels with output rank k of Y_lab(prod_lab(l, r)) (archs/diffuser_atoms15.py:52-57):
    rank 0 from 000, 110, 220; rank 1 from 011, 101, 121, 211, 111; rank 2 from 022, 202, 112, 222, 212."""
    out = [None, None, None]
    for lab in ("000", "110", "220", "011", "101", "121", "211", "111", "022", "202", "112", "222", "212"):
        lk, rk, ok = int(lab[0]), int(lab[1]), int(lab[2])
        prod = [_product_scalar(lab, l[lk][c], r[rk][c]) for c in range(chan)]
        t = torch.tensor(_tens_linear_scalar(Y[lab].tolist(), prod, ok), dtype=F64)
        out[ok] = t if out[ok] is None else out[ok] + t
    return out


# ----------------------------------------------------------------------------------------- SelfTensProds
def _self_inputs(seed=21, dims=(4, 3, 2), chan=5, B=2, N=3):
    g = torch.Generator().manual_seed(seed)
    dim_a, dim_v, dim_d = dims
    w = {"L0": _rn(g, chan, dim_a), "R0": _rn(g, chan, dim_a), "L1": _rn(g, chan, dim_v), "R1": _rn(g, chan, dim_v),
         "L2": _rn(g, chan, dim_d), "R2": _rn(g, chan, dim_d),
         "Y": {lab: _rn(g, dims[int(lab[2])], chan, scale=0.5) for lab in OP.BEE_ORDER},
         "gn_a": _rn(g, dim_a), "gn_v": _rn(g, dim_v, 1), "gn_d": _rn(g, dim_d, 1, 1)}
    return w, _rn(g, B, N, dim_a), _rn(g, B, N, dim_v, 3), _rn(g, B, N, dim_d, 3, 3), dims, chan


def _tens_group_norm_scalar(y, gamma, groups, rank, eps=1e-5):
    """managan/tensor_products.py:215-232: per (box, group) mean over (nodes, channels of the group) of the sum of
    squares over components; x * gamma / sqrt(eps + m2); no mean subtraction, no beta.  y: (B, N, dim, 3..)."""
    B, N, dim = y.shape[:3]
    per = dim // groups
    out = torch.zeros_like(y)
    flat = y.reshape(B, N, dim, -1)
    for b in range(B):
        for gi in range(groups):
            tot = 0.0
            for i in range(N):
                for k in range(per):
                    tot += sum(float(t) ** 2 for t in flat[b, i, gi * per + k])
            m2 = tot / (N * per)
            for i in range(N):
                for k in range(per):
                    o = gi * per + k
                    out[b, i, o] = y[b, i, o] * float(gamma.reshape(-1)[o]) / math.sqrt(eps + m2)
    return out


def _self_scalar(x_a, x_v, x_d, w, dims, chan, groups):
    B, N = x_a.shape[:2]
    ys = [torch.zeros(B, N, dims[0], dtype=F64), torch.zeros(B, N, dims[1], 3, dtype=F64),
          torch.zeros(B, N, dims[2], 3, 3, dtype=F64)]
    for b in range(B):
        for i in range(N):
            xs = [x_a[b, i].tolist(), x_v[b, i].tolist(), x_d[b, i].tolist()]
            l = [_tens_linear_scalar(w[f"L{k}"].tolist(), xs[k], k) for k in range(3)]    # left operands from L_k
            r = [_tens_linear_scalar(w[f"R{k}"].tolist(), xs[k], k) for k in range(3)]    # right operands from R_k
            for k, t in enumerate(_apply_Y_scalar(w["Y"], l, r, chan)):
                ys[k][b, i] = t
    return [_tens_group_norm_scalar(ys[k], w[("gn_a", "gn_v", "gn_d")[k]], groups, k) for k in range(3)]


@pytest.mark.parametrize("groups", [1, 2])
def test_self_tens_prods_against_scalar_loops(groups):
    dims = (4, 2, 2) if groups == 2 else (4, 3, 2)
    w, x_a, x_v, x_d, dims, chan = _self_inputs(dims=dims)
    got = OL.self_tens_prods(x_a, x_v, x_d, w, groups=groups)
    want = _self_scalar(x_a, x_v, x_d, w, dims, chan, groups)
    for k in range(3):
        assert torch.allclose(got[k], want[k], rtol=1e-11, atol=1e-12), k


# ---------------------------------------------------------------------------------------------- Messages
def _jacobi_10_scalar(i, t):
    """P_i^{(1,0)}(t) from the three-term recurrence of the Jacobi polynomials (a = 1, b = 0), independent of the
    closed-form coefficient table the oracle builds."""
    a, b = 1.0, 0.0
    p_prev, p = 1.0, 0.5 * ((a + b + 2) * t + (a - b))
    if i == 0:
        return p_prev
    for n in range(1, i):
        c = 2 * n + a + b
        a1 = 2 * (n + 1) * (n + a + b + 1) * c
        a2 = (c + 1) * (a * a - b * b)
        a3 = c * (c + 1) * (c + 2)
        a4 = 2 * (n + a) * (n + b) * (c + 2)
        p_prev, p = p, ((a2 + a3 * t) * p - a4 * p_prev) / a1
    return p


def _messages_scalar(src, dst, N, r_ij, x_a, x_v, x_d, w, r0, dims, chan):
    """archs/diffuser_atoms15.py:238-253 as loops over edges."""
    La = [_tens_linear_scalar(w["L0"].tolist(), x_a[i].tolist(), 0) for i in range(N)]
    Lv = [_tens_linear_scalar(w["L1"].tolist(), x_v[i].tolist(), 1) for i in range(N)]
    Ld = [_tens_linear_scalar(w["L2"].tolist(), x_d[i].tolist(), 2) for i in range(N)]
    outs = [torch.zeros(N, dims[0], dtype=F64), torch.zeros(N, dims[1], 3, dtype=F64), torch.zeros(N, dims[2], 3, 3, dtype=F64)]
    for e in range(len(src)):
        i, j = src[e], dst[e]
        r = r_ij[e].tolist()
        d = math.sqrt(sum(t * t for t in r))
        z = d / r0
        enc = [_jacobi_10_scalar(k, 2 * z - 1) * max(1 - z, 0.0) for k in range(8)]
        phi_a = _linear_scalar(w["enc_W"].tolist(), w["enc_b"].tolist(), enc)
        sr = [t * 7.0 / r0 for t in r]
        s = math.sqrt(1.0 + sum(t * t for t in sr))
        rh = [t / s for t in sr]
        phi_v = [[phi_a[c] * rh[x] for x in range(3)] for c in range(chan)]
        phi_d = [[[phi_a[c] * rh[y] * rh[x] for y in range(3)] for x in range(3)] for c in range(chan)]
        psi = _apply_Y_scalar(w["Y"], [La[j], Lv[j], Ld[j]], [phi_a, phi_v, phi_d], chan)      # left = gathered node
        m = w["mlp_a"]
        mlp = _mlp3_scalar(m, psi[0].tolist(), _leaky)
        direct = _linear_scalar(m["W_direct"].tolist(), None, psi[0].tolist())
        psi[0] = psi[0] + torch.tensor(mlp, dtype=F64) + torch.tensor(direct, dtype=F64)
        for k in range(3):
            outs[k][i] += 0.1 * psi[k]
    return outs


def _messages_inputs(seed=31, dims=(4, 3, 2), chan=5, N=5):
    g = torch.Generator().manual_seed(seed)
    dim_a, dim_v, dim_d = dims
    w = {"L0": _rn(g, chan, dim_a), "L1": _rn(g, chan, dim_v), "L2": _rn(g, chan, dim_d),
         "Y": {lab: _rn(g, dims[int(lab[2])], chan, scale=0.5) for lab in OP.BEE_ORDER},
         "enc_W": _rn(g, chan, 8, scale=0.5), "enc_b": _rn(g, chan, scale=0.5)}
    m = _rand_mlp(dim_a, 2 * dim_a, g)
    # diffuser_atoms15.MLP: dim -> 2 dim -> 2 dim -> dim plus a bias-free direct linear
    m["W3"], m["b3"] = _rn(g, dim_a, 2 * dim_a, scale=0.4), _rn(g, dim_a, scale=0.2)
    m["W_direct"] = _rn(g, dim_a, dim_a, scale=0.4)
    w["mlp_a"] = m
    src = torch.tensor([0, 0, 1, 2, 2, 2, 4])
    dst = torch.tensor([1, 4, 0, 0, 1, 3, 2])
    r_ij = _rn(g, len(src), 3, scale=2.0)
    return w, src, dst, r_ij, _rn(g, 1, N, dim_a), _rn(g, 1, N, dim_v, 3), _rn(g, 1, N, dim_d, 3, 3), dims, chan, N


def test_bee_messages_against_scalar_loops():
    w, src, dst, r_ij, x_a, x_v, x_d, dims, chan, N = _messages_inputs()
    got = OL.bee_messages(src, dst, 1, N, r_ij, x_a, x_v, x_d, w, 6.0)
    want = _messages_scalar(src.tolist(), dst.tolist(), N, r_ij, x_a[0], x_v[0], x_d[0], w, 6.0, dims, chan)
    for k in range(3):
        assert torch.allclose(got[k][0], want[k], rtol=1e-10, atol=1e-11), k
        assert not got[k][0, 3].any()


# --------------------------------------------------- the pins above do catch the slips they are there for
def test_scalar_pins_detect_plausible_slips():
    """Each mutation is a mistake a restatement could plausibly contain; every one moves the result of the scalar
    statement far outside the agreement asserted above."""
    w, x_a, x_v, n = _update_inputs()
    a, v = OL.painn_update(x_a, x_v, w, n)
    slips = {"l<->r": dict(w, W_l=w["W_r"], W_r=w["W_l"]),                                 # |r| from lin_l
             "y slices rotated": dict(w, mlp=dict(w["mlp"], W3=torch.roll(w["mlp"]["W3"], n, 0),
                                                  b3=torch.roll(w["mlp"]["b3"], n, 0)))}
    for name, ww in slips.items():
        ea, ev = _update_scalar(x_a.tolist(), x_v.tolist(), ww, n)
        assert not (torch.allclose(a, ea, atol=1e-6) and torch.allclose(v, ev, atol=1e-6)), name
    w, x_a, x_v, x_d, dims, chan = _self_inputs()
    got = OL.self_tens_prods(x_a, x_v, x_d, w, groups=1)
    swapped = dict(w, L0=w["R0"], R0=w["L0"], L1=w["R1"], R1=w["L1"], L2=w["R2"], R2=w["L2"])
    want = _self_scalar(x_a, x_v, x_d, swapped, dims, chan, 1)
    assert not all(torch.allclose(got[k], want[k], atol=1e-6) for k in range(3)), "L<->R"
    y_swapped = dict(w, Y=dict(w["Y"], **{"011": w["Y"]["101"], "101": w["Y"]["011"]}))
    want = _self_scalar(x_a, x_v, x_d, y_swapped, dims, chan, 1)
    assert not torch.allclose(got[1], want[1], atol=1e-6), "Y_011<->Y_101"

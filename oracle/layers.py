"""TEST INFRASTRUCTURE ONLY — CPU restatement (PyTorch) of the layer math that
calls the hot path.  Functional style: every function takes explicit weight
tensors so the same weights can be fed to the HIP modules and to this file.

Follows (relative to the reference checkout):
  managan/graph_layers.py:37-59            gather to edges, sum edges -> src nodes (segment_coo)
  managan/graph_layers.py:62-66            boxwrap (floor-mod)
  archs/meanflow_painn8.py:25-35           PaiNN radial_encode (duplicated-frequency cos|sin)
  archs/meanflow_painn8.py:38-51           MLP = Linear,SiLU,Linear,SiLU,Linear
  archs/meanflow_painn8.py:53-75           Update
  archs/meanflow_painn8.py:77-100          Message
  managan/jacobi_radenc.py:8-37            radial_encode_8 (shifted Jacobi(1,0) x relu(1-z))
  archs/diffuser_atoms14.py:32-48          normed_sq_dist, sq_radial_encode, radial_encode (hyperbolic distance)
  archs/diffuser_atoms5.py:25-30           radial_encode_edge (cosines x relu(1 - |r|^2 / rmax))
  managan/tensor_products.py:167-182       tens_sigmoid
  managan/tensor_products.py:215-232       TensGroupNorm
  managan/layers_common.py:201-223         ScalGroupNorm
  archs/diffuser_atoms15.py:29-57          the 13 Y_* linears and their sums
  archs/diffuser_atoms15.py:59-95          SelfTensProds
  archs/diffuser_atoms15.py:98-110         MLP with direct path and LeakyReLU(0.1)
  archs/diffuser_atoms15.py:206-225        DisplacementTensors
  archs/diffuser_atoms15.py:227-253        Messages (Bee)
"""
import math
import torch
import torch.nn.functional as F

from . import products as P


# ------------------------------------------------------------------ graph ops
def edges_read_dst(dst, x_node, batch, nodes):
    rest = x_node.shape[2:]
    return x_node.reshape(batch * nodes, *rest)[dst]


def edges_reduce_src(src, x_edge, batch, nodes):
    """out[s] = sum of x_edge[e] over edges with src[e] == s."""
    rest = x_edge.shape[1:]
    out = torch.zeros(batch * nodes, *rest, dtype=x_edge.dtype)
    out.index_add_(0, src, x_edge)
    return out.reshape(batch, nodes, *rest)


def boxwrap(box, delta_pos):
    return (delta_pos + 0.5 * box) % box - 0.5 * box


# ------------------------------------------------------------ radial encodings
def radial_encode_painn(r, n, rmax):
    hn = (n + 1) // 2
    coeffs = (math.pi / rmax) * (1 + torch.arange(0, hn) // 2).to(r.dtype)
    dist = torch.linalg.vector_norm(r, dim=-1)[..., None]
    phase = coeffs * dist
    return torch.cat([torch.cos(phase), torch.sin(phase[..., :(n - hn)])], dim=-1)


def _shifted_jacobi_10_coeffs(n):
    """Coefficients (ascending powers of x) of P_n^{(1,0)}(2x-1).

    Closed form: P_n^{(a,b)}(t) = sum_s C(n+a, n-s) C(n+b, s) ((t-1)/2)^s ((t+1)/2)^(n-s);
    with t = 2x-1: (t-1)/2 = x-1, (t+1)/2 = x."""
    from math import comb
    coeffs = [0.0] * (n + 1)
    for s in range(n + 1):
        w = comb(n + 1, n - s) * comb(n, s)
        # (x-1)^s x^(n-s) = sum_k C(s,k) (-1)^(s-k) x^(k + n - s)
        for k in range(s + 1):
            coeffs[k + n - s] += w * comb(s, k) * (-1.0) ** (s - k)
    return coeffs


def jacobi_matrix(dim, dtype=torch.float32):
    A = torch.zeros(dim, dim + 1, dtype=dtype)
    for i in range(dim):
        c = _shifted_jacobi_10_coeffs(i)
        for j, v in enumerate(c):
            A[i, j] = v
    return A


def radial_encode_8(r, rmax):
    A = jacobi_matrix(8, r.dtype)
    z = (torch.linalg.vector_norm(r, dim=-1) / rmax)[..., None]
    pows = z ** torch.arange(A.shape[1])
    return F.linear(pows, A) * torch.relu(1.0 - z)


def sq_radial_encode(r, n, rmax):
    """archs/diffuser_atoms14.py:32-48 (radial_encode = sq_radial_encode o normed_sq_dist): with q = |r|^2 / rmax^2 and
    h = sqrt(1 + q), column m is sin(c_m h) (sqrt(1/2) - h), c_m = (pi / sqrt 2) exp(m n^-0.7).  r: (..., 3) -> (..., n)."""
    sq_dist = (r ** 2).sum(-1, keepdim=True) / rmax ** 2
    coeffs = (math.pi * 2 ** -0.5) * torch.exp(n ** -0.7 * torch.arange(0, n, dtype=r.dtype))
    hyperdist = torch.sqrt(1 + sq_dist)
    return torch.sin(coeffs * hyperdist) * (0.5 ** 0.5 - hyperdist)


def radial_encode_edge(r, n, rmax):
    """archs/diffuser_atoms5.py:25-30: column m is cos(m pi sqrt(x)) relu(1 - x) with x = |r|^2 / rmax.  The squared
    length is divided by rmax, not by rmax^2: the envelope reaches zero at |r| = sqrt(rmax), as in the reference.
    r: (..., 3) -> (..., n)."""
    npi = math.pi * torch.arange(0, n, dtype=r.dtype)
    x_sq = (r ** 2).sum(-1) / rmax
    return torch.cos(npi * torch.sqrt(x_sq)[..., None]) * torch.relu(1. - x_sq)[..., None]


# ---------------------------------------------------------- norms and squashes
def tens_sigmoid(inds, x):
    dims = tuple(-(1 + n) for n in range(inds))
    xx = (x ** 2).sum(dims, keepdim=True) if inds > 0 else x ** 2
    return x / torch.sqrt(1.0 + xx)


def scal_group_norm(x, groups, gamma, beta, eps):
    batch, nodes, chan = x.shape
    xg = x.reshape(batch, nodes, groups, -1)
    mean = xg.mean([1, 3], keepdim=True)
    sh = xg - mean
    var = (sh ** 2).mean([1, 3], keepdim=True)
    ans = sh / torch.sqrt(eps + var)
    return beta + gamma * ans.reshape(batch, nodes, chan)


def tens_group_norm(inds, x, groups, gamma, eps=1e-5):
    """gamma: (chan, 1.. ) broadcastable; no mean subtraction, no beta."""
    batch, nodes, chan = x.shape[:3]
    xg = x.reshape(batch, nodes, groups, -1, 3 ** inds)
    m2 = (xg ** 2).sum(-1, keepdim=True).mean([1, 3], keepdim=True)
    ans = xg / torch.sqrt(eps + m2)
    return gamma * ans.reshape(batch, nodes, chan, *([3] * inds))


# ----------------------------------------------------------------------- PaiNN
def mlp_silu(x, w):
    """w: dict with W1,b1,W2,b2,W3,b3 (nn.Linear convention: y = x W^T + b)."""
    h = F.silu(F.linear(x, w["W1"], w["b1"]))
    h = F.silu(F.linear(h, w["W2"], w["b2"]))
    return F.linear(h, w["W3"], w["b3"])


def painn_message(src, dst, batch, nodes, x_a, x_v, r_ij, w_dist, w_actv, r0, n, n_rbf=None,
                  epsilon=0.1):
    """Returns (dx_a (B,N,n), dx_v (B,N,n,3))."""
    n_rbf = n if n_rbf is None else n_rbf
    filt = mlp_silu(radial_encode_painn(r_ij, n_rbf, r0), w_dist)       # (E, 4n)
    actv = mlp_silu(edges_read_dst(dst, x_a, batch, nodes), w_actv)     # (E, 4n)
    p = filt * actv
    direction = r_ij / torch.sqrt(epsilon + (r_ij ** 2).sum(-1, keepdim=True))
    v = edges_read_dst(dst, x_v, batch, nodes)                          # (E, n, 3)
    cross = torch.linalg.cross(v, direction[:, None].expand_as(v))
    m_v = v * p[..., :n, None]
    m_v = m_v + cross * p[..., n:2 * n, None]
    m_v = m_v + direction[:, None] * p[..., 2 * n:3 * n, None]
    return (edges_reduce_src(src, p[..., 3 * n:], batch, nodes),
            edges_reduce_src(src, m_v, batch, nodes))


def painn_update(x_a, x_v, w, n):
    """w: W_l, W_r, W_v (TensLinear, (n,n)), mlp (dict), gn_gamma, gn_beta."""
    v_l = P.tensor_linear(1, w["W_l"], x_v)
    v_r = P.tensor_linear(1, w["W_r"], x_v)
    ip = (v_l * v_r).sum(-1)
    y = mlp_silu(torch.cat([x_a, torch.linalg.vector_norm(v_r, dim=-1)], dim=-1), w["mlp"])
    v = P.tensor_linear(1, w["W_v"], x_v) * y[..., :n, None]
    ip = scal_group_norm(ip * y[..., n:2 * n], 4, w["gn_gamma"], w["gn_beta"], 1.0)
    a = ip + y[..., 2 * n:]
    v = v / torch.sqrt(1.0 + (v ** 2).sum(-1, keepdim=True))
    return a, v


# ------------------------------------------------------------------ Bee blocks
def mlp_leaky(x, w):
    """lin_direct(x) + [Linear(d,2d), LeakyReLU(.1), Linear(2d,2d), LeakyReLU(.1), Linear(2d,d)](x)."""
    h = F.leaky_relu(F.linear(x, w["W1"], w["b1"]), 0.1)
    h = F.leaky_relu(F.linear(h, w["W2"], w["b2"]), 0.1)
    return F.linear(x, w["W_direct"]) + F.linear(h, w["W3"], w["b3"])


def apply_Y(prods, Y):
    """Y: dict label -> (dim_out, chan).  Returns (y_0, y_1, y_2)."""
    out = [None, None, None]
    for lab, p in zip(P.BEE_ORDER, prods):
        o = int(lab[2])
        t = P.tensor_linear(o, Y[lab], p)
        out[o] = t if out[o] is None else out[o] + t
    return tuple(out)


def bee_messages(src, dst, batch, nodes, r_ij, x_a, x_v, x_d, w, r0, radial_dtype=None):
    """w: L0,L1,L2, Y (dict), enc_W (chan,8), enc_b (chan), mlp_a (dict).  radial_dtype: evaluate radial_encode_8 in
    that dtype and round once (its fp32 monomial form carries ~1e-3 of rounding noise of its own, which would
    otherwise dominate every fp32 evaluation of this function)."""
    enc8 = radial_encode_8(r_ij, r0) if radial_dtype is None else radial_encode_8(r_ij.to(radial_dtype), r0).to(r_ij.dtype)
    enc = F.linear(enc8, w["enc_W"], w["enc_b"])      # (E, chan)
    rh = tens_sigmoid(1, r_ij * (7.0 / r0))
    phi_a = enc
    phi_v = enc[..., None] * rh[..., None, :]
    phi_d = enc[..., None, None] * rh[..., None, None, :] * rh[..., None, :, None]
    a_j = edges_read_dst(dst, P.tensor_linear(0, w["L0"], x_a), batch, nodes)
    v_j = edges_read_dst(dst, P.tensor_linear(1, w["L1"], x_v), batch, nodes)
    d_j = edges_read_dst(dst, P.tensor_linear(2, w["L2"], x_d), batch, nodes)
    prods = P.bee(a_j, v_j, d_j, phi_a, phi_v, phi_d)
    psi_a, psi_v, psi_d = apply_Y(prods, w["Y"])
    psi_a = psi_a + mlp_leaky(psi_a, w["mlp_a"])
    return (0.1 * edges_reduce_src(src, psi_a, batch, nodes),
            0.1 * edges_reduce_src(src, psi_v, batch, nodes),
            0.1 * edges_reduce_src(src, psi_d, batch, nodes))


def displacement_tensors(src, batch, nodes, r_ij, w, r0, radial_dtype=None):
    """DisplacementTensors.forward (archs/diffuser_atoms15.py:216-225).  w: lin_W (dim_a, 8), lin_b (dim_a),
    mlp (dict for mlp_leaky, dim_a -> dim_a), readout_v (dim_v, dim_a), readout_d (dim_d, dim_a).
    radial_dtype: as in bee_messages."""
    enc8 = radial_encode_8(r_ij, r0) if radial_dtype is None else radial_encode_8(r_ij.to(radial_dtype), r0).to(r_ij.dtype)
    rad = mlp_leaky(F.linear(enc8, w["lin_W"], w["lin_b"]), w["mlp"])     # (E, dim_a)
    u = tens_sigmoid(1, r_ij * (7.0 / r0))
    phi_v = rad[..., None] * u[..., None, :]
    phi_d = rad[..., None, None] * u[..., None, None, :] * u[..., None, :, None]
    A_a = edges_reduce_src(src, rad, batch, nodes)
    A_v = edges_reduce_src(src, phi_v, batch, nodes)
    A_d = edges_reduce_src(src, phi_d, batch, nodes)
    return A_a, P.tensor_linear(1, w["readout_v"], A_v), P.tensor_linear(2, w["readout_d"], A_d)


def self_tens_prods(x_a, x_v, x_d, w, groups=8):
    """w: L0,R0,L1,R1,L2,R2, Y (dict), gn_a, gn_v, gn_d (gammas)."""
    B, N = x_a.shape[:2]
    a = x_a.reshape(B * N, -1)
    v = x_v.reshape(B * N, -1, 3)
    d = x_d.reshape(B * N, -1, 3, 3)
    prods = P.bee(P.tensor_linear(0, w["L0"], a), P.tensor_linear(1, w["L1"], v),
                  P.tensor_linear(2, w["L2"], d), P.tensor_linear(0, w["R0"], a),
                  P.tensor_linear(1, w["R1"], v), P.tensor_linear(2, w["R2"], d))
    y_a, y_v, y_d = apply_Y(prods, w["Y"])
    y_a = y_a.reshape(B, N, -1)
    y_v = y_v.reshape(B, N, -1, 3)
    y_d = y_d.reshape(B, N, -1, 3, 3)
    return (tens_group_norm(0, y_a, groups, w["gn_a"]),
            tens_group_norm(1, y_v, groups, w["gn_v"]),
            tens_group_norm(2, y_d, groups, w["gn_d"]))

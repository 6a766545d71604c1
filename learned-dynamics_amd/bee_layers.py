"""Rank-0/1/2 ("a/v/d") blocks built on the 13 Cartesian products, mirroring the
module names, constructor arguments and parameter names of
archs/diffuser_atoms15.py:29-110,227-253 of the reference (add_tens_prod_submodules,
SelfTensProds, MLP, Messages) and TensGroupNorm of managan/tensor_products.py:215-232.

Inference path.  Exact algebraic restructurings relative to the reference
(they change only the order of fp32 additions):
  * the ten bias-free output linears Y_lab of the vector and rank-2 products are
    applied AFTER the sum over edges, on N rows instead of E rows, and the five
    that feed one output run as one GEMM (weights concatenated along K);
  * phi_a = lin_enc(radial_encode_8(r)) (K = 8) is recomputed inside the edge
    kernel from the 8 encoded values; phi_v, phi_d, the gathered node features
    and the 13 per-edge products are never written to memory, except the three
    scalar products that feed the per-edge MLP;
  * 0.1 * sum is applied once per node;  x + lin_direct(x) uses W_direct + I.
radial_encode_8 is evaluated in fp64 (the reference's fp32 monomial evaluation is
ill-conditioned: alternating coefficients up to ~1e5).
"""
import torch
import torch.nn as nn

from . import differentiable as diff
from . import ops
from .codegen_tensor_products import Bee
from .graph_layers import Graph
from .tensor_products import TensLinear

LABELS_0 = ("000", "110", "220")
LABELS_1 = ("011", "101", "121", "211", "111")
LABELS_2 = ("022", "202", "112", "222", "212")


def add_tens_prod_submodules(self, dim_a, dim_v, dim_d, chan):
    for lab in ops.BEE_ORDER:
        rank = int(lab[2])
        setattr(self, f"Y_{lab}", TensLinear(rank, chan, (dim_a, dim_v, dim_d)[rank]))


def apply_tens_prod_submodules(self, prods):
    """prods: the 13 products in Bee order -> (y_0, y_1, y_2); one accumulating GEMM per product."""
    outs = [None, None, None]
    for lab, p in zip(ops.BEE_ORDER, prods):
        rank = int(lab[2])
        W = getattr(self, f"Y_{lab}").W
        if outs[rank] is None:
            outs[rank] = ops.tensor_linear_fwd(rank, W, p)
        else:
            ops.tensor_linear_fwd(rank, W, p, out=outs[rank], accumulate=True)
    return tuple(outs)


def _derived(module, key, params, make):
    """A tensor computed from parameters (a concatenation, a scaled copy), cached on the module until
    one of the parameters changes (object or version), so that pre-split weight planes and norms
    keyed on the tensor object stay valid from one forward to the next."""
    cache = module.__dict__.setdefault("_derived_cache", {})
    stamp = ops.stamp(params)
    hit = cache.get(key)
    if hit is None or hit[0] != stamp:
        with ops.derived_tensors():
            hit = cache[key] = (stamp, make())
    return hit[1]


def _cat_Y(module, labels, scale=None):
    """[Y_lab.W for lab in labels] concatenated along K (optionally scaled): one GEMM per output rank."""
    params = tuple(getattr(module, f"Y_{lab}").W for lab in labels)

    def make():
        W = torch.cat(params, dim=1)
        return W if scale is None else W * scale
    return _derived(module, ("cat_Y", labels, scale), params, make)


def _linear(x, W, bias, act, bound, out=None, accumulate=False, want_bound=True):
    """Plain-row linear with fused bias / activation.  With the split-fp16 matrix path active and
    a row bound of |x| at hand, the bound is used (no pass over x) and the bound of the output rows
    is returned with y; otherwise (y, None).  want_bound=False: the output feeds no GEMM, no bound is formed."""
    rows, dim_in, dim_out = x.shape[0], W.shape[1], W.shape[0]
    if (bound is not None and ops.get_linear_mode() == ops.LINEAR_F16X2
            and ops.f16x2_supported(rows, dim_in, dim_out, x)):
        y = ops.tensor_linear_f16x2(W, x, bound, bias=bias, act=act, out=out, accumulate=accumulate)
    else:
        y = ops.tensor_linear_fwd(0, W, x, bias=bias, act=act, out=out, accumulate=accumulate)
    return y, (ops.linear_out_bound(W, bias, bound) if bound is not None and want_bound and not accumulate else None)


class TensGroupNorm(nn.Module):
    """managan/tensor_products.py:215-232: x / sqrt(eps + mean over (nodes, group channels) of |x|^2), times gamma."""

    def __init__(self, inds, chan, groups, epsilon=1e-5):
        super().__init__()
        assert chan % groups == 0
        self.inds, self.chan, self.groups, self.epsilon = inds, chan, groups, epsilon
        self.gamma = nn.Parameter(torch.ones(chan, *[1] * inds))

    def forward(self, x, res=None):
        """gamma * x / sqrt(eps + second moment of the group) (+ res)."""
        if diff.wants_grad(self, x, res):
            y = diff.tens_group_norm(self, x)
            return y if res is None else y + res
        return ops.group_norm(ops.GN_TENSOR, x.contiguous(), self.groups, self.gamma.reshape(-1).contiguous(), None,
                              self.epsilon, res=res)


class SelfTensProds(nn.Module):
    """archs/diffuser_atoms15.py:59-95"""

    def __init__(self, dim_a, dim_v, dim_d, chan, groups=8):
        super().__init__()
        self.L0 = TensLinear(0, dim_a, chan)
        self.R0 = TensLinear(0, dim_a, chan)
        self.L1 = TensLinear(1, dim_v, chan)
        self.R1 = TensLinear(1, dim_v, chan)
        self.L2 = TensLinear(2, dim_d, chan)
        self.R2 = TensLinear(2, dim_d, chan)
        add_tens_prod_submodules(self, dim_a, dim_v, dim_d, chan)
        self.gn_a = TensGroupNorm(0, dim_a, groups)
        self.gn_v = TensGroupNorm(1, dim_v, groups)
        self.gn_d = TensGroupNorm(2, dim_d, groups)

    def forward(self, x_a, x_v, x_d, residual=False):
        """Returns the three normalised product features, or x + them with residual=True."""
        if diff.wants_grad(self, x_a, x_v, x_d):
            y = diff.self_tens_prods(self, x_a, x_v, x_d)
            return tuple(diff.add(x, t) for x, t in zip((x_a, x_v, x_d), y)) if residual else y
        in_a, in_v, in_d = x_a, x_v, x_d
        *rest, dim_a = x_a.shape
        dim_v, dim_d = x_v.shape[-2], x_d.shape[-3]
        rows = 1
        for d in rest:
            rows *= d
        x_a = x_a.reshape(rows, dim_a).contiguous()
        x_v = x_v.reshape(rows, dim_v, 3).contiguous()
        x_d = x_d.reshape(rows, dim_d, 3, 3).contiguous()
        # L_k x_k and R_k x_k are written component-major; the 13 products then land as
        # (row, comp, label, chan), so the 13 output linears are three GEMMs with K = 3 chan,
        # 5 chan, 5 chan instead of thirteen accumulating ones
        C = ops.LAYOUT_COMP_CHAN
        chan = self.L0.W.shape[0]
        # L_k and R_k act on the same x_k: its rows per component are formed once for both
        fused_products = ops.bee_products_linear_supported(rows, chan)
        # few rank-2 output channels: see below; the row maxima of the six operands are then not needed
        node_pass = ops.bee_rank2_supported(chan, dim_d)
        as_rows = [None, ops.components_as_rows(1, x_v),
                   None if (node_pass and dim_d <= 16) else ops.components_as_rows(2, x_d)]
        # ... and with at most 16 rank-2 input channels it also forms L2 x_d and R2 x_d itself
        inside2 = node_pass and dim_d <= 16
        # (and the row maxima of x_a, which the split-fp16 path scales by)
        bound_a = ops.row_absmax(x_a) if ops.get_linear_mode() == ops.LINEAR_F16X2 else None
        def input_linear(k, lin, x):
            if k == 2 and inside2:
                return lambda: None
            return lambda: ops.tensor_linear_fwd(k, lin.W, x, y_layout=C if k else ops.LAYOUT_CHAN_COMP,
                                                 want_rowmax=not node_pass, x_rows=as_rows[k],
                                                 row_bound=bound_a if k == 0 else None)
        pairs = ops.concurrent([input_linear(k, lin, x)
                                for side in ((self.L0, self.L1, self.L2), (self.R0, self.R1, self.R2))
                                for k, (lin, x) in enumerate(zip(side, (x_a, x_v, x_d)))], rows)
        ops_in = [p[0] for p in pairs] if not node_pass else list(pairs)
        if node_pass:
            # one pass over the nodes applies the rank-2 output linear to the products of a node on the fp32 matrix
            # cores and stores the scalar and vector products (18 chan floats per node) for two plain GEMMs, whose row
            # bounds it emits
            Ys = [_cat_Y(self, labels) for labels in (LABELS_0, LABELS_1, LABELS_2)]
            extra = {}
            if inside2:
                extra = dict(x_d=x_d, L2t=_derived(self, "L2_transposed", (self.L2.W,), lambda: self.L2.W.t().contiguous()),
                             R2t=_derived(self, "R2_transposed", (self.R2.W,), lambda: self.R2.W.t().contiguous()))
            y_d, P0, P1, nmax = ops.bee_node_products_rank2(*ops_in, Ys[2], want_lower_ranks=True, **extra)
            y_a, y_v = ops.concurrent([
                lambda: ops.tensor_linear_fwd(0, Ys[0], P0.reshape(rows, 3 * chan), row_bound=nmax),
                lambda: ops.tensor_linear_fwd(1, Ys[1], P1.reshape(rows, 3, 5 * chan), x_layout=C, row_bound=nmax,
                                              rows_per_bound=3)], rows)
        elif fused_products:
            # products and output linears in one kernel per output rank: the 13 products are never stored.
            # Its row scales need a bound of the products per node: 9 max|l| max|r| (at most 9 terms per
            # component), from the row maxima the six GEMMs above emit
            def node_max(side):
                cols = [(m if m is not None else ops.row_absmax(t.reshape(rows, -1))).reshape(rows, -1)
                        for t, m in side]
                return torch.cat(cols, dim=1).amax(dim=1)
            bound = 9.0 * node_max(pairs[:3]) * node_max(pairs[3:])
            Ys = [_cat_Y(self, labels) for labels in (LABELS_0, LABELS_1, LABELS_2)]
            y_a, y_v, y_d = ops.concurrent([(lambda k=k: ops.bee_products_linear(k, Ys[k], *ops_in, bound))
                                            for k in range(3)], rows)
        else:
            P0, P1, P2, nmax = ops.bee_node_products(*ops_in, want_node_max=True)
            # nmax: per-node maxima of the products, the row bounds of the three GEMMs
            Ys = [_cat_Y(self, labels) for labels in (LABELS_0, LABELS_1, LABELS_2)]
            y_a, y_v, y_d = ops.concurrent([
                lambda: ops.tensor_linear_fwd(0, Ys[0], P0.reshape(rows, 3 * chan), row_bound=nmax),
                lambda: ops.tensor_linear_fwd(1, Ys[1], P1.reshape(rows, 3, 5 * chan), x_layout=C, row_bound=nmax,
                                              rows_per_bound=3),
                lambda: ops.tensor_linear_fwd(2, Ys[2], P2.reshape(rows, 9, 5 * chan), x_layout=C, row_bound=nmax,
                                              rows_per_bound=9)], rows)
        y_a = y_a.reshape(*rest, dim_a)
        y_v = y_v.reshape(*rest, dim_v, 3)
        y_d = y_d.reshape(*rest, dim_d, 3, 3)
        if residual:
            res = (in_a.contiguous(), in_v.contiguous(), in_d.contiguous())
            return tuple(ops.concurrent([lambda: self.gn_a(y_a, res=res[0]), lambda: self.gn_v(y_v, res=res[1]),
                                         lambda: self.gn_d(y_d, res=res[2])], rows))
        return tuple(ops.concurrent([lambda: self.gn_a(y_a), lambda: self.gn_v(y_v), lambda: self.gn_d(y_d)], rows))


class MLP(nn.Module):
    """lin_direct(x) + [Linear(d,2d), LeakyReLU(.1), Linear(2d,2d), LeakyReLU(.1), Linear(2d,d)](x)
    (archs/diffuser_atoms15.py:98-110)"""

    def __init__(self, dim_a):
        super().__init__()
        self.lin_direct = nn.Linear(dim_a, dim_a, bias=False)
        self.layers = nn.Sequential(
            nn.Linear(dim_a, 2 * dim_a),
            nn.LeakyReLU(0.1),
            nn.Linear(2 * dim_a, 2 * dim_a),
            nn.LeakyReLU(0.1),
            nn.Linear(2 * dim_a, dim_a),
        )

    def forward(self, x, plus_identity=False, bound=None):
        """Returns mlp(x), or x + mlp(x) with plus_identity=True.  bound: upper bounds of the row
        maxima of |x| ((rows, 1) or (1, 1)) if the caller has them."""
        if diff.wants_grad(self, x):
            y = diff.mlp_leaky(self, x)
            return x + y if plus_identity else y
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        Wd = self.lin_direct.weight
        if plus_identity:
            Wd = _derived(self, "direct_plus_identity", (Wd,),
                          lambda: Wd + torch.eye(Wd.shape[0], device=Wd.device, dtype=Wd.dtype))
        L = self.layers
        if bound is None and ops.get_linear_mode() == ops.LINEAR_F16X2:
            bound = ops.row_absmax(x2)
        out, _ = _linear(x2, Wd, None, ops.ACT_NONE, bound, want_bound=False)
        h, b1 = _linear(x2, L[0].weight, L[0].bias, ops.ACT_LEAKY, bound)
        h, b2 = _linear(h, L[2].weight, L[2].bias, ops.ACT_LEAKY, b1)
        _linear(h, L[4].weight, L[4].bias, ops.ACT_NONE, b2, out=out, accumulate=True)
        return out.reshape(*lead, out.shape[-1])


    def summed_over_rows(self, x, row_ptr, n_out, plus_identity=False, bound=None, scale=1.0, seg=None, s_x=None,
                         count=None, add_to=None):
        """scale * (sum over the rows of each CSR segment of forward(x, plus_identity)), x (rows, d) ->
        (n_out, d).  Only the first two layers are nonlinear: the direct linear and the last layer commute
        with the sum, so they run on the n_out summed rows instead of on every row:
            sum_e mlp(x_e) = (W_direct [+ I]) sum_e x_e + W_last sum_e h_e + (rows in the segment) b_last
        with h = act(W_2 act(W_1 x + b_1) + b_2).  seg (rows,) int32: the segment of every row; with it the
        second layer sums its output rows in its own epilogue and h is never stored.  s_x: sum_e x_e if the
        caller already has it; count (n_out, 1) float32: the rows per segment, if the caller has them.
        The scale is carried by the two node-level matrices and the bias (scaled copies cached with the weights).
        add_to (n_out, d) contiguous: the result is added to it in place (and it is returned)."""
        Wd0, W_last0, b_last0 = self.lin_direct.weight, self.layers[4].weight, self.layers[4].bias
        Wd = _derived(self, ("direct_scaled", plus_identity, scale), (Wd0,),
                      lambda: scale * (Wd0 + torch.eye(Wd0.shape[0], device=Wd0.device, dtype=Wd0.dtype)
                                       if plus_identity else Wd0))
        W_last = W_last0 if scale == 1.0 else _derived(self, ("last_scaled", scale), (W_last0,), lambda: scale * W_last0)
        b_last = b_last0 if scale == 1.0 else _derived(self, ("last_bias_scaled", scale), (b_last0,), lambda: scale * b_last0)
        L = self.layers
        if bound is None and ops.get_linear_mode() == ops.LINEAR_F16X2:
            bound = ops.row_absmax(x)
        h, b1 = _linear(x, L[0].weight, L[0].bias, ops.ACT_LEAKY, bound)
        if (seg is not None and b1 is not None
                and ops.f16x2_rowsum_supported(h.shape[0], L[2].in_features, L[2].out_features, h)):
            s_h, _ = ops.tensor_linear_f16x2_rowsum(L[2].weight, h, b1, row_ptr, seg, n_out, bias=L[2].bias,
                                                    act=ops.ACT_LEAKY)
        else:
            h, _ = _linear(h, L[2].weight, L[2].bias, ops.ACT_LEAKY, b1, want_bound=False)
            s_h = ops.segment_sum_csr(h, row_ptr, n_out)
        del h
        if s_x is None:
            s_x = ops.segment_sum_csr(x, row_ptr, n_out)
        if add_to is None:
            out = ops.tensor_linear_fwd(0, Wd, s_x)
        else:
            out = ops.tensor_linear_fwd(0, Wd, s_x, out=add_to, accumulate=True)
        ops.tensor_linear_fwd(0, W_last, s_h, out=out, accumulate=True)
        if count is None:
            count = (row_ptr[1:] - row_ptr[:-1]).to(out.dtype)[:, None]
        return out.addcmul_(count, b_last[None, :])


class DisplacementTensors(nn.Module):
    """archs/diffuser_atoms15.py:206-225: ACE-like embedding of the neighbourhood.  The radial MLP runs per edge
    through the matrix path; its output times the squashed direction and its outer square is summed per node
    inside one kernel (ops.displacement_sums), so the (edges, dim_a, 3) and (edges, dim_a, 3, 3) tensors the
    reference builds for its scatter sums are never stored."""

    def __init__(self, r0: float, dim_a: int, dim_v: int, dim_d: int):
        super().__init__()
        self.r0 = r0
        self.mlp_radial = nn.Sequential(nn.Linear(8, dim_a), MLP(dim_a))
        self.readout_v = TensLinear(1, dim_a, dim_v)
        self.readout_d = TensLinear(2, dim_a, dim_d)

    def forward(self, graph: Graph, r_ij):
        """r_ij (edges, 3) -> A_a (batch, nodes, dim_a), A_v (batch, nodes, dim_v, 3), A_d (batch, nodes, dim_d, 3, 3)."""
        if diff.wants_grad(self, r_ij):
            return diff.displacement_tensors(self, graph, r_ij)
        r_ij = r_ij.contiguous()
        enc, _ = ops.bee_edge_geometry(r_ij, self.r0)                            # radial_encode_8: (edges, 8)
        first = self.mlp_radial[0]
        x = ops.tensor_linear_fwd(0, first.weight, enc, bias=first.bias)
        rad = self.mlp_radial[1](x)                                              # (edges, dim_a)
        A_a, A_v, A_d = ops.displacement_sums(graph.row_ptr, r_ij, rad, 7.0 / self.r0)
        B, N = graph.batch, graph.nodes
        return (A_a.reshape(B, N, -1), self.readout_v(A_v.reshape(B, N, -1, 3)),
                self.readout_d(A_d.reshape(B, N, -1, 3, 3)))


class Messages(nn.Module):
    """archs/diffuser_atoms15.py:227-253"""

    def __init__(self, r0: float, dim_a: int, dim_v: int, dim_d: int, chan: int):
        super().__init__()
        self.r0 = r0
        self.L0 = TensLinear(0, dim_a, chan)
        self.L1 = TensLinear(1, dim_v, chan)
        self.L2 = TensLinear(2, dim_d, chan)
        add_tens_prod_submodules(self, dim_a, dim_v, dim_d, chan)
        self.lin_enc = nn.Linear(8, chan)
        self.mlp_a = MLP(dim_a)

    def _cat_Y(self, labels, scale=None):
        return _cat_Y(self, labels, scale)

    def forward(self, graph: Graph, r_ij, x_a, x_v, x_d, node_order="cell", add_to_inputs=False):
        """x_a (batch, nodes, dim_a), x_v (..., dim_v, 3), x_d (..., dim_d, 3, 3), r_ij (edges, 3).
        Returns 0.1 * sum over edges of the messages: (B_a, B_v, B_d) with the input shapes.
        node_order: row processing order of the edge kernel ("cell": the graph's cell order when it has
        one, None: index order, or an int32 tensor); it does not change the results.
        add_to_inputs: returns (x_a + B_a, x_v + B_v, x_d + B_d) instead, the residual step of the denoiser's
        block (archs/diffuser_atoms15.py:276-279).  Without autograd and with contiguous inputs the sums are formed
        IN the inputs' memory by the kernels that produce the messages (their last use as inputs is over by then), so
        the caller must own x_a, x_v, x_d; three full-size additions per block are not launched."""
        if diff.wants_grad(self, r_ij, x_a, x_v, x_d):
            out = diff.bee_messages(self, graph, r_ij, x_a, x_v, x_d)
            return tuple(diff.add(x, d) for x, d in zip((x_a, x_v, x_d), out)) if add_to_inputs else out
        in_place = add_to_inputs and x_a.is_contiguous() and x_v.is_contiguous() and x_d.is_contiguous()
        if isinstance(node_order, str):
            node_order = getattr(graph, "cell_order", None)
        B, N = x_a.shape[:2]
        rows = B * N
        C = ops.LAYOUT_COMP_CHAN
        La, Lv, Ld, (enc, rhat) = ops.concurrent([
            lambda: ops.tensor_linear_fwd(0, self.L0.W, x_a.reshape(rows, -1).contiguous()),
            lambda: ops.tensor_linear_fwd(1, self.L1.W, x_v.reshape(rows, -1, 3).contiguous(), y_layout=C),
            lambda: ops.tensor_linear_fwd(2, self.L2.W, x_d.reshape(rows, -1, 3, 3).contiguous(), y_layout=C),
            lambda: ops.bee_edge_geometry(r_ij.contiguous(), self.r0)], rows)
        Y0, Y1, Y2 = self._cat_Y(LABELS_0), self._cat_Y(LABELS_1, 0.1), self._cat_Y(LABELS_2, 0.1)
        # few rank-2 output channels: the edge kernel applies Y2 to its sums itself and S2 (nodes, 9, 5 chan) never exists
        fused_d = ops.bee_rank2_supported(La.shape[1], Y2.shape[0])
        P0, S1, S2, nmax, emax = ops.bee_message(graph.row_ptr, graph.dst32, rhat, enc, La, Lv, Ld, self.lin_enc.weight,
                                                 self.lin_enc.bias, node_order=node_order, want_node_max=True,
                                                 Y2=Y2 if fused_d else None,
                                                 out_d=x_d.reshape(rows, -1, 9) if (fused_d and in_place) else None)
        E, chan = P0.shape[0], P0.shape[2]
        # scalar channel: per-edge linear + MLP, then the edge sum
        P0 = P0.reshape(E, 3 * chan)
        bound = emax if ops.get_linear_mode() == ops.LINEAR_F16X2 else None     # row maxima of P0 from the edge kernel

        def scalar_channel(bound=bound):
            if bound is not None and ops.f16x2_rowsum_supported(E, 3 * chan, Y0.shape[0], P0):
                # psi_a and its sum over the edges of each node from one kernel
                s_psi, psi_a = ops.tensor_linear_f16x2_rowsum(Y0, P0, bound, graph.row_ptr, graph.src32, rows,
                                                              want_rows=True)
                # from here on the edge kernel's row maxima travel with a factor and an offset (the layers' norms)
                bound = ops.linear_out_bound(Y0, None, ops.ScaledBound(bound))
            else:
                psi_a, bound = _linear(P0, Y0, None, ops.ACT_NONE, bound)
                s_psi = None
            return self.mlp_a.summed_over_rows(psi_a, graph.row_ptr, rows, plus_identity=True, bound=bound, scale=0.1,
                                               seg=graph.src32, s_x=s_psi, count=graph.degree,
                                               add_to=x_a.reshape(rows, -1) if in_place else None)
        # vector and rank-2 channels: output linears after the edge sum, on node rows (beside the per-edge MLP of the
        # scalar channel when the system is small)
        into_v = dict(out=x_v.reshape(rows, -1, 3), accumulate=True) if in_place else {}
        into_d = dict(out=x_d.reshape(rows, -1, 3, 3), accumulate=True) if in_place else {}
        jobs = [scalar_channel,
                lambda: ops.tensor_linear_fwd(1, Y1, S1.reshape(rows, 3, 5 * chan), x_layout=C, row_bound=nmax,
                                              rows_per_bound=3, **into_v)]
        if not fused_d:
            jobs.append(lambda: ops.tensor_linear_fwd(2, Y2, S2.reshape(rows, 9, 5 * chan), x_layout=C, row_bound=nmax,
                                                      rows_per_bound=9, **into_d))
        outs = ops.concurrent(jobs, rows)
        B_a, B_v, B_d = outs[0], outs[1], (S2 if fused_d else outs[2])
        shapes = ((B, N, -1), (B, N, -1, 3), (B, N, -1, 3, 3))
        if add_to_inputs and not in_place:
            B_a, B_v, B_d = (x + d.reshape(x.shape) for x, d in zip((x_a, x_v, x_d), (B_a, B_v, B_d)))
        return tuple(t.reshape(sh) for t, sh in zip((B_a, B_v, B_d), shapes))

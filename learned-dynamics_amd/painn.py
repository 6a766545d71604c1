"""PaiNN message-passing blocks on the HIP kernels, mirroring the module names,
constructor arguments and parameter names of archs/meanflow_painn8.py:25-125 of
the reference (radial_encode, MLP, Message, Update, Block).

Inference path.  Exact algebraic restructurings relative to the reference:
  * mlp_actv is applied to the N node rows and gathered inside the edge kernel,
    instead of being applied to the E gathered rows (a row-wise function
    commutes with a gather);
  * the gather of x_v, the cross product, the three scaled sums and both
    segment sums run as ONE kernel over CSR rows; nothing of size E x n x 3 is
    written to memory;
  * the three TensLinear maps of Update that read x_v run as one GEMM with the
    weights stacked.
Message takes an optional n_rbf (number of radial functions); the default n
reproduces the reference.
"""
import math

import torch
import torch.nn as nn

from . import differentiable as diff
from . import ops
from .graph_layers import Graph
from .graph_layers import graph_setup as _graph_setup
from .tensor_products import TensLinear


def graph_setup(r0, box, pos, neighbours_max=64, celllist_max=32):
    """archs/meanflow_painn8.py:167-172; the edge vectors carry a gradient for pos when one is asked for."""
    graph, r_ij = _graph_setup(r0, box, pos.detach(), neighbours_max=neighbours_max, celllist_max=celllist_max)
    if diff.differentiated(pos):
        r_ij = diff.edge_vectors(graph, pos, box)
    return graph, r_ij


def radial_encode(r, n, rmax):
    """r: (..., 3) -> (..., n)"""
    lead = r.shape[:-1]
    return ops.painn_radial_encode(r.reshape(-1, 3).contiguous(), n, rmax).reshape(*lead, n)


def _linear(x, lin, act, bound=None, want_bound=True):
    """One nn.Linear with fused bias and activation.  bound: upper bounds of the row maxima of |x|
    ((rows, 1) or (1, 1)) if the caller knows them.  Returns (y, bound of the rows of |y| or None);
    want_bound=False leaves the second out (a last layer, whose output feeds no GEMM)."""
    rows = x.shape[0]
    if ops.get_linear_mode() == ops.LINEAR_F16X2 and ops.f16x2_supported(rows, lin.in_features, lin.out_features, x):
        if bound is None:
            bound = ops.row_absmax(x)
        y = ops.tensor_linear_f16x2(lin.weight, x, bound, bias=lin.bias, act=act)
    else:
        y = ops.tensor_linear_fwd(0, lin.weight, x, bias=lin.bias, act=act)
    if bound is None or not want_bound:
        return y, None
    if isinstance(bound, ops.ScaledBound) or bound.size(0) > 1:
        # one bound per row: the array stays as it is and the layer's norms go into a factor and an offset that the
        # next kernel applies (a constant bound, below, is a cached tensor and costs no launch either)
        if not isinstance(bound, ops.ScaledBound):
            bound = ops.ScaledBound(bound)
        return y, bound.through(*ops.linear_out_bound_factors(lin.weight, lin.bias))
    return y, ops.linear_out_bound(lin.weight, lin.bias, bound)


class MLP(nn.Module):
    """Linear, SiLU, Linear, SiLU, Linear (archs/meanflow_painn8.py:38-51); bias and
    activation are fused into the GEMM epilogue.  The wide layers run on the split-fp16 matrix
    path; the row bounds it scales by are carried from layer to layer through the weight norms
    (|SiLU(z)| <= |z|), so only the first layer ever looks at the data for them."""

    def __init__(self, dim_in, dim_out):
        super().__init__()
        self.layers = nn.Sequential(
            nn.Linear(dim_in, dim_out),
            nn.SiLU(),
            nn.Linear(dim_out, dim_out),
            nn.SiLU(),
            nn.Linear(dim_out, dim_out),
        )

    def forward(self, x_a, bound=None):
        if diff.wants_grad(self, x_a):
            return diff.mlp_silu(self, x_a)
        lead = x_a.shape[:-1]
        h = x_a.reshape(-1, x_a.shape[-1]).contiguous()
        h, bound = _linear(h, self.layers[0], ops.ACT_SILU, bound)
        return self.after_first(h, bound).reshape(*lead, -1)

    def hidden(self, x, bound=None):
        """The (rows, dim_out) input of the last layer and the bound of its rows."""
        h, bound = _linear(x, self.layers[0], ops.ACT_SILU, bound)
        return _linear(h, self.layers[2], ops.ACT_SILU, bound)

    def after_first(self, h, bound=None):
        """Layers 2 and 3 on the (rows, dim_out) output of the first layer + SiLU."""
        h, bound = _linear(h, self.layers[2], ops.ACT_SILU, bound)
        return _linear(h, self.layers[4], ops.ACT_NONE, bound, want_bound=False)[0]


class ScalGroupNorm(nn.Module):
    """Group norm over the nodes of a box and the channels of a group
    (managan/layers_common.py:201-223)."""

    def __init__(self, chan, groups, epsilon=1e-5):
        super().__init__()
        assert chan % groups == 0
        self.chan, self.groups, self.epsilon = chan, groups, epsilon
        self.gamma = nn.Parameter(torch.ones(chan))
        self.beta = nn.Parameter(torch.zeros(chan))

    def forward(self, x, mul=None, add=None, res=None):
        """beta + gamma * norm(x * mul) + add + res (the extra operands are optional fusions)."""
        if diff.wants_grad(self, x, mul, add, res):
            y = diff.scal_group_norm(self, x if mul is None else x * mul)
            for extra in (add, res):
                y = y if extra is None else y + extra
            return y
        return ops.group_norm(ops.GN_SCALAR, x, self.groups, self.gamma, self.beta, self.epsilon, mul=mul, add=add,
                              res=res)


class Update(nn.Module):
    """archs/meanflow_painn8.py:53-75"""

    def __init__(self, n):
        super().__init__()
        self.n = n
        self.lin_l = TensLinear(1, n, n)
        self.lin_r = TensLinear(1, n, n)
        self.lin_v = TensLinear(1, n, n)
        self.mlp = MLP(2 * n, 3 * n)
        assert n % 4 == 0
        self.gn = ScalGroupNorm(n, 4, epsilon=1.)

    def forward(self, x_a, x_v, residual=False):
        """Returns (dx_a, dx_v), or (x_a + dx_a, x_v + dx_v) with residual=True."""
        if diff.wants_grad(self, x_a, x_v):
            da, dv = diff.painn_update(self, x_a, x_v)
            return (diff.add(x_a, da), diff.add(x_v, dv)) if residual else (da, dv)
        n = self.n
        B, N = x_a.shape[:2]
        rows = B * N
        flat_a = x_a.reshape(rows, n).contiguous()
        flat_v = x_v.reshape(rows, n, 3).contiguous()
        params = (self.lin_l.W, self.lin_r.W, self.lin_v.W)
        cache = self.__dict__.setdefault("_lrv_cache", {})
        stamp = ops.stamp(params)
        if cache.get("stamp") != stamp:                                         # (3n, n): one GEMM for l, r, v; kept
            with ops.derived_tensors():                                         # while the weights are unchanged, so
                cache.update(stamp=stamp, W=torch.cat(params, dim=0))           # its packed planes stay valid too
        W = cache["W"]
        # component-major (rows, 3, 3n): the GEMM stores whole rows, the two kernels below read with unit stride
        lrv = ops.tensor_linear_fwd(1, W, flat_v, y_layout=ops.LAYOUT_COMP_CHAN)
        ip, cat, cat_max = ops.painn_update_pre(lrv, flat_a, want_rowmax=True)  # l.r, [x_a | |r|] and its row maxima
        y = self.mlp(cat, cat_max)                                              # (rows, 3n)
        y3 = y.reshape(B, N, 3 * n)
        out_a = self.gn(ip.reshape(B, N, n), mul=y3[..., n:2 * n], add=y3[..., 2 * n:],
                        res=flat_a.reshape(B, N, n) if residual else None)
        out_v = ops.painn_update_vec(lrv, y, flat_v if residual else None)
        return out_a, out_v.reshape(B, N, n, 3)


class Message(nn.Module):
    """archs/meanflow_painn8.py:77-100"""

    def __init__(self, r0: float, n: int, n_rbf: int = None):
        super().__init__()
        self.r0 = r0
        self.n = n
        self.n_rbf = n if n_rbf is None else n_rbf
        self.epsilon = 0.1
        self.mlp_dist = MLP(self.n_rbf, 4 * n)
        self.mlp_actv = MLP(n, 4 * n)

    GRID_K = 64          # reduction dimension of the grid's first layer after padding

    def _hidden(self, r_ij):
        """Radial encoding + first layer + SiLU of the filter MLP: (edges, 4n) and the bound of its rows."""
        first = self.mlp_dist.layers[0]
        if ops.painn_radial_linear_supported(self.n_rbf, first.out_features):
            h = ops.painn_radial_linear(r_ij, self.n_rbf, self.r0, first.weight, first.bias, ops.ACT_SILU)
            # the encoding is cosines and sines: entries at most 1
            return h, ops.linear_out_bound(first.weight, first.bias, None)
        return _linear(ops.painn_radial_encode(r_ij, self.n_rbf, self.r0), first, ops.ACT_SILU,
                       ops.linear_in_unit_bound(r_ij.device))

    def filters(self, r_ij):
        """(edges, 3) -> (edges, 4n): the per-edge filter, the one large per-edge tensor."""
        return self.mlp_dist.after_first(*self._hidden(r_ij))

    use_sliced = True
    use_cell_order = True

    def _sliced_actv_last(self):
        """Last layer of mlp_actv with its rows in the slice-major column order of painn_table_message_sliced."""
        last = self.mlp_actv.layers[4]
        cache = self.__dict__.setdefault("_slice_cache", {})
        stamp = ops.stamp((last.weight, last.bias))
        if cache.get("stamp") != stamp:
            with ops.derived_tensors():
                perm = ops.painn_slice_permutation(self.n, last.weight.device)
                lin = nn.Linear(last.in_features, last.out_features, device=last.weight.device)
                lin.weight.copy_(last.weight[perm])
                lin.bias.copy_(last.bias[perm])
            cache.update(stamp=stamp, lin=lin)
        return cache["lin"]

    def _permuted_last(self):
        """Last layer of the filter MLP with its rows in the column order of the fused kernel."""
        last = self.mlp_dist.layers[4]
        cache = self.__dict__.setdefault("_perm_cache", {})
        stamp = ops.stamp((last.weight, last.bias))
        if cache.get("stamp") != stamp:
            with ops.derived_tensors():
                perm = ops.painn_filter_permutation(self.n, last.weight.device)
                cache.update(stamp=stamp, W=last.weight[perm].contiguous(), b=last.bias[perm].contiguous())
        return cache["W"], cache["b"]

    # The filter sees an edge only through its length d, and radial_encode is made of cos / sin (k pi d / r0) with
    # integer k: the filter is a smooth function of d with period 2 r0.  It is evaluated on a grid over one period
    # (a few thousand rows through the same kernels as the exact path) and every edge interpolates between the four
    # grid rows around its d.  A grid is accepted per set of weights, element by element: at the grid's midpoints,
    # where the 4-point Lagrange error peaks, |interpolated - exact| must stay below TABLE_ATOL + TABLE_RTOL |exact|
    # for every one of the 4n filter columns.  Both sides of that comparison are evaluated in float64
    # (ops.linear_f64), because the quantity bounded is the interpolation error alone: the float32 GEMMs that
    # evaluate the grid at run time round exactly as they do when they evaluate the filter of every edge, and that
    # rounding (1e-6 of a row's scale) would drown an error of this size.  The bound is a tenth of the layer
    # tolerance (abs 1e-6, rel 1e-5), so an accepted grid uses a tenth of the error a filter element may have.
    TABLE_ROWS = (512, 2048, 4096, 8192)      # 512 rows fit in LDS beside a slice of 16 channels
    TABLE_ATOL = 1e-7
    TABLE_RTOL = 1e-6
    TABLE_RECHECK = 64          # while training, the decision is re-made every this many changes of the weights
    use_table = True

    def _grid_encoding(self, rows, shift, device, width=None):
        """radial_encode at the lengths (k + shift) 2 r0 / rows, k = 0 .. rows - 1: (rows, n_rbf).  The lengths are
        known exactly, so the phases are formed in float64 and only the encodings are rounded to float32.
        width: zero columns appended up to this many (a reduction dimension the matrix path accepts)."""
        cache = self.__dict__.setdefault("_grid_cache", {})
        if width is not None and width > self.n_rbf:
            key = (rows, shift, str(device), width)
            if key not in cache:
                enc = self._grid_encoding(rows, shift, device)
                cache[key] = torch.nn.functional.pad(enc, (0, width - self.n_rbf)).contiguous()
            return cache[key]
        key = (rows, shift, str(device))
        if key not in cache:
            cache[key] = self._grid_phases(rows, shift).to(torch.float32).to(device).contiguous()
        return cache[key]

    keep_table = False        # opt-in: the grid of one set of weights is kept from one forward to the next

    def filter_table(self, rows, shift=0.0):
        """The filter at d = (k + shift) 2 r0 / rows, k = 0 .. rows - 1: (rows, 4n).  Evaluated in every call unless
        keep_table is set: then the grid (a function of the weights alone, like their packed planes) is kept per
        version of the weights, which saves the forward its 512-row MLP."""
        if not (self.keep_table and shift == 0.0) or diff.wants_grad(self.mlp_dist):
            return self._evaluate_filter_table(rows, shift)
        key = (ops.stamp(list(self.mlp_dist.parameters())), rows, ops.get_linear_mode())
        kept = self.__dict__.get("_kept_table")
        if kept is None or kept[0] != key:
            with ops.derived_tensors():
                kept = self.__dict__["_kept_table"] = (key, self._evaluate_filter_table(rows, shift))
        return kept[1]

    def _evaluate_filter_table(self, rows, shift=0.0):
        first = self.mlp_dist.layers[0]
        device = first.weight.device
        unit = ops.linear_in_unit_bound(device)
        if (self.n_rbf < self.GRID_K and ops.get_linear_mode() == ops.LINEAR_F16X2 and not diff.wants_grad(self.mlp_dist)
                and ops.f16x2_supported(rows, self.GRID_K, first.out_features, first.weight)):
            # a reduction dimension of n_rbf is below what the matrix path takes: the encodings (constants of the
            # grid) and the weight's columns are padded with zeros, which leaves every product as it was
            enc = self._grid_encoding(rows, shift, device, self.GRID_K)
            h = ops.tensor_linear_f16x2(ops.zero_padded_columns(first.weight, self.GRID_K), enc, unit,
                                        bias=first.bias, act=ops.ACT_SILU)
            return self.mlp_dist.after_first(h, ops.linear_out_bound(first.weight, first.bias, unit))
        return self.mlp_dist(self._grid_encoding(rows, shift, device), unit)

    def _grid_phases(self, rows, shift):
        """The float64 encodings at d = (k + shift) 2 r0 / rows (host tensor)."""
        n = self.n_rbf
        hn = (n + 1) // 2
        d = (torch.arange(rows, dtype=torch.float64) + shift) * (2.0 * self.r0 / rows)
        phase = (math.pi / self.r0) * (1 + torch.arange(hn) // 2).to(torch.float64)[None, :] * d[:, None]
        return torch.cat([torch.cos(phase), torch.sin(phase[:, :n - hn])], dim=-1)

    def filter_table_f64(self, rows, shift=0.0):
        """filter_table in float64 arithmetic (the float32 parameters widened exactly): (rows, 4n) double."""
        L = self.mlp_dist.layers
        device = L[0].weight.device
        cache = self.__dict__.setdefault("_grid_cache", {})
        key = (rows, shift, str(device), "f64")
        if key not in cache:
            cache[key] = self._grid_phases(rows, shift).to(device).contiguous()
        with ops.derived_tensors():
            h = ops.linear_f64(L[0].weight.detach(), L[0].bias.detach(), cache[key], ops.ACT_SILU)
            h = ops.linear_f64(L[2].weight.detach(), L[2].bias.detach(), h, ops.ACT_SILU)
            return ops.linear_f64(L[4].weight.detach(), L[4].bias.detach(), h, ops.ACT_NONE)

    def table_error(self, rows):
        """max over the grid's midpoints and the 4n filter columns of
        |4-point interpolation - exact| / (TABLE_ATOL + TABLE_RTOL |exact|), both in float64: a device scalar.
        A grid of this many rows is accepted when the value is at most 1."""
        tab = self.filter_table_f64(rows)
        mid = self.filter_table_f64(rows, 0.5)
        interp = (9.0 / 16.0) * (tab + tab.roll(-1, 0)) - (1.0 / 16.0) * (tab.roll(1, 0) + tab.roll(-2, 0))
        return ((interp - mid).abs() / (self.TABLE_ATOL + self.TABLE_RTOL * mid.abs())).amax()

    def table_rows(self):
        """Rows of the smallest grid of TABLE_ROWS that table_error accepts for the current weights, or 0 if none
        does (then the filter is evaluated per edge).  Decided once per set of weights (one host read-back per
        candidate grid).  While the weights are being trained (autograd is recording for them) the decision is kept
        for TABLE_RECHECK changes of the weights before it is made again: one optimizer step moves the
        interpolation error by far less than the factor ten between TABLE_ATOL / TABLE_RTOL and the layer
        tolerance, and the check costs host synchronisations that a training step should not pay every time."""
        params = list(self.mlp_dist.parameters())
        stamp = ops.stamp(params, keep_unversioned=True)
        cache = self.__dict__.setdefault("_table_cache", {})
        if cache.get("stamp") != stamp:
            training = diff.wants_grad(self.mlp_dist)
            cache["changes"] = cache.get("changes", 0) + 1
            if not ("rows" in cache and training and cache.get("trained") and cache["changes"] % self.TABLE_RECHECK):
                chosen = 0
                with torch.no_grad():
                    for rows in self.TABLE_ROWS:
                        if float(self.table_error(rows)) <= 1.0:
                            chosen = rows
                            break
                cache["rows"] = chosen
            cache.update(stamp=stamp, trained=training)
        return cache["rows"]

    def forward(self, graph: Graph, x_a, x_v, r_ij, residual=False):
        """x_a: (batch, atoms, n), x_v: (batch, atoms, n, 3), r_ij: (edges, 3).
        Returns (dx_a, dx_v), or (x_a + dx_a, x_v + dx_v) with residual=True."""
        if diff.wants_grad(self, x_a, x_v, r_ij):
            da, dv = diff.painn_message(self, graph, x_a, x_v, r_ij)
            return (diff.add(x_a, da), diff.add(x_v, dv)) if residual else (da, dv)
        B, N, n = x_a.shape
        flat_a = x_a.reshape(B * N, n).contiguous()
        flat_v = x_v.reshape(B * N, n, 3).contiguous()
        r_ij = r_ij.contiguous()
        res_a, res_v = (flat_a, flat_v) if residual else (None, None)
        actv = None
        if self.use_table and n % 4 == 0 and r_ij.shape[0] >= 4 * self.TABLE_ROWS[0]:
            rows = self.table_rows()
            if rows and rows <= ops.PAINN_SLICED_MAX_ROWS and n % ops.PAINN_SLICE == 0 and self.use_sliced:
                # the grid fits in LDS: actv comes out of its MLP with the columns regrouped slice by slice
                h_a, b_a = self.mlp_actv.hidden(flat_a)
                actv_s = _linear(h_a, self._sliced_actv_last(), ops.ACT_NONE, b_a, want_bound=False)[0]
                # rows in cell order when the graph has one: consecutive rows then gather the same neighbours
                order = getattr(graph, "cell_order", None) if self.use_cell_order else None
                out_a, out_v = ops.painn_table_message_sliced(graph.row_ptr, graph.dst32, r_ij, self.filter_table(rows),
                                                              2.0 * self.r0, actv_s, flat_v, self.epsilon, res_a, res_v,
                                                              node_order=order)
                return out_a.reshape(B, N, n), out_v.reshape(B, N, n, 3)
            actv = self.mlp_actv(flat_a)
            if rows and r_ij.shape[0] >= 4 * rows:
                # the grid is re-evaluated in every call (a few thousand rows): nothing of a forward is cached
                out_a, out_v = ops.painn_table_message(graph.row_ptr, graph.dst32, r_ij, self.filter_table(rows),
                                                       2.0 * self.r0, actv, flat_v, self.epsilon, res_a, res_v)
                return out_a.reshape(B, N, n), out_v.reshape(B, N, n, 3)
        if getattr(graph, "padded", False):
            # the edge arrays are longer than the graph: only the kernels above, which reach the edges through
            # row_ptr, are valid; the per-edge GEMMs below would also process the rows past the edge count
            raise RuntimeError("Message.forward on a capacity-sized graph needs the filter-grid path "
                               "(n a multiple of 16, a grid accepted for these weights, edge capacity >= 4 x grid rows)")
        if actv is None:
            actv = self.mlp_actv(flat_a)
        if ops.painn_filter_message_supported(n, 4 * n, r_ij.shape[0]):
            # the filter's last layer runs inside the edge kernel: the (edges, 4n) filter is never stored
            first, second = self.mlp_dist.layers[0], self.mlp_dist.layers[2]
            if ops.painn_filter_hidden_supported(self.n_rbf, second.out_features, r_ij.shape[0]):
                # encoding, first and second layer in one kernel: the first layer's output is never stored
                b1 = ops.linear_out_bound(first.weight, first.bias, None)
                h = ops.painn_filter_hidden(r_ij, self.r0, first.weight, first.bias, second.weight, second.bias, b1)
                bound = ops.linear_out_bound(second.weight, second.bias, b1)
            else:
                h, bound = self._hidden(r_ij)
                h, bound = _linear(h, second, ops.ACT_SILU, bound)
            W3, b3 = self._permuted_last()
            out_a, out_v = ops.painn_filter_message(W3, b3, h, bound, graph.row_ptr, graph.src32, graph.dst32, r_ij,
                                                    actv, flat_v, self.epsilon, res_a, res_v)
            return out_a.reshape(B, N, n), out_v.reshape(B, N, n, 3)
        filt = self.filters(r_ij)
        out_a, out_v = ops.painn_message(graph.row_ptr, graph.dst32, r_ij, filt, actv, flat_v,
                                         self.epsilon, res_a, res_v)
        return out_a.reshape(B, N, n), out_v.reshape(B, N, n, 3)


class Block(nn.Module):
    """archs/meanflow_painn8.py:102-125.  graph_bond may be None (no bond-graph message)."""

    def __init__(self, r0: float, n: int, pos_mutable: bool = False, n_rbf: int = None):
        super().__init__()
        self.pos_mutable = pos_mutable
        self.r0 = r0
        self.message = Message(r0, n, n_rbf)
        self.message_bond = Message(r0, n, n_rbf)
        self.update = Update(n)
        if self.pos_mutable:
            self.lin_push_pos = TensLinear(1, n, 1)

    def forward(self, tup):
        pos, graph, r_ij, graph_bond, r_ij_bond, x_a, x_v, box = tup
        if graph is None:
            graph, r_ij = graph_setup(self.r0, box, pos)
        if graph_bond is not None:
            x_a, x_v = self.message_bond(graph_bond, x_a, x_v, r_ij_bond, residual=True)
        x_a, x_v = self.message(graph, x_a, x_v, r_ij, residual=True)
        x_a, x_v = self.update(x_a, x_v, residual=True)
        if self.pos_mutable:
            pos = diff.add(pos, self.lin_push_pos(x_v).squeeze(-2))
            graph, r_ij = None, None
        return pos, graph, r_ij, graph_bond, r_ij_bond, x_a, x_v, box

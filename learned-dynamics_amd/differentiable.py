"""The layers as the reference writes them, out of differentiable pieces: what the modules run when a gradient is
asked for (training, or the Jacobian-vector product of the meanflow loss, archs/meanflow_painn8.py:274-282).

The fused inference kernels have no backward pass.  Every heavy operation here is an autograd function of this
package whose forward AND backward passes are HIP kernels (tensor_linear with its weight / input gradients, the 13
products with their two gradient kernels, gather and segment sum, which are each other's adjoints) and whose
backward is itself differentiable; the elementwise glue in between (activations, norms, the radial encodings, the
cross product, the periodic wrap) is plain torch arithmetic on the device, which autograd differentiates as it does
for the reference.  Results equal the fused path up to fp32 summation order (tests/test_gpu_autograd.py).

Forward mode: the functions that a forward pass runs also carry jvp rules, written with the same functions, so `jvp`
below returns a value and its derivative along a direction from one pass on dual tensors, both differentiable
afterwards; add / sub / mul are the arithmetic to use where only one operand can carry a tangent.
"""
import math

import torch
import torch.autograd.forward_ad as fwAD
import torch.nn.functional as F

from . import graph_layers as gl
from . import ops
from .codegen_tensor_products import Bee
from .tensor_products import tensor_linear


def has_tangent(t):
    """True for a tensor that carries a forward-mode tangent (inside jvp below)."""
    if t is None or getattr(fwAD, "_current_level", 0) < 0:       # (no dual level is open: nothing to unpack)
        return False
    return fwAD.unpack_dual(t).tangent is not None


def differentiated(t):
    """True when a derivative with respect to t is being taken, in either mode."""
    return t is not None and ((torch.is_grad_enabled() and t.requires_grad) or has_tangent(t))


def wants_grad(module, *tensors):
    """True when a gradient could flow to an input or a parameter (autograd is recording), or an input carries a
    forward-mode tangent: the cases the fused inference kernels do not serve."""
    if any(has_tangent(t) for t in tensors):
        return True
    if not torch.is_grad_enabled():
        return False
    if any(t is not None and t.requires_grad for t in tensors):
        return True
    return any(p.requires_grad for p in module.parameters())


def _one_sided(a, b):
    """(the operand with a tangent, the other, whether they were exchanged) when exactly one of a, b carries a
    forward-mode tangent, else None."""
    ta, tb = torch.is_tensor(a) and has_tangent(a), torch.is_tensor(b) and has_tangent(b)
    if ta == tb:
        return None
    return (b, a, True) if tb else (a, b, False)


def add(a, b):
    """a + b.  When only one operand carries a forward-mode tangent the tangent passes through unchanged: torch's own
    rule forms a symbolic zero for the other operand (a number or a parameter has none) and adds it through a slow
    path (Python meta kernels, 0.15 ms of host time per call).  Outside forward mode this is a + b."""
    one = _one_sided(a, b)
    if one is None:
        return a + b
    p, t = fwAD.unpack_dual(one[0])
    out = p + one[1]
    return fwAD.make_dual(out, t if t.shape == out.shape else t.expand(out.shape))


def sub(a, b):
    """a - b, in forward mode as add."""
    one = _one_sided(a, b)
    if one is None:
        return a - b
    p, t = fwAD.unpack_dual(one[0])
    out, t = (one[1] - p, -t) if one[2] else (p - one[1], t)
    return fwAD.make_dual(out, t if t.shape == out.shape else t.expand(out.shape))


def mul(a, b):
    """a * b, in forward mode as add: the tangent is the one operand's tangent times the other operand."""
    one = _one_sided(a, b)
    if one is None:
        return a * b
    p, t = fwAD.unpack_dual(one[0])
    return fwAD.make_dual(p * one[1], t * one[1])


def div(a, b):
    """a / b for a b without a tangent, in forward mode as add."""
    if not (torch.is_tensor(a) and has_tangent(a)) or (torch.is_tensor(b) and has_tangent(b)):
        return a / b
    p, t = fwAD.unpack_dual(a)
    return fwAD.make_dual(p / b, t / b)


def jvp(f, primals, tangents, create_graph=True, strict=False):
    """(f(*primals), the derivative of f at primals along tangents) in forward mode: every autograd function of this
    package that a forward pass runs has a jvp rule made of the package's differentiable functions, so the pair costs
    about two forward passes and both results can be differentiated afterwards (loss.backward()).
    torch.autograd.functional.jvp(f, primals, tangents, create_graph=True), which the reference's meanflow loss calls
    (archs/meanflow_painn8.py:274-282), gets the same derivative out of two nested backward passes, and the loss then
    differentiates all three; its first result is the same f(*primals) that the loss evaluates again as v_pred
    (archs/meanflow_painn8.py:291-292), so one call here stands for both.  The signature and the order of the results
    are functional.jvp's, so the name is the only change at a call site; create_graph and strict are accepted for that
    and change nothing (both results are always recorded when autograd is recording; without it, under no_grad, neither
    is).  primals and tangents may be single tensors."""
    if torch.is_tensor(primals):
        primals, tangents = (primals,), (tangents,)
    def unpack(out):
        value, tangent = fwAD.unpack_dual(out)
        return value, (tangent if tangent is not None else torch.zeros_like(value))

    with fwAD.dual_level():
        out = f(*(fwAD.make_dual(p, t) for p, t in zip(primals, tangents)))
        if isinstance(out, (tuple, list)):               # several results: (values, tangents), like functional.jvp
            pairs = [unpack(o) for o in out]
            return tuple(v for v, _ in pairs), tuple(t for _, t in pairs)
        return unpack(out)


def linear(lin, x, x_bound=None, want_bound=False):
    """nn.Linear through the tensor_linear kernels (weight and input gradients are kernels too).  x_bound / want_bound:
    row maxima handed from one layer to the next (tensor_products.tensor_linear)."""
    lead = x.shape[:-1]
    out = tensor_linear(0, lin.weight, x.reshape(-1, x.shape[-1]).contiguous(), bias=lin.bias, x_bound=x_bound,
                        want_bound=want_bound)
    if want_bound:
        return out[0].reshape(*lead, -1), out[1]
    return out.reshape(*lead, -1)


class _SiluOrder(torch.autograd.Function):
    """SiLU^(order)(z).  Its derivative is the next member of the same family times the incoming gradient, so the
    family is closed under differentiation: every derivative order of an MLP costs one kernel per activation (plus one
    product while a higher derivative is still being recorded) instead of autograd's chain of elementwise formulas for
    the derivative of SiLU's derivative."""

    @staticmethod
    def forward(ctx, z, order):
        ctx.save_for_backward(z)
        ctx.save_for_forward(z)
        ctx.order = order
        return ops.silu_order(z.contiguous(), order)

    @staticmethod
    def jvp(ctx, z_t, _):
        z, = ctx.saved_tensors
        return z_t * _silu_order(z, ctx.order + 1)

    @staticmethod
    def backward(ctx, g):
        z, = ctx.saved_tensors
        if not torch.is_grad_enabled():
            return ops.silu_order(z.contiguous(), ctx.order + 1, mul=g.contiguous()), None
        return g * _silu_order(z, ctx.order + 1), None


def _silu_order(z, order):
    if order > ops.SILU_MAX_ORDER:
        raise RuntimeError(f"SiLU is differentiable {ops.SILU_MAX_ORDER} times here")
    return _SiluOrder.apply(z, order)


def silu(z):
    """nn.SiLU on a CUDA float32 tensor, differentiable up to ops.SILU_MAX_ORDER times."""
    if z.is_cuda and z.dtype == torch.float32:
        return _silu_order(z, 0)
    return F.silu(z)


def mlp_silu(mlp, x):
    """painn.MLP: Linear, SiLU, Linear, SiLU, Linear (archs/meanflow_painn8.py:38-51).  |SiLU(z)| <= |z|: the row
    maxima that a layer's kernel emits for z bound the next layer's input."""
    L = mlp.layers
    z, b = linear(L[0], x, want_bound=True)
    z, b = linear(L[2], silu(z), x_bound=b, want_bound=True)
    return linear(L[4], silu(z), x_bound=b)


def mlp_leaky(mlp, x):
    """bee_layers.MLP: lin_direct(x) + layers(x) with LeakyReLU(0.1) (archs/diffuser_atoms15.py:98-110)."""
    L = mlp.layers
    z, b = linear(L[0], x, want_bound=True)
    z, b = linear(L[2], F.leaky_relu(z, 0.1), x_bound=b, want_bound=True)
    return linear(mlp.lin_direct, x) + linear(L[4], F.leaky_relu(z, 0.1), x_bound=b)


def radial_encode_painn(r, n, rmax):
    """archs/meanflow_painn8.py:25-35"""
    hn = (n + 1) // 2
    coeffs = (math.pi / rmax) * (1 + torch.arange(0, hn, device=r.device) // 2)
    phase = mul(torch.linalg.vector_norm(r, dim=-1)[..., None], coeffs)
    return torch.cat([torch.cos(phase), torch.sin(phase[..., :(n - hn)])], dim=-1)


_JACOBI = {}


def _jacobi_matrix(device):
    """Coefficients of the shifted Jacobi polynomials P_i^(1,0)(2x - 1), i < 8 (managan/jacobi_radenc.py:8-22)."""
    key = str(device)
    if key not in _JACOBI:
        A = torch.zeros(8, 9, dtype=torch.float64)
        for n in range(8):
            for s in range(n + 1):
                w = math.comb(n + 1, n - s) * math.comb(n, s)
                for k in range(s + 1):
                    A[n, k + n - s] += w * math.comb(s, k) * (-1.0) ** (s - k)
        _JACOBI[key] = A.to(device)
    return _JACOBI[key]


def radial_encode_8(r, rmax):
    """managan/jacobi_radenc.py:24-37; the polynomials are evaluated in float64 (Horner) like the inference kernel:
    their monomial form in fp32 loses three digits."""
    z = div(torch.linalg.vector_norm(r, dim=-1), rmax)[..., None].double()
    A = _jacobi_matrix(r.device)
    acc = A[:, 8].expand(*z.shape[:-1], 8)
    for k in range(7, -1, -1):
        acc = add(mul(acc, z), A[:, k])
    return (acc * torch.relu(sub(1.0, z))).to(r.dtype)


def tens_sigmoid(inds, x):
    dims = tuple(-(1 + n) for n in range(inds))
    xx = (x ** 2).sum(dims, keepdim=True) if inds > 0 else x ** 2
    return x / torch.sqrt(add(xx, 1.0))


def scal_group_norm(gn, x):
    """managan/layers_common.py:201-223"""
    B, N, chan = x.shape
    xg = x.reshape(B, N, gn.groups, -1)
    sh = xg - xg.mean([1, 3], keepdim=True)
    var = (sh ** 2).mean([1, 3], keepdim=True)
    return add(mul((sh / torch.sqrt(add(var, gn.epsilon))).reshape(B, N, chan), gn.gamma), gn.beta)


def tens_group_norm(gn, x):
    """managan/tensor_products.py:215-232"""
    B, N, chan = x.shape[:3]
    xg = x.reshape(B, N, gn.groups, -1, 3 ** gn.inds)
    m2 = (xg ** 2).sum(-1, keepdim=True).mean([1, 3], keepdim=True)
    return mul((xg / torch.sqrt(add(m2, gn.epsilon))).reshape(x.shape), gn.gamma)


def edge_vectors(graph, pos, box):
    """boxwrap(box, pos[dst] - pos[src]) with a gradient for pos (archs/meanflow_painn8.py:167-172)."""
    pos_src, pos_dst = gl.edges_read(graph, pos)
    tbox = torch.tensor(box, device=pos.device, dtype=pos.dtype)
    delta = pos_dst - pos_src
    if has_tangent(delta):
        # the wrap shifts by a locally constant multiple of the box: its Jacobian is the identity
        p, t = fwAD.unpack_dual(delta)
        return fwAD.make_dual(gl.boxwrap(tbox, p), t)
    return gl.boxwrap(tbox, delta)


def _painn_combine_plain(dist, actv, v, direction):
    """archs/meanflow_painn8.py:94-100, as the reference writes it"""
    n = v.size(1)
    prod = dist * actv
    cross = torch.linalg.cross(v, direction[:, None].expand_as(v))
    m = v * prod[..., :n, None] + cross * prod[..., n:2 * n, None] + direction[:, None] * prod[..., 2 * n:3 * n, None]
    return m, prod[..., 3 * n:]


_TERMS_ALL, _TERMS_V, _TERMS_DIR = 15, 3, 6      # the four terms of the message; those that contain v; those with the direction


def _sum_opt(parts):
    parts = [p for p in parts if p is not None]
    return sum(parts[1:], parts[0]) if parts else None


class _PainnCombine(torch.autograd.Function):
    """Lines 94-100 of archs/meanflow_painn8.py as one kernel with the graph operations on either side folded in:
    actv and v come per node and the kernel reads the destination's row (by_dst); m and a are summed over the edges
    of their source node (by_src).  Returns (out_v (nodes, n, 3), out_a (nodes, n)).  `terms` masks the four terms of
    the message.  The pairing sum (G_v . out_v + G_a . out_a) is linear in (G_v, G_a), in dist and in actv, and in v
    and the direction once restricted to the terms that contain them: every derivative of this function and of
    _PainnCombineGrad is one of the two with a cotangent in one argument's place and that argument's mask, so the
    pair is closed under differentiation and recorded backward passes run on the same two kernels."""

    @staticmethod
    def forward(ctx, dist, actv_node, v_node, direction, by_dst, by_src, terms):
        ctx.by_dst, ctx.by_src, ctx.terms = by_dst, by_src, terms
        ctx.save_for_backward(dist, actv_node, v_node, direction)
        ctx.save_for_forward(dist, actv_node, v_node, direction)
        ctx.set_materialize_grads(False)
        # (the edges are sorted by their source node: its CSR is the row pointer of the sums)
        return ops.painn_combine_fwd_rows(dist.contiguous(), actv_node.contiguous(), v_node.contiguous(),
                                          direction.contiguous(), by_dst.index, by_src.row_ptr, by_src.n_rows, terms=terms)

    @staticmethod
    def jvp(ctx, dist_t, actv_t, v_t, dir_t, *_):
        """The function is linear in each argument within the terms that contain it: the tangent is the sum of the
        function itself with one argument's tangent in that argument's place."""
        dist, actv, v, direction = ctx.saved_tensors
        idx, t = (ctx.by_dst, ctx.by_src), ctx.terms
        slots = [(dist_t, (dist_t, actv, v, direction), t), (actv_t, (dist, actv_t, v, direction), t),
                 (v_t, (dist, actv, v_t, direction), t & _TERMS_V), (dir_t, (dist, actv, v, dir_t), t & _TERMS_DIR)]
        pairs = [_PainnCombine.apply(*args, *idx, mask) for x_t, args, mask in slots if x_t is not None and mask]
        return _sum_opt([p[0] for p in pairs]), _sum_opt([p[1] for p in pairs])

    @staticmethod
    def backward(ctx, g_v, g_a):
        if g_v is None or g_a is None:
            ref_v, ref_a = ctx.saved_tensors[2], ctx.saved_tensors[1]
            nodes = ctx.by_src.n_rows
            g_v = g_v if g_v is not None else ref_v.new_zeros(nodes, ref_v.size(1), 3)
            g_a = g_a if g_a is not None else ref_a.new_zeros(nodes, ref_v.size(1))
        want = tuple(ctx.needs_input_grad[:4])
        grads = _PainnCombineGrad.apply(g_v, g_a, *ctx.saved_tensors, ctx.by_dst, ctx.by_src, ctx.terms, want)
        return tuple(g if need else None for g, need in zip(grads, want)) + (None, None, None)


class _PainnCombineGrad(torch.autograd.Function):
    """(g_v, g_a, dist, actv, v, direction) -> the gradients of _PainnCombine's four inputs: d_dist (edges, 4n),
    d_actv (nodes, 4n), dv (nodes, n, 3), d_direction (edges, 3): one kernel; the gradient rows of an edge's source
    node are read through the source index, the gradients of actv and v are summed over the edges of a destination
    inside it (mg_painn_combine_bwd_rows)."""

    @staticmethod
    def forward(ctx, g_v, g_a, dist, actv_node, v_node, direction, by_dst, by_src, terms, want):
        """want: which of the four gradients to compute (the others come back as empty tensors)."""
        ctx.by_dst, ctx.by_src, ctx.terms, ctx.want = by_dst, by_src, terms, want
        ctx.save_for_backward(g_v, g_a, dist, actv_node, v_node, direction)
        args = (dist.contiguous(), actv_node.contiguous(), v_node.contiguous(), direction.contiguous(), g_v.contiguous(),
                g_a.contiguous())
        if want[1] or want[2]:
            # the gradients of actv and v are summed over the edges of a destination inside the kernel
            d_dist, d_actv, dv, d_dir = ops.painn_combine_bwd_rows(*args, by_dst.row_ptr, by_dst.perm, by_src.index,
                                                                   terms=terms, want=want)
        else:
            d_dist, d_actv, dv, d_dir = ops.painn_combine_bwd(*args, node=by_dst.index, grad_row=by_src.index,
                                                              terms=terms, want=want)
        outs = [d_dist, d_actv, dv, d_dir]
        for k in range(4):
            if outs[k] is None:
                outs[k] = dist.new_empty(0)
                ctx.mark_non_differentiable(outs[k])
        return tuple(outs)

    @staticmethod
    def backward(ctx, h_dist, h_actv, h_v, h_dir):
        g_v, g_a, dist, actv, v, direction = ctx.saved_tensors
        idx, t = (ctx.by_dst, ctx.by_src), ctx.terms
        need = ctx.needs_input_grad
        # one entry per cotangent: the four arguments with the cotangent in its own argument's place, and the mask
        slots = [(h_dist, (h_dist, actv, v, direction), t), (h_actv, (dist, h_actv, v, direction), t),
                 (h_v, (dist, actv, h_v, direction), t & _TERMS_V), (h_dir, (dist, actv, v, h_dir), t & _TERMS_DIR)]
        slots = [(k, args, mask) for k, (h, args, mask) in enumerate(slots) if h is not None and ctx.want[k]]
        out_g_v = out_g_a = None
        if need[0] or need[1]:
            pairs = [_PainnCombine.apply(*args, *idx, mask) for _, args, mask in slots]
            out_g_v, out_g_a = _sum_opt([p[0] for p in pairs]), _sum_opt([p[1] for p in pairs])
        grads = [[], [], [], []]
        for k, args, mask in slots:
            # (output k of such a call would be the derivative in the cotangent itself: not wanted)
            want = tuple(bool(need[2 + j]) and j != k for j in range(4))
            if any(want):
                outs = _PainnCombineGrad.apply(g_v, g_a, *args, *idx, mask, want)
                for j in range(4):
                    if want[j]:
                        grads[j].append(outs[j])
        return ((out_g_v, out_g_a) + tuple(_sum_opt(g) if nd else None for g, nd in zip(grads, need[2:6]))
                + (None, None, None, None))


def painn_combine(graph, dist, actv_node, v_node, direction):
    """dist (E, 4n), direction (E, 3) per edge; actv_node (batch, nodes, 4n), v_node (batch, nodes, n, 3) per node, read
    at each edge's destination.  Returns the sums over the edges of each source node: (out_v (batch, nodes, n, 3),
    out_a (batch, nodes, n))."""
    actv_flat, v_flat = gl._flat_nodes(graph, actv_node), gl._flat_nodes(graph, v_node)
    if (ops.painn_combine_supported(v_flat.size(1)) and all(t.is_contiguous() and t.data_ptr() % 16 == 0
                                                            for t in (dist, actv_flat, v_flat, direction))):
        out_v, out_a = _PainnCombine.apply(dist, actv_flat, v_flat, direction, graph.by_dst, graph.by_src, _TERMS_ALL)
    else:
        m, a = _painn_combine_plain(dist, gl._Gather.apply(actv_flat, graph.by_dst),
                                    gl._Gather.apply(v_flat, graph.by_dst), direction)
        out_v, out_a = gl._ScatterSum.apply(m, graph.by_src), gl._ScatterSum.apply(a.contiguous(), graph.by_src)
    return (out_v.reshape(graph.batch, graph.nodes, *out_v.shape[1:]),
            out_a.reshape(graph.batch, graph.nodes, *out_a.shape[1:]))


def _table_interp_plain(table, d, period):
    """4-point Lagrange interpolation of a periodic grid in tensor arithmetic (differentiable in the grid and in d):
    the formula table_interp's kernels implement, kept as the yardstick its tests differentiate in float64."""
    rows = table.size(0)
    u = d * (float(rows) / period)
    fl = torch.floor(u).detach()
    t = (u - fl)[:, None]
    i = fl.long()
    tp, tm, tq = t + 1.0, t - 1.0, t - 2.0
    w = (-(1.0 / 6.0) * t * tm * tq, 0.5 * tp * tm * tq, -0.5 * tp * t * tq, (1.0 / 6.0) * tp * t * tm)
    return sum(w[j] * table[(i - 1 + j) % rows] for j in range(4))


class _SortedLengths:
    """The edges sorted by the grid row below their length: what the sums into the grid run by; computed on first
    use and shared by every pass over the same lengths."""

    def __init__(self, d, rows, period):
        self.d, self.rows, self.period = d, rows, period
        self._sorted = None

    def get(self):
        if self._sorted is None:
            self._sorted = ops.painn_table_sorted_edges(self.d.detach(), self.rows, self.period)
        return self._sorted


class _TableInterp(torch.autograd.Function):
    """order 0: the filter of every edge interpolated from its grid; order k: the interpolant's k-th derivative in
    the edge length (its weights are cubics: orders 0 .. 3 exist, the fourth derivative is zero).  The gradient for
    the grid is _TableScatter of the same order, the gradient for the lengths a row-wise product with _TableInterp of
    the next order: the family is closed under differentiation, so any number of nested derivatives run on these
    kernels.  Outside a recorded backward pass both gradients come from one fused call."""

    @staticmethod
    def forward(ctx, table, d, period, order, order_by):
        ctx.period, ctx.order, ctx.order_by = period, order, order_by
        ctx.save_for_backward(table, d)
        return ops.painn_table_interp_fwd(table, d, period, order)

    @staticmethod
    def backward(ctx, g):
        table, d = ctx.saved_tensors
        g = g.contiguous()
        need_t, need_d = ctx.needs_input_grad[0], ctx.needs_input_grad[1] and ctx.order < 3
        if not torch.is_grad_enabled():
            perm, bucket_ptr = ctx.order_by.get()
            d_table, dd = ops.painn_table_interp_bwd(g, table, d, ctx.period, perm, bucket_ptr, want_length_grad=need_d,
                                                     order=ctx.order)
            return (d_table if need_t else None), dd, None, None, None
        d_table = dd = None
        if need_t:
            d_table = _TableScatter.apply(g, d, ctx.period, ctx.order, table.size(0), ctx.order_by)
        if need_d:
            dd = (g * _TableInterp.apply(table, d, ctx.period, ctx.order + 1, ctx.order_by)).sum(-1)
        return d_table, dd, None, None, None


class _TableScatter(torch.autograd.Function):
    """The adjoint of _TableInterp in the grid: every edge's row g[e] added to the four grid rows around its length
    with the (order-th derivative) weights, in the order of a sort by grid row.  Linear in g; its gradients are
    _TableInterp calls."""

    @staticmethod
    def forward(ctx, g, d, period, order, rows, order_by):
        ctx.period, ctx.order, ctx.order_by = period, order, order_by
        ctx.save_for_backward(g, d)
        perm, bucket_ptr = order_by.get()
        return ops.painn_table_interp_bwd(g.contiguous(), None, d, period, perm, bucket_ptr, want_length_grad=False,
                                          order=order, table_rows=rows)[0]

    @staticmethod
    def backward(ctx, dd_table):
        g, d = ctx.saved_tensors
        dd_table = dd_table.contiguous()
        d_g = dd = None
        if ctx.needs_input_grad[0]:
            d_g = _TableInterp.apply(dd_table, d, ctx.period, ctx.order, ctx.order_by)
        if ctx.needs_input_grad[1] and ctx.order < 3:
            dd = (g * _TableInterp.apply(dd_table, d, ctx.period, ctx.order + 1, ctx.order_by)).sum(-1)
        return d_g, dd, None, None, None, None


def table_interp(table, d, period):
    """The grid `table` (rows, cols) of a function of period `period` interpolated at the lengths d (edges):
    (edges, cols), differentiable in both any number of times."""
    table, d = table.contiguous(), d.contiguous()
    return _TableInterp.apply(table, d, period, 0, _SortedLengths(d, table.size(0), period))


def _filter_grid_rows(msg, r_ij):
    """Rows of the grid the differentiable filter interpolates from, or 0 for the MLP on every edge."""
    E = r_ij.shape[0]
    rows = msg.table_rows() if (getattr(msg, "use_table", False) and E >= 4 * msg.TABLE_ROWS[0]) else 0
    if r_ij.requires_grad or has_tangent(r_ij):
        # The gradient for the edge vectors would go through the interpolant's derivative: differences of neighbouring
        # grid rows divided by the spacing, which amplifies the fp32-level noise of the grid values (1e-6 of their size
        # from the GEMMs that evaluate them) by rows / period: 4e-5 of the largest gradient entry at 2048 rows, 2e-4 at
        # 512 (where the interpolation error of the derivative dominates), against 7e-7 for the MLP on every edge.
        # A grid evaluated in float64 does not help (3e-5 at 2048 rows): the float32 differences themselves cancel
        # that many digits.  Positions that are differentiated (the meanflow loss, blocks that move them) keep the
        # per-edge MLP.
        return 0
    return rows if rows and E >= 4 * rows and ops.painn_table_interp_supported(rows, 4 * msg.n) else 0


def painn_filter(msg, r_ij):
    """mlp_dist(radial_encode(r_ij)) (archs/meanflow_painn8.py:92), (edges, 4n).  The filter is a smooth periodic
    function of the edge length: when the module's grid test accepts a grid for the current weights (the test the
    inference path uses, Message.table_rows) the MLP runs on the grid's rows and every edge interpolates, so that the
    backward pass differentiates the MLP on a few hundred rows instead of on every edge.  Only when the edge vectors
    need no gradient (_filter_grid_rows)."""
    rows = _filter_grid_rows(msg, r_ij)
    if rows:
        table = mlp_silu(msg.mlp_dist, msg._grid_encoding(rows, 0.0, r_ij.device))
        d = torch.linalg.vector_norm(r_ij, dim=-1).contiguous()
        return table_interp(table, d, 2.0 * msg.r0)
    return mlp_silu(msg.mlp_dist, radial_encode_painn(r_ij, msg.n_rbf, msg.r0))


def _unit_vectors(r_ij, epsilon):
    return r_ij / torch.sqrt(add((r_ij ** 2).sum(-1, keepdim=True), epsilon))


_SLICE_PERMUTATIONS = {}


def _slice_permutation(n, device):
    key = (n, str(device))
    if key not in _SLICE_PERMUTATIONS:
        _SLICE_PERMUTATIONS[key] = ops.painn_slice_permutation(n, device)
    return _SLICE_PERMUTATIONS[key]


class _PainnGridMessage(torch.autograd.Function):
    """(grid (rows, 4n), actv (nodes, 4n), v (nodes, n, 3)) -> (out_v, out_a) of the message for edge vectors that are
    not differentiated, with the filter interpolated from the grid.  Forward: the inference kernel of the layer
    (mg_painn_table_message: lengths, directions, interpolation, the lines 94-100 of archs/meanflow_painn8.py and the
    sum over the edges of a node in one pass; no per-edge filter is stored).  Backward: the gradient kernel of the
    unfused formulation with the filter of every edge interpolated again inside it and the gradients of actv and v
    summed per destination inside it (mg_painn_combine_bwd_rows), then the scatter into the grid.  A recorded backward pass differentiates the unfused formulation instead."""

    @staticmethod
    def forward(ctx, table, actv, v, r_ij, graph, period, epsilon):
        ctx.graph, ctx.period, ctx.epsilon = graph, period, epsilon
        table, actv, v = table.contiguous(), actv.contiguous(), v.contiguous()
        ctx.save_for_backward(table, actv, v, r_ij)
        n = v.size(1)
        if table.size(0) <= ops.PAINN_SLICED_MAX_ROWS and n % ops.PAINN_SLICE == 0:
            # the grid fits in LDS: the kernel that holds it there takes actv with its columns grouped slice by slice
            actv_s = actv[:, _slice_permutation(n, actv.device)].contiguous()
            out_a, out_v = ops.painn_table_message_sliced(graph.row_ptr, graph.dst32, r_ij, table, period, actv_s, v, epsilon,
                                                          node_order=getattr(graph, "cell_order", None))
        else:
            out_a, out_v = ops.painn_table_message(graph.row_ptr, graph.dst32, r_ij, table, period, actv, v, epsilon)
        return out_v, out_a

    @staticmethod
    def backward(ctx, g_v, g_a):
        table, actv, v, r_ij = ctx.saved_tensors
        graph, need = ctx.graph, ctx.needs_input_grad
        if torch.is_grad_enabled():
            with torch.enable_grad():
                leaves = [t if t.requires_grad else t.detach().requires_grad_() for t in (table, actv, v)]
                out = _grid_message_unfused(*leaves, r_ij, graph, ctx.period, ctx.epsilon)
                grads = torch.autograd.grad(out, leaves, (g_v, g_a), create_graph=True, allow_unused=True)
            return tuple(g if nd else None for g, nd in zip(grads, need)) + (None, None, None, None)
        by_dst, by_src = graph.by_dst, graph.by_src
        d = torch.linalg.vector_norm(r_ij, dim=-1).contiguous()
        want = (bool(need[0]), bool(need[1]), bool(need[2]), False)
        # (actv and v are read at an edge's destination: their gradients are summed over a destination's edges inside)
        d_dist, d_actv, dv, _ = ops.painn_combine_bwd_rows(None, actv, v, _unit_vectors(r_ij, ctx.epsilon).contiguous(),
                                                           g_v.contiguous(), g_a.contiguous(), by_dst.row_ptr, by_dst.perm,
                                                           by_src.index, terms=_TERMS_ALL, want=want, table=table,
                                                           period=ctx.period, d=d)
        d_table = None
        if need[0]:
            rows = table.size(0)
            perm, bucket_ptr = ops.painn_table_sorted_edges(d, rows, ctx.period)
            d_table = ops.painn_table_interp_bwd(d_dist, None, d, ctx.period, perm, bucket_ptr, want_length_grad=False,
                                                 order=0, table_rows=rows)[0]
        return (d_table, d_actv if need[1] else None, dv if need[2] else None, None, None, None, None)


def _grid_message_unfused(table, actv, v, r_ij, graph, period, epsilon):
    d = torch.linalg.vector_norm(r_ij, dim=-1).contiguous()
    return _PainnCombine.apply(table_interp(table, d, period), actv, v, _unit_vectors(r_ij, epsilon).contiguous(),
                               graph.by_dst, graph.by_src, _TERMS_ALL)


def painn_message(msg, graph, x_a, x_v, r_ij):
    """archs/meanflow_painn8.py:85-100"""
    # the MLP acts on rows, so it commutes with the gather: N rows go through it, not E (the reference gathers first),
    # and the gathers themselves are folded into the combining kernel
    actv = mlp_silu(msg.mlp_actv, x_a)
    rows = _filter_grid_rows(msg, r_ij)
    n = x_v.size(-2)
    if (rows and n % 4 == 0 and ops.painn_combine_supported(n) and not any(has_tangent(t) for t in (x_a, x_v))
            and r_ij.is_contiguous() and not getattr(graph, "padded", False)):
        table = mlp_silu(msg.mlp_dist, msg._grid_encoding(rows, 0.0, r_ij.device))
        out_v, out_a = _PainnGridMessage.apply(table, gl._flat_nodes(graph, actv), gl._flat_nodes(graph, x_v), r_ij, graph,
                                               2.0 * msg.r0, msg.epsilon)
        return (out_a.reshape(graph.batch, graph.nodes, *out_a.shape[1:]),
                out_v.reshape(graph.batch, graph.nodes, *out_v.shape[1:]))
    dist = painn_filter(msg, r_ij)
    out_v, out_a = painn_combine(graph, dist, actv, x_v, _unit_vectors(r_ij, msg.epsilon))
    return out_a, out_v


def painn_update(upd, x_a, x_v):
    """archs/meanflow_painn8.py:63-75"""
    n = upd.n
    v_l, v_r = upd.lin_l(x_v), upd.lin_r(x_v)
    ip = (v_l * v_r).sum(-1)
    y = mlp_silu(upd.mlp, torch.cat([x_a, torch.linalg.vector_norm(v_r, dim=-1)], dim=-1))
    v = upd.lin_v(x_v) * y[..., :n, None]
    a = scal_group_norm(upd.gn, ip * y[..., n:2 * n]) + y[..., 2 * n:]
    return a, v / torch.sqrt(add((v ** 2).sum(-1, keepdim=True), 1.))


def apply_tens_prod_submodules(module, prods):
    """archs/diffuser_atoms15.py:52-57"""
    from .ops import BEE_ORDER
    out = [None, None, None]
    for lab, p in zip(BEE_ORDER, prods):
        y = getattr(module, f"Y_{lab}")(p)
        k = int(lab[2])
        out[k] = y if out[k] is None else out[k] + y
    return tuple(out)


def _message_products_plain(a_node, v_node, d_node, enc, rh, by_dst, by_src):
    """The 13 products of the gathered node operands with the edge filters (enc, enc (x) rh, enc (x) rh (x) rh); those
    of rank 1 and 2 summed over the edges of their source node (archs/diffuser_atoms15.py:241-252 with the sum moved
    before the output linears).  Built from functions that are differentiable any number of times."""
    from .ops import BEE_ORDER
    phi_v, phi_d = _EdgeFilters.apply(enc, rh)
    prods = Bee.apply(gl._Gather.apply(a_node, by_dst), gl._Gather.apply(v_node, by_dst), gl._Gather.apply(d_node, by_dst),
                      enc.contiguous(), phi_v, phi_d)
    return tuple(p if lab[2] == "0" else gl._ScatterSum.apply(p.contiguous(), by_src) for lab, p in zip(BEE_ORDER, prods))


_S1_LABELS, _S2_LABELS = ("011", "101", "121", "211", "111"), ("022", "202", "112", "222", "212")


class _MessageProducts(torch.autograd.Function):
    """The same with everything between the node operands and the per-node sums folded into kernels.  Forward: the
    inference kernel of the layer (mg_bee_message: filters formed in registers, node rows gathered at the destination,
    products summed over the edges of a node; only the three scalar products are stored per edge) when `enc_source`
    = (the 8 radial functions, weight and bias of the encoding linear) is given, else the indexed product kernel and
    segment sums.  Backward: the filters are recomputed, the two gradient kernels read the node operands at the
    destination and the gradients of the summed products at the source through the indices, and the filters' adjoint
    folds the three filter gradients into those of enc and rh.  A recorded backward pass (create_graph=True)
    differentiates the plain formulation instead."""

    @staticmethod
    def forward(ctx, a_node, v_node, d_node, enc, rh, by_dst, by_src, enc_source):
        from .ops import BEE_ORDER
        ctx.by_dst, ctx.by_src = by_dst, by_src
        a_node, v_node, d_node, enc, rh = (t.contiguous() for t in (a_node, v_node, d_node, enc, rh))
        ctx.save_for_backward(a_node, v_node, d_node, enc, rh)
        ctx.save_for_forward(a_node, v_node, d_node, enc, rh)
        N, C = a_node.shape
        if enc_source is not None:
            enc8, W, b = enc_source
            b = b if b is not None else torch.zeros(C, dtype=torch.float32, device=enc.device)
            P0, S1, S2 = ops.bee_message(by_src.row_ptr, by_dst.index, rh, enc8.contiguous(), a_node,
                                         v_node.transpose(1, 2).contiguous(),
                                         d_node.reshape(N, C, 9).transpose(1, 2).contiguous(),
                                         W.detach().contiguous(), b.detach().contiguous())
            by_label = {lab: P0[:, k].contiguous() for k, lab in enumerate(("000", "110", "220"))}
            for k, lab in enumerate(_S1_LABELS):
                by_label[lab] = S1[:, :, k].transpose(1, 2).contiguous()
            for k, lab in enumerate(_S2_LABELS):
                by_label[lab] = S2[:, :, k].transpose(1, 2).contiguous().reshape(N, C, 3, 3)
            return tuple(by_label[lab] for lab in BEE_ORDER)
        phi_v, phi_d = ops.bee_edge_filters_fwd(enc, rh)
        prods = ops.bee_fwd_indexed(a_node, v_node, d_node, by_dst.index, enc, phi_v, phi_d)
        return tuple(p if lab[2] == "0" else ops.segment_sum_csr(p, by_src.row_ptr, by_src.n_rows)
                     for lab, p in zip(BEE_ORDER, prods))

    @staticmethod
    def jvp(ctx, a_t, v_t, d_t, enc_t, rh_t, *_):
        """Forward mode through the plain formulation: the products are bilinear in (node operands, edge filters), so
        the tangent is P(gathered tangents, filters) + P(gathered operands, the filters' tangent), summed per node
        like the products themselves (an operand without a tangent arrives as zeros)."""
        from .ops import BEE_ORDER
        a_node, v_node, d_node, enc, rh = ctx.saved_tensors
        by_dst, by_src = ctx.by_dst, ctx.by_src
        gather = lambda ts: [gl._Gather.apply(t, by_dst) for t in ts]
        phi_v, phi_d = _EdgeFilters.apply(enc, rh)
        phi_v_t, phi_d_t = _edge_filters_tangent(enc, rh, enc_t, rh_t)
        left = Bee.apply(*gather((a_t, v_t, d_t)), enc, phi_v, phi_d)
        right = Bee.apply(*gather((a_node, v_node, d_node)), enc_t.contiguous(), phi_v_t.contiguous(), phi_d_t.contiguous())
        prods = [a + b for a, b in zip(left, right)]
        return tuple(p if lab[2] == "0" else gl._ScatterSum.apply(p.contiguous(), by_src) for lab, p in zip(BEE_ORDER, prods))

    @staticmethod
    def backward(ctx, *dys):
        saved, by_dst, by_src = ctx.saved_tensors, ctx.by_dst, ctx.by_src
        need = ctx.needs_input_grad
        if torch.is_grad_enabled():
            with torch.enable_grad():
                leaves = [t if t.requires_grad else t.detach().requires_grad_() for t in saved]
                out = _message_products_plain(*leaves, by_dst, by_src)
                grads = torch.autograd.grad(out, leaves, dys, create_graph=True)
            return tuple(g if nd else None for g, nd in zip(grads, need)) + (None, None, None)
        a_node, v_node, d_node, enc, rh = saved
        dys = [dy.contiguous() for dy in dys]
        E = enc.size(0)
        phi_v, phi_d = ops.bee_edge_filters_fwd(enc, rh)
        d_l = (None, None, None)
        d_enc = d_rh = None
        if any(need[:3]):
            per_edge = ops.bee_bwd_indexed(0, enc, phi_v, phi_d, None, dys, by_src.index, E)
            d_l = tuple(ops.segment_sum_csr(t, by_dst.row_ptr, by_dst.n_rows, perm=by_dst.perm) if nd else None
                        for t, nd in zip(per_edge, need[:3]))
        if need[3] or need[4]:
            dr_0, dr_1, dr_2 = ops.bee_bwd_indexed(1, a_node, v_node, d_node, by_dst.index, dys, by_src.index, E)
            d_enc, d_rh = ops.bee_edge_filters_bwd(enc, rh, dr_1, dr_2)
            d_enc = d_enc + dr_0
        return (*d_l, d_enc if need[3] else None, d_rh if need[4] else None, None, None, None)


def message_products(graph, a_node, v_node, d_node, enc, rh, enc_source=None):
    """a_node (batch, nodes, chan), v_node (.., chan, 3), d_node (.., chan, 3, 3): the node operands, read at each
    edge's destination; enc (edges, chan), rh (edges, 3): what the edge filters are made of.  Returns the 13 products
    in ops.BEE_ORDER: those of rank 0 per edge, those of rank 1 and 2 summed over the edges of their source node
    ((batch * nodes, chan, ...)).  enc_source: see _MessageProducts."""
    flat = [gl._flat_nodes(graph, t) for t in (a_node, v_node, d_node)]
    enc, rh = enc.contiguous(), rh.contiguous()
    if ops.bee_indexed_supported(enc.size(1)) and all(t.data_ptr() % 16 == 0 for t in flat + [enc]):
        return _MessageProducts.apply(*flat, enc, rh, graph.by_dst, graph.by_src, enc_source)
    return _message_products_plain(*flat, enc, rh, graph.by_dst, graph.by_src)


def _edge_filters_plain(enc, rh):
    """archs/diffuser_atoms15.py:241-243"""
    return enc[..., None] * rh[..., None, :], enc[..., None, None] * rh[..., None, None, :] * rh[..., None, :, None]


def _edge_filters_tangent(enc, rh, enc_t, rh_t):
    """The derivative of _edge_filters_plain along (enc_t, rh_t): the product rule on its two and three factors."""
    phi_v_t = enc_t[..., None] * rh[..., None, :] + enc[..., None] * rh_t[..., None, :]
    rr = rh[..., None, None, :] * rh[..., None, :, None]
    rr_t = rh_t[..., None, None, :] * rh[..., None, :, None] + rh[..., None, None, :] * rh_t[..., None, :, None]
    return phi_v_t, enc_t[..., None, None] * rr + enc[..., None, None] * rr_t


class _EdgeFilters(torch.autograd.Function):
    """phi_v = enc (x) rh and phi_d = enc (x) rh (x) rh as one kernel, and their adjoint as another; a recorded
    backward pass differentiates the broadcasting arithmetic instead."""

    @staticmethod
    def forward(ctx, enc, rh):
        ctx.save_for_backward(enc, rh)
        ctx.save_for_forward(enc, rh)
        return ops.bee_edge_filters_fwd(enc.contiguous(), rh.contiguous())

    @staticmethod
    def jvp(ctx, enc_t, rh_t):
        return _edge_filters_tangent(*ctx.saved_tensors, enc_t, rh_t)

    @staticmethod
    def backward(ctx, g_v, g_d):
        enc, rh = ctx.saved_tensors
        if torch.is_grad_enabled():
            with torch.enable_grad():
                leaves = [t if t.requires_grad else t.detach().requires_grad_() for t in (enc, rh)]
                grads = torch.autograd.grad(_edge_filters_plain(*leaves), leaves, (g_v, g_d), create_graph=True)
            return tuple(g if nd else None for g, nd in zip(grads, ctx.needs_input_grad))
        d_enc, d_rh = ops.bee_edge_filters_bwd(enc.contiguous(), rh.contiguous(), g_v.contiguous(), g_d.contiguous())
        return (d_enc if ctx.needs_input_grad[0] else None), (d_rh if ctx.needs_input_grad[1] else None)


def bee_messages(msg, graph, r_ij, x_a, x_v, x_d):
    """archs/diffuser_atoms15.py:238-253"""
    enc8 = radial_encode_8(r_ij, msg.r0)
    enc = linear(msg.lin_enc, enc8)
    rh = tens_sigmoid(1, mul(r_ij, 7. / msg.r0))
    # The output linears of the vector and rank-2 channels have no bias and nothing nonlinear follows them before the
    # sum over edges, so they commute with it: the products are summed per node first and the ten linears run on N
    # rows, not E (the reference applies them per edge).  The scalar channel goes through an MLP per edge.
    prods = message_products(graph, msg.L0(x_a), msg.L1(x_v), msg.L2(x_d), enc, rh,
                             enc_source=(enc8.detach(), msg.lin_enc.weight, msg.lin_enc.bias))
    from .ops import BEE_ORDER
    psi_a, sums = None, [None, None, None]
    for lab, p in zip(BEE_ORDER, prods):
        k = int(lab[2])
        y = getattr(msg, f"Y_{lab}")(p if k == 0 else p.reshape(graph.batch, graph.nodes, *p.shape[1:]))
        if k == 0:
            psi_a = y if psi_a is None else psi_a + y
        else:
            sums[k] = y if sums[k] is None else sums[k] + y
    psi_a = psi_a + mlp_leaky(msg.mlp_a, psi_a)
    return mul(gl.edges_reduce_src(graph, psi_a), 0.1), mul(sums[1], 0.1), mul(sums[2], 0.1)


def displacement_tensors(mod, graph, r_ij):
    """archs/diffuser_atoms15.py:216-225 out of differentiable pieces: the radial MLP per edge, the edge filters
    rad (x) u and rad (x) u (x) u as one kernel (their adjoint another), sums over the edges of a source node, the two
    readouts on node rows."""
    first = mod.mlp_radial[0]
    rad = mlp_leaky(mod.mlp_radial[1], linear(first, radial_encode_8(r_ij, mod.r0)))
    u = tens_sigmoid(1, mul(r_ij, 7. / mod.r0))
    phi_v, phi_d = _EdgeFilters.apply(rad.contiguous(), u.contiguous())
    A_a, A_v, A_d = (gl.edges_reduce_src(graph, t) for t in (rad, phi_v, phi_d))
    return A_a, mod.readout_v(A_v), mod.readout_d(A_d)


def self_tens_prods(mod, x_a, x_v, x_d):
    """archs/diffuser_atoms15.py:75-95"""
    *rest, dim_a = x_a.shape
    dim_v, dim_d = x_v.shape[-2], x_d.shape[-3]
    a, v, d = x_a.reshape(-1, dim_a), x_v.reshape(-1, dim_v, 3), x_d.reshape(-1, dim_d, 3, 3)
    prods = Bee.apply(mod.L0(a), mod.L1(v), mod.L2(d), mod.R0(a), mod.R1(v), mod.R2(d))
    y_a, y_v, y_d = apply_tens_prod_submodules(mod, prods)
    return (tens_group_norm(mod.gn_a, y_a.reshape(*rest, dim_a)), tens_group_norm(mod.gn_v, y_v.reshape(*rest, dim_v, 3)),
            tens_group_norm(mod.gn_d, y_d.reshape(*rest, dim_d, 3, 3)))

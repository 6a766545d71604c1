"""TensLinear / TensorProdBare / TensorProds and the small tensor norms,
mirroring managan/tensor_products.py of the reference (same class names,
constructor arguments and parameter names, so state dicts load unchanged) on
top of the HIP kernels."""
import torch
import torch.nn as nn

from . import ops


def _row_bound(inds, x):
    """Row maxima of |x| for plain rows that the split-fp16 kernels would otherwise scan themselves (the forward
    GEMM and the weight gradient both scale by them): computed once per tensor and handed to both."""
    if inds != 0 or ops.get_linear_mode() != ops.LINEAR_F16X2 or x.dim() < 2:
        return None
    x2 = x.reshape(-1, x.shape[-1])
    if x2.size(0) < 4096 or x2.size(1) < 64 or x2.data_ptr() % 16 != 0:
        return None
    return ops.row_absmax(x2)


class _TensorLinearFn(torch.autograd.Function):
    """tensor_linear with gradients for W and x (extensions/tensor_ops/tensor_ops.cpp:31-169).  The backward pass is
    itself made of differentiable functions (this one and _WeightGradFn), so the operation can be differentiated any
    number of times, as torch.autograd.functional.jvp(create_graph=True) of the meanflow loss needs
    (archs/meanflow_painn8.py:274-282); the reference's C++ backward calls raw kernels and cannot.
    x_bound: row maxima of |x| when the caller already holds them (a scaling hint, not differentiated).
    bias (plain rows only): added in the kernel's epilogue; its gradient comes out of the weight-gradient pass."""

    @staticmethod
    def forward(ctx, inds, W, x, x_bound=None, bias=None, want_bound=False):
        ctx.inds = inds
        x = x.contiguous()
        if x_bound is None:
            x_bound = _row_bound(inds, x)
        ctx.x_bound = x_bound
        ctx.has_bias = bias is not None
        ctx.want_bound = want_bound
        ctx.save_for_backward(W, x)
        ctx.save_for_forward(W, x)
        ctx.set_materialize_grads(False)
        bias = None if bias is None else bias.contiguous()
        if not want_bound:
            return ops.tensor_linear_fwd(inds, W, x, bias=bias, row_bound=x_bound)
        # the kernel's partial row maxima of |y| (an empty tensor when the kernel that ran does not produce them)
        y, y_bound = ops.tensor_linear_fwd(inds, W, x, bias=bias, row_bound=x_bound, want_rowmax=True)
        if y_bound is None:
            y_bound = y.new_empty(0)
        ctx.mark_non_differentiable(y_bound)
        return y, y_bound

    @staticmethod
    def jvp(ctx, _inds, W_t, x_t, *rest):
        """Forward-mode derivative: y_t = x_t W^T + x W_t^T + bias_t, each piece this same function, so that a
        backward pass through the tangent runs on the same kernels.  (One tangent per argument that apply was given.)"""
        W, x = ctx.saved_tensors
        bias_t = rest[1] if len(rest) > 1 else None
        parts = []
        if x_t is not None:
            parts.append(_TensorLinearFn.apply(ctx.inds, W, x_t))
        if W_t is not None:
            parts.append(_TensorLinearFn.apply(ctx.inds, W_t, x, ctx.x_bound))
        if bias_t is not None:
            parts.append(bias_t.expand_as(parts[0]) if parts else bias_t)
        y_t = sum(parts[1:], parts[0]) if parts else None
        return (y_t, None) if ctx.want_bound else y_t

    @staticmethod
    def backward(ctx, dy, *_):
        W, x = ctx.saved_tensors
        if dy is None:
            return None, None, None, None, None, None
        dy = dy.contiguous()
        dW = dx = db = None
        dy_bound = _row_bound(ctx.inds, dy)
        want_bias = ctx.has_bias and ctx.needs_input_grad[4]
        if ctx.needs_input_grad[1] or want_bias:
            dW, db = _WeightGradFn.apply(ctx.inds, dy, x, dy_bound, ctx.x_bound, want_bias)
            if not want_bias:
                db = None
        if ctx.needs_input_grad[2]:
            dx = _TensorLinearFn.apply(ctx.inds, W.t(), dy, dy_bound)   # strides of W are honoured: no copy
        return None, dW, dx, None, db, None


class _WeightGradFn(torch.autograd.Function):
    """dW[o, i] = sum over rows and components of dy[.., o, :] x[.., i, :], and with want_bias db[o] = sum over rows of
    dy[.., o] (else an empty tensor): bilinear / linear in (dy, x), and their own gradients are two tensor_linear
    calls."""

    @staticmethod
    def forward(ctx, inds, dy, x, dy_bound=None, x_bound=None, want_bias=False):
        ctx.inds = inds
        ctx.bounds = (dy_bound, x_bound)
        ctx.want_bias = want_bias
        ctx.save_for_backward(dy, x)
        out = ops.tensor_linear_wgrad(inds, dy.contiguous(), x.contiguous(), dy_bound=dy_bound, x_bound=x_bound,
                                      want_bias=want_bias)
        if want_bias:
            return out
        db = dy.new_empty(0)
        ctx.mark_non_differentiable(db)
        return out, db

    @staticmethod
    def backward(ctx, ddW, ddb):
        dy, x = ctx.saved_tensors
        dy_bound, x_bound = ctx.bounds
        g_dy = g_x = None
        if ctx.needs_input_grad[1]:
            # (.., o, :) = ddW x (+ ddb)
            g_dy = _TensorLinearFn.apply(ctx.inds, ddW, x, x_bound, ddb if ctx.want_bias else None)
        if ctx.needs_input_grad[2]:
            g_x = _TensorLinearFn.apply(ctx.inds, ddW.t(), dy, dy_bound)       # (.., i, :) = ddW^T dy
        return None, g_dy, g_x, None, None, None


def tensor_linear(inds, W, x, bias=None, x_bound=None, want_bound=False):
    """bias (inds = 0 only): y = x W^T + bias in one kernel.  x_bound: upper bounds of the row maxima of |x|
    ((rows, parts)) when the caller holds them.  want_bound: returns (y, bound) with the kernel's partial row maxima
    of |y|, or None where the kernel that ran does not produce them: they bound |f(y)| for any f with |f(z)| <= |z|
    (SiLU, LeakyReLU) and save the next layer its pass over the rows."""
    if bias is not None and inds != 0:
        raise RuntimeError("a bias is defined for plain rows only")
    x = x.contiguous()          # (here, where autograd records the copy: the function saves x for later derivatives)
    if not want_bound:
        return _TensorLinearFn.apply(inds, W, x, x_bound, bias)
    y, y_bound = _TensorLinearFn.apply(inds, W, x, x_bound, bias, True)
    return y, (y_bound if y_bound.numel() else None)


class TensLinear(nn.Module):
    """Linear layer for arbitrary tensor activations (managan/tensor_products.py:26-37)."""

    def __init__(self, inds, dim_in, dim_out):
        super().__init__()
        self.W = nn.Parameter(torch.empty(dim_out, dim_in))
        self.inds = inds
        self.self_init()

    def self_init(self):
        _, fan_in = self.W.shape
        nn.init.normal_(self.W, std=fan_in ** -0.5)

    def forward(self, x):
        return tensor_linear(self.inds, self.W, x.contiguous())


class TensorProdBare(nn.Module):
    """Tensor product with no linear maps around it (managan/tensor_products.py:91-106)."""

    def __init__(self, inds_l, inds_r, inds_o):
        super().__init__()
        assert (inds_l + inds_r - inds_o) % 2 == 0, "parity mismatch"
        contracts = (inds_l + inds_r - inds_o) // 2
        assert 0 <= contracts <= min(inds_l, inds_r), \
            f"{contracts} contractions is out of range for {inds_l}, {inds_r} index tensors"
        self.inds = (inds_l, inds_r, inds_o)

    def forward(self, x_l, x_r):
        if torch.is_grad_enabled() and (x_l.requires_grad or x_r.requires_grad):
            return _ProdBareFn.apply(*self.inds, x_l, x_r)
        return ops.tensor_prod_bare(*self.inds, x_l.contiguous(), x_r.contiguous())


def _swap_index_groups(x, first, second):
    """x (..., chan, (3,)^(first + second)) with its trailing indices in two groups: the groups exchanged.  With
    ranks up to 2 that is a transposition when both groups hold one index, and nothing otherwise."""
    return x.transpose(-1, -2).contiguous() if first == 1 and second == 1 else x


class _ProdBareFn(torch.autograd.Function):
    """One product y[keep_l, keep_r] = sum_con l[keep_l, con] r[keep_r, con] (the reference relies on
    torch.einsum's autograd, managan/tensor_products.py:104-106).  Both gradients are products of the same family
    with index groups exchanged,
        dl[keep_l, con] = sum_keep_r dy[keep_l, keep_r] r[keep_r, con]     type (inds_o, inds_r, inds_l)
        dr[keep_r, con] = sum_keep_l dy[keep_l, keep_r] l[keep_l, con]     type (inds_o, inds_l, inds_r)
    and they are taken through this function again, so the product is differentiable any number of times at the
    cost of one product kernel per gradient."""

    @staticmethod
    def forward(ctx, il, ir, io, x_l, x_r):
        ctx.inds = (il, ir, io)
        ctx.save_for_backward(x_l, x_r)
        ctx.save_for_forward(x_l, x_r)
        ctx.set_materialize_grads(False)
        return ops.tensor_prod_bare(il, ir, io, x_l.contiguous(), x_r.contiguous())

    @staticmethod
    def jvp(ctx, _il, _ir, _io, l_t, r_t):
        """Bilinear: the product with one operand's tangent in its place, summed over the operands that have one."""
        x_l, x_r = ctx.saved_tensors
        parts = [_ProdBareFn.apply(*ctx.inds, a, b) for a, b in ((l_t, x_r), (x_l, r_t)) if a is not None and b is not None]
        return sum(parts[1:], parts[0])

    @staticmethod
    def backward(ctx, dy):
        if dy is None:
            return None, None, None, None, None
        il, ir, io = ctx.inds
        k = (il + ir - io) // 2                       # contracted indices; il - k and ir - k are kept
        x_l, x_r = ctx.saved_tensors
        dl = dr = None
        if ctx.needs_input_grad[3]:
            dl = _ProdBareFn.apply(io, ir, il, dy, _swap_index_groups(x_r, ir - k, k))
        if ctx.needs_input_grad[4]:
            dr = _ProdBareFn.apply(io, il, ir, _swap_index_groups(dy, il - k, ir - k), _swap_index_groups(x_l, il - k, k))
        return None, None, None, dl, dr


def _prod_with_grad(inds, x_l, x_r):
    """The product through the 13-product autograd function: the operands take their ranks' slots, the other slots
    are zeros, and the output of type (inds_l inds_r inds_o) is picked.  Ten times the arithmetic of _ProdBareFn;
    kept as an independent route that the tests compare it with."""
    from .codegen_tensor_products import Bee
    il, ir, io = inds
    lead = x_l.shape[:x_l.dim() - il - 1]
    chan = x_l.shape[len(lead)]
    if tuple(x_r.shape[:x_r.dim() - ir]) != tuple(lead) + (chan,):
        raise RuntimeError(f"operands do not broadcast: {tuple(x_l.shape)} vs {tuple(x_r.shape)}")
    rows = 1
    for d in lead:
        rows *= int(d)
    def slots(x, rank):
        out = [torch.zeros(rows, chan, *([3] * k), dtype=torch.float32, device=x.device) for k in range(3)]
        out[rank] = x.reshape(rows, chan, *([3] * rank))
        return out
    ys = Bee.apply(*slots(x_l, il), *slots(x_r, ir))
    y = ys[ops.BEE_ORDER.index(f"{il}{ir}{io}")]
    return y.reshape(*lead, chan, *([3] * io))


def _torch_ext():
    from . import _lib
    return _lib.load_torch_ext()


class TensorProds(nn.Module):
    """Tensor product sandwiched by linear maps (managan/tensor_products.py:109-121)."""

    def __init__(self, inds_l: int, inds_r: int, inds_o: int, dim_l: int, dim_r: int, dim_o: int, rank: int):
        super().__init__()
        self.prod = TensorProdBare(inds_l, inds_r, inds_o)
        self.lin_l = TensLinear(inds_l, dim_l, rank)
        self.lin_r = TensLinear(inds_r, dim_r, rank)
        self.lin_o = TensLinear(inds_o, rank, dim_o)

    def forward(self, x_l, x_r):
        W_l, W_r, W_o = self.lin_l.W, self.lin_r.W, self.lin_o.W
        wants_grad = torch.is_grad_enabled() and any(t.requires_grad for t in (x_l, x_r, W_l, W_r, W_o))
        if not wants_grad:
            # one launch, nothing stored between; through the C++ binding (a node-sized call is host time)
            ext = _torch_ext()
            if ext.tensor_prods_supported(*self.prod.inds, W_l.shape[1], W_r.shape[1], W_l.shape[0], W_o.shape[0]):
                return ext.tensor_prods(*self.prod.inds, W_l, W_r, W_o, x_l, x_r)
        return self.lin_o(self.prod(self.lin_l(x_l), self.lin_r(x_r)))


def tens_sigmoid(inds, x):
    """x / sqrt(1 + |x|^2) over the trailing `inds` tensor indices (managan/tensor_products.py:167-182)."""
    from . import differentiable as diff
    if diff.differentiated(x):
        return diff.tens_sigmoid(inds, x)
    return ops.tens_sigmoid(inds, x.contiguous())


class TensSigmoid(nn.Module):
    """managan/tensor_products.py:184-189"""

    def __init__(self, inds):
        super().__init__()
        self.inds = inds

    def forward(self, x):
        return tens_sigmoid(self.inds, x)


def __getattr__(name):
    # TensGroupNorm (managan/tensor_products.py:215-232) lives beside the layers that use it, which import this module
    if name == "TensGroupNorm":
        from .bee_layers import TensGroupNorm
        return TensGroupNorm
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")

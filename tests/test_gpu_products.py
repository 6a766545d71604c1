"""HIP tensor products against the CPU oracle (oracle/products.py).
Tolerance: rel 1e-5 / abs 1e-6 in fp32, as the path's contract states."""
import importlib

import pytest
import torch

from oracle import products as OP

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-5, 1e-6


def _inputs(rows, chan, seed, ranks=(0, 1, 2)):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(rows, chan, *([3] * k), generator=g) for k in ranks]


def _close(a, b):
    torch.testing.assert_close(a.cpu(), b, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("rows,chan", [(10, 256), (1, 1), (7, 33), (513, 17), (4096, 64)])
def test_bee_fwd(ops, rows, chan):
    l = _inputs(rows, chan, 0x947)
    r = _inputs(rows, chan, 0x948)
    ys = ops.bee_fwd(*[t.cuda() for t in l], *[t.cuda() for t in r])
    ref = OP.bee(*l, *r)
    assert len(ys) == 13
    for lab, y, y_ref in zip(OP.BEE_ORDER, ys, ref):
        assert tuple(y.shape) == tuple(y_ref.shape), lab
        _close(y, y_ref)


def test_bee_fwd_empty(ops):
    l = [t.cuda() for t in _inputs(0, 8, 1)]
    r = [t.cuda() for t in _inputs(0, 8, 2)]
    ys = ops.bee_fwd(*l, *r)
    assert [tuple(y.shape) for y in ys][:4] == [(0, 8), (0, 8), (0, 8), (0, 8, 3)]


@pytest.mark.parametrize("rows,chan", [(10, 256), (3, 5), (300, 40)])
def test_bee_bwd(ops, rows, chan):
    l = _inputs(rows, chan, 11)
    r = _inputs(rows, chan, 12)
    g = torch.Generator().manual_seed(13)
    dys = [torch.randn(rows, chan, *([3] * int(lab[2])), generator=g) for lab in OP.BEE_ORDER]
    dl_ref, dr_ref = OP.products_backward(OP.BEE_ORDER, l, r, dys)
    dl = ops.bee_bwl(*[t.cuda() for t in r], *[t.cuda() for t in dys])
    dr = ops.bee_bwr(*[t.cuda() for t in l], *[t.cuda() for t in dys])
    for a, b in zip(dl + dr, dl_ref + dr_ref):
        torch.testing.assert_close(a.cpu(), b, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("rows,chan", [(10, 256), (5, 3)])
def test_cow(ops, rows, chan):
    l = _inputs(rows, chan, 21, (0, 1))
    r = _inputs(rows, chan, 22, (0, 1))
    lc, rc = [t.cuda() for t in l], [t.cuda() for t in r]
    for y, y_ref in zip(ops.cow_o0_fwd(*lc, *rc), OP.cow0(*l, *r)):
        _close(y, y_ref)
    for y, y_ref in zip(ops.cow_o1_fwd(*lc, *rc), OP.cow1(*l, *r)):
        _close(y, y_ref)
    g = torch.Generator().manual_seed(23)
    for order, bwl, bwr in ((OP.COW0_ORDER, ops.cow_o0_bwl, ops.cow_o0_bwr),
                            (OP.COW1_ORDER, ops.cow_o1_bwl, ops.cow_o1_bwr)):
        dys = [torch.randn(rows, chan, *([3] * int(lab[2])), generator=g) for lab in order]
        dl_ref, dr_ref = OP.products_backward(order, l + [None], r + [None], dys)
        dl = bwl(*rc, *[t.cuda() for t in dys])
        dr = bwr(*lc, *[t.cuda() for t in dys])
        for a, b in zip(dl + dr, dl_ref[:2] + dr_ref[:2]):
            torch.testing.assert_close(a.cpu(), b, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("lro", [(0, 0, 0), (1, 1, 0), (2, 2, 0), (0, 1, 1), (1, 0, 1), (1, 2, 1), (2, 1, 1),
                                 (0, 2, 2), (2, 0, 2), (1, 1, 2), (2, 2, 2)])
def test_tensor_prod_bare(ops, lro):
    il, ir, io = lro
    g = torch.Generator().manual_seed(31)
    x_l = torch.randn(6, 9, 20, *([3] * il), generator=g)
    x_r = torch.randn(6, 9, 20, *([3] * ir), generator=g)
    y = ops.tensor_prod_bare(il, ir, io, x_l.cuda(), x_r.cuda())
    _close(y, OP.tensor_prod_bare(il, ir, io, x_l, x_r))


def test_tensor_prod_bare_rejects(ops):
    x = torch.randn(4, 8, 3).cuda()
    with pytest.raises(RuntimeError):
        ops.tensor_prod_bare(1, 1, 1, x, x)      # parity mismatch (chiral)


def test_config1_trio(ops):
    """BASELINE config 1 shapes: x (4096,64), v (4096,64,3)."""
    g = torch.Generator().manual_seed(0x947 + 1)
    x = torch.randn(4096, 64, generator=g)
    v = torch.randn(4096, 64, 3, generator=g)
    y0, y1, y2 = ops.tensor_prods_avd(x.cuda(), v.cuda(), v.cuda())
    _close(y0, OP.tensor_prod_bare(1, 1, 0, v, v))
    _close(y1, OP.tensor_prod_bare(0, 1, 1, x, v))
    _close(y2, OP.tensor_prod_bare(1, 1, 2, v, v))


def test_unaligned_views(ops):
    """Operands that are not 16-byte aligned take the scalar staging path."""
    rows, chan = 9, 40
    l = _inputs(rows, chan, 41)
    r = _inputs(rows, chan, 42)

    def shifted(t):
        buf = torch.empty(t.numel() + 1, device="cuda")
        view = buf[1:].view(t.shape)
        view.copy_(t)
        return view

    ys = ops.bee_fwd(*[shifted(t) for t in l], *[shifted(t) for t in r])
    for y, y_ref in zip(ys, OP.bee(*l, *r)):
        _close(y, y_ref)


_TP_TYPES = [(0, 0, 0), (1, 1, 0), (2, 2, 0), (0, 1, 1), (1, 0, 1), (1, 2, 1), (2, 1, 1), (0, 2, 2), (2, 0, 2), (1, 1, 2),
             (2, 2, 2)]


def _tp_case(lro, rows, dims, seed):
    il, ir, io = lro
    dim_l, dim_r, rank, dim_o = dims
    g = torch.Generator().manual_seed(seed)
    x_l = torch.randn(rows, dim_l, *([3] * il), generator=g)
    x_r = torch.randn(rows, dim_r, *([3] * ir), generator=g)
    W_l = torch.randn(rank, dim_l, generator=g) * dim_l ** -0.5
    W_r = torch.randn(rank, dim_r, generator=g) * dim_r ** -0.5
    W_o = torch.randn(dim_o, rank, generator=g) * rank ** -0.5
    return x_l, x_r, W_l, W_r, W_o


@pytest.mark.parametrize("lro", _TP_TYPES)
def test_tensor_prods_one_launch(ops, lro):
    """lin_o(prod(lin_l, lin_r)) in one kernel (managan/tensor_products.py:109-121): every product type, channel
    counts that all differ (80 output channels: two grid rows of output tiles), a row count that fills neither a
    wave's 16 rows nor a workgroup's 64."""
    from parity import assert_parity
    dims = (32, 48, 64, 80)
    x_l, x_r, W_l, W_r, W_o = _tp_case(lro, 150, dims, 100 + sum(lro))
    assert ops.tensor_prods_supported(*lro, *dims)
    y = ops.tensor_prods(*lro, W_l.cuda(), W_r.cuda(), W_o.cuda(), x_l.cuda(), x_r.cuda())
    ref32 = OP.tensor_prods(*lro, W_l, W_r, W_o, x_l, x_r)
    ref64 = OP.tensor_prods(*lro, W_l.double(), W_r.double(), W_o.double(), x_l.double(), x_r.double())
    assert_parity(y, ref32, ref64, what=f"tensor_prods {lro}")


def test_tensor_prods_module_routes_and_agrees(ops):
    """TensorProds.forward takes the one-launch kernel when nothing asks for a gradient and the three-step path
    otherwise; both agree with the oracle; strided weights (a transposed view) and leading batch axes are honoured;
    unsupported channel counts fall back."""
    from parity import assert_parity
    tp = importlib.import_module("learned-dynamics_amd.tensor_products")
    torch.manual_seed(5)
    mod = tp.TensorProds(1, 1, 2, 64, 64, 64, 64).cuda()
    g = torch.Generator().manual_seed(6)
    v = torch.randn(3, 50, 64, 3, generator=g)
    w = torch.randn(3, 50, 64, 3, generator=g)
    W = [p.detach().cpu() for p in (mod.lin_l.W, mod.lin_r.W, mod.lin_o.W)]
    ref32 = OP.tensor_prods(1, 1, 2, *W, v, w)
    ref64 = OP.tensor_prods(1, 1, 2, *[t.double() for t in W], v.double(), w.double())
    with torch.no_grad():
        fused = mod(v.cuda(), w.cuda())
    stepwise = mod(v.cuda(), w.cuda())                       # parameters require grad: three-step path
    assert fused.shape == (3, 50, 64, 3, 3) and stepwise.requires_grad and not fused.requires_grad
    assert_parity(fused, ref32, ref64, what="TensorProds fused")
    assert_parity(stepwise, ref32, ref64, what="TensorProds stepwise")
    Wt = W[0].t().contiguous().cuda().t()                    # same values, column-major storage
    y = ops.tensor_prods(1, 1, 2, Wt, W[1].cuda(), W[2].cuda(), v.cuda(), w.cuda())
    assert torch.equal(y, fused)
    assert not ops.tensor_prods_supported(1, 1, 2, 64, 64, 40, 64)
    assert not ops.tensor_prods_supported(1, 1, 1, 64, 64, 64, 64)
    small = tp.TensorProds(0, 1, 1, 24, 24, 40, 24).cuda()   # not multiples of 16: composed path
    with torch.no_grad():
        ys = small(v[..., :24, 0].contiguous().cuda(), w[..., :24, :].contiguous().cuda())
    Ws = [p.detach().cpu() for p in (small.lin_l.W, small.lin_r.W, small.lin_o.W)]
    _close(ys, OP.tensor_prods(0, 1, 1, *Ws, v[..., :24, 0], w[..., :24, :]))
    with pytest.raises(RuntimeError, match="multiples of 16"):
        ops.tensor_prods(0, 1, 1, *[t.cuda() for t in Ws], v[..., :24, 0].contiguous().cuda(), w[..., :24, :].contiguous().cuda())
    assert ops.tensor_prods(1, 1, 2, *[t.cuda() for t in W], v[:0].cuda(), w[:0].cuda()).shape == (0, 50, 64, 3, 3)

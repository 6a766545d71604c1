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

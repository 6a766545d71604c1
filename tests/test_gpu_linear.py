"""MFMA tensor_linear against the oracle (plain matmul): rel 1e-5 / abs 1e-6 against the float64 evaluation, widened
only by twice the distance of the float32 evaluation of the same formula from it (tests/parity.py)."""
import importlib

import pytest
import torch

from oracle import products as OP
from parity import assert_parity_of

pytestmark = pytest.mark.gpu


def _check(y, formula, what="tensor_linear"):
    """formula(dtype): the reference on the CPU in that dtype."""
    assert_parity_of(y, formula, what)


@pytest.mark.parametrize("inds", [0, 1, 2])
@pytest.mark.parametrize("dims", [(64, 64), (117, 210), (16, 512), (128, 32), (8, 128), (20, 256), (1, 64), (64, 1)])
def test_tensor_linear(ops, inds, dims):
    dim_in, dim_out = dims
    g = torch.Generator().manual_seed(100 + inds)
    W = torch.randn(dim_out, dim_in, generator=g) * dim_in ** -0.5
    x = torch.randn(10, 37, dim_in, *([3] * inds), generator=g)
    y = ops.tensor_linear_fwd(inds, W.cuda(), x.cuda())
    assert tuple(y.shape) == (10, 37, dim_out) + (3,) * inds
    _check(y, lambda dt: OP.tensor_linear(inds, W.to(dt), x.to(dt)))


@pytest.mark.parametrize("inds", [0, 1, 2])
def test_tensor_linear_transposed_weight(ops, inds):
    g = torch.Generator().manual_seed(7)
    W = torch.randn(96, 48, generator=g)
    x = torch.randn(50, 96, *([3] * inds), generator=g)
    y = ops.tensor_linear_fwd(inds, W.cuda().t(), x.cuda())
    _check(y, lambda dt: OP.tensor_linear(inds, W.t().to(dt), x.to(dt)))


def test_tensor_linear_large_rows(ops):
    g = torch.Generator().manual_seed(8)
    W = torch.randn(512, 512, generator=g) / 512 ** 0.5
    x = torch.randn(3000, 512, generator=g)
    b = torch.randn(512, generator=g)
    y = ops.tensor_linear_fwd(0, W.cuda(), x.cuda(), bias=b.cuda(), act=ops.ACT_SILU)
    lin = lambda dt: torch.nn.functional.linear(x.to(dt), W.to(dt), b.to(dt))
    _check(y, lambda dt: torch.nn.functional.silu(lin(dt)))
    y2 = ops.tensor_linear_fwd(0, W.cuda(), x.cuda(), bias=b.cuda(), act=ops.ACT_LEAKY)
    _check(y2, lambda dt: torch.nn.functional.leaky_relu(lin(dt), 0.1))


def test_tensor_linear_accumulate(ops):
    g = torch.Generator().manual_seed(9)
    W = torch.randn(40, 24, generator=g)
    x = torch.randn(33, 24, 3, generator=g)
    base = torch.randn(33, 40, 3, generator=g)
    out = base.cuda().clone()
    ops.tensor_linear_fwd(1, W.cuda(), x.cuda(), out=out, accumulate=True)
    _check(out, lambda dt: base.to(dt) + OP.tensor_linear(1, W.to(dt), x.to(dt)))


@pytest.mark.parametrize("inds", [0, 1, 2])
@pytest.mark.parametrize("rows,dim_in,dim_out", [(4096, 128, 1), (77, 16, 3), (1001, 132, 4), (5, 1280, 2), (1, 64, 1)])
def test_tensor_linear_with_a_few_output_channels(ops, inds, rows, dim_in, dim_out):
    """Readout shapes (at most four output channels) have a kernel of their own: every layout, weight stride,
    bias / activation and the accumulating form against float64."""
    g = torch.Generator().manual_seed(300 + 10 * inds + dim_out)
    T = 3 ** inds
    W = torch.randn(dim_out, dim_in, generator=g) * dim_in ** -0.5
    x = torch.randn(rows, dim_in, *([3] * inds), generator=g)
    ref = lambda dt: torch.einsum("oi,ri...->ro...", W.to(dt), x.to(dt))
    y = ops.tensor_linear_fwd(inds, W.cuda(), x.cuda())
    assert tuple(y.shape) == (rows, dim_out) + (3,) * inds
    _check(y, ref)
    # a weight with strides (the transposed view the input gradient of an n -> few linear would pass is the other
    # shape; this is the forward of a layer whose weight is stored transposed)
    Wt = W.t().contiguous().cuda().t()
    assert dim_out == 1 or Wt.stride() == (1, dim_out)
    _check(ops.tensor_linear_fwd(inds, Wt, x.cuda()), ref)
    # component-major output
    ycm = ops.tensor_linear_fwd(inds, W.cuda(), x.cuda(), y_layout=ops.LAYOUT_COMP_CHAN)
    _check(ycm.reshape(rows, T, dim_out), lambda dt: ref(dt).reshape(rows, dim_out, T).transpose(1, 2))
    # accumulate
    base = torch.randn(rows, dim_out, *([3] * inds), generator=g)
    out = base.cuda().clone()
    ops.tensor_linear_fwd(inds, W.cuda(), x.cuda(), out=out, accumulate=True)
    _check(out, lambda dt: base.to(dt) + ref(dt))
    if inds == 0:
        b = torch.randn(dim_out, generator=g)
        yb = ops.tensor_linear_fwd(0, W.cuda(), x.cuda(), bias=b.cuda(), act=ops.ACT_SILU)
        _check(yb, lambda dt: torch.nn.functional.silu(ref(dt) + b.to(dt)))


def test_tensor_linear_empty_and_errors(ops):
    W = torch.randn(8, 4).cuda()
    y = ops.tensor_linear_fwd(1, W, torch.empty(0, 4, 3).cuda())
    assert tuple(y.shape) == (0, 8, 3)
    with pytest.raises(RuntimeError, match="channel dim size mismatch"):
        ops.tensor_linear_fwd(0, W, torch.randn(3, 5).cuda())
    with pytest.raises(RuntimeError, match="3d"):
        ops.tensor_linear_fwd(1, W, torch.randn(3, 4, 2).cuda())
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.tensor_linear_fwd(0, W, torch.randn(4, 3).cuda().t())
    with pytest.raises(RuntimeError, match="up to 2"):
        ops.tensor_linear_fwd(3, W, torch.randn(2, 4, 3, 3, 3).cuda())


@pytest.mark.parametrize("inds", [0, 1, 2])
def test_tensor_linear_autograd(pkg, inds):
    tp = importlib.import_module("learned-dynamics_amd.tensor_products")
    g = torch.Generator().manual_seed(10)
    W = torch.randn(70, 50, generator=g)
    x = torch.randn(6, 21, 50, *([3] * inds), generator=g)
    dy = torch.randn(6, 21, 70, *([3] * inds), generator=g)
    Wr, xr = W.clone().requires_grad_(True), x.clone().requires_grad_(True)
    OP.tensor_linear(inds, Wr, xr).backward(dy)
    Wg, xg = W.cuda().requires_grad_(True), x.cuda().requires_grad_(True)
    tp.tensor_linear(inds, Wg, xg).backward(dy.cuda())
    torch.testing.assert_close(xg.grad.cpu(), xr.grad, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(Wg.grad.cpu(), Wr.grad, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("shape", [(5000, 512, 512, 0), (3000, 96, 200, 0), (2000, 64, 128, 1), (1500, 160, 72, 2),
                                   (1024, 64, 64, 0), (4096, 768, 256, 0),
                                   # large enough for the 256x256-tile kernel (ragged last tile; transposed output)
                                   (140001, 64, 512, 0), (90001, 32, 256, 1)])
def test_linear_modes_agree_with_float64(ops, mode, shape):
    """fp32 MFMA (mode 0), bf16x3-split MFMA (mode 1) and two-piece fp16 split (mode 2) against a float64
    product: all must sit at fp32 rounding level; the split paths use pre-packed weights and may
    transpose (row, comp) outputs."""
    rows, dim_in, dim_out, inds = shape
    T = 3 ** inds
    g = torch.Generator().manual_seed(77)
    W = torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5
    b = torch.randn(dim_out, generator=g)
    x_cm = torch.randn(rows, T, dim_in, generator=g)                   # component-major rows
    def ref_aos(dt):
        ref = torch.nn.functional.silu(x_cm.to(dt) @ W.to(dt).t() + b.to(dt))            # (rows, T, O)
        return ref.transpose(1, 2).reshape(rows, dim_out, *([3] * inds))

    prev = ops.get_linear_mode()
    try:
        ops.set_linear_mode(mode)
        C = ops.LAYOUT_COMP_CHAN
        y = ops.tensor_linear_fwd(inds, W.cuda(), x_cm.cuda() if inds else x_cm[:, 0].contiguous().cuda(),
                                  bias=b.cuda(), act=ops.ACT_SILU, x_layout=C if inds else 0)
    finally:
        ops.set_linear_mode(prev)
    _check(y, ref_aos, f"tensor_linear mode {mode} {shape}")


@pytest.mark.parametrize("shape", [(70000, 512, 512, 1), (3001, 256, 192, 0), (1500, 96, 16, 2), (2048, 1280, 64, 0),
                                   (1024, 64, 8, 0), (40000, 160, 130, 1), (140001, 64, 256, 2),
                                   # column tiles chosen to divide the width and narrowed for few rows
                                   (49152, 128, 384, 1), (16384, 256, 384, 0), (512, 512, 512, 1), (300, 64, 96, 2),
                                   (700, 64, 2080, 0), (2048, 64, 1056, 0),
                                   # few rows, at most 64 columns, long K: the waves of a workgroup split K
                                   (18432, 1280, 16, 0), (6144, 1280, 64, 2), (33, 512, 32, 1), (1000, 544, 40, 0),
                                   (8192, 768, 64, 1), (32768, 768, 16, 1), (1, 2048, 3, 0)])
def test_linear_f16x2_rows_of_very_different_size(ops, shape):
    """mg_tensor_linear_f16x2 through the C ABI.  Rows spanning twelve orders of magnitude: the per-row
    power-of-two scales keep the error relative to EACH row's own scale at fp32 rounding level (a single
    scale for the tensor would not); weight rows of different size likewise.  Also: accumulate, the row
    maxima the epilogue emits, and their use as the next call's bounds."""
    rows, dim_in, dim_out, act = shape
    g = torch.Generator().manual_seed(rows + dim_out)
    W = torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5
    W[::3] *= 1e-4
    W[1::5] *= 300.0
    b = torch.randn(dim_out, generator=g) * 1e-3
    x = torch.randn(rows, dim_in, generator=g)
    x *= 10.0 ** torch.randint(-6, 7, (rows, 1), generator=g).float()
    pre = x.double() @ W.double().t() + b.double()
    ref = {0: pre, 1: torch.nn.functional.silu(pre), 2: torch.where(pre > 0, pre, 0.1 * pre)}[act]
    # error budget per entry: fp32-level rounding of a length-K dot product whose terms are bounded by
    # |x row| * |W row|, plus rel 2e-6 of the result (rounding, hardware exp2 / reciprocal in SiLU)
    budget = (x.abs().amax(1, keepdim=True).double() * W.abs().amax(1).double() * 4e-7 * dim_in ** 0.5
              + 2e-6 * ref.abs() + 1e-30)
    y, ymax = ops.tensor_linear_f16x2(W.cuda(), x.cuda(), bias=b.cuda(), act=act, want_rowmax=True)
    assert bool(((y.cpu().double() - ref).abs() <= budget).all())
    assert torch.equal(ymax.amax(dim=1), y.abs().amax(dim=1))
    # explicit bounds: exact maxima, and a loose shared bound (accuracy must not depend on tightness)
    y2 = ops.tensor_linear_f16x2(W.cuda(), x.cuda(), ops.row_absmax(x.cuda()) * 100.0, bias=b.cuda(), act=act)
    assert bool(((y2.cpu().double() - ref).abs() <= budget).all())
    # accumulate into an existing result, bounds taken from the previous call's emitted maxima
    W2 = torch.randn(dim_in, dim_out, generator=g) / dim_out ** 0.5
    if dim_out % 32 == 0 and dim_out >= 64:
        base = torch.randn(rows, dim_in, generator=g)
        out = base.cuda().clone()
        ops.tensor_linear_f16x2(W2.cuda(), y, ymax, out=out, accumulate=True)
        ref2 = base.double() + y.cpu().double() @ W2.double().t()
        budget2 = (y.cpu().abs().amax(1, keepdim=True).double() * W2.abs().amax(1).double() * 4e-7 * dim_out ** 0.5
                   + 2e-6 * ref2.abs() + 4e-7 * base.abs().double() + 1e-30)
        assert bool(((out.cpu().double() - ref2).abs() <= budget2).all())


@pytest.mark.parametrize("nodes,T,dim_in,dim_out", [(700, 9, 320, 16), (2048, 9, 1280, 16), (2048, 3, 1280, 64),
                                                    (37, 3, 640, 24)])
def test_linear_f16x2_component_outputs_and_node_bounds(ops, nodes, T, dim_in, dim_out):
    """Rows that are (node, comp) pairs with one bound per node, output stored (node, chan, comp); the shapes with
    K >= 512 take the kernel whose waves split K."""
    g = torch.Generator().manual_seed(4)
    W = torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5
    x = torch.randn(nodes, T, dim_in, generator=g)
    bound = x.abs().amax(dim=(1, 2)).reshape(nodes, 1)
    y = ops.tensor_linear_f16x2(W.cuda(), x.reshape(nodes * T, dim_in).cuda(), bound.cuda(), out_comps=T,
                                rows_per_bound=T)
    ref = lambda dt: (x.to(dt) @ W.to(dt).t()).transpose(1, 2)
    assert y.shape == (nodes, dim_out, T)
    _check(y, ref, "f16x2, component outputs, one bound per node")
    base = torch.randn(nodes, dim_out, T, generator=g)
    out = base.cuda().clone()
    ops.tensor_linear_f16x2(W.cuda(), x.reshape(nodes * T, dim_in).cuda(), bound.cuda(), out=out, accumulate=True,
                            out_comps=T, rows_per_bound=T)
    _check(out, lambda dt: base.to(dt) + ref(dt), "f16x2, component outputs, accumulate")


@pytest.mark.parametrize("inds,rows,dim_in,dim_out", [(1, 12000, 64, 256), (2, 4000, 16, 128), (1, 11000, 40, 64)])
def test_rows_per_component_formed_once_for_several_weights(ops, inds, rows, dim_in, dim_out):
    """components_as_rows + x_rows=: two weights applied to the same x give, bit for bit, what two plain calls give;
    None (and the plain route) when the input would not take that path."""
    g = torch.Generator().manual_seed(inds + rows)
    x = torch.randn(rows, dim_in, *([3] * inds), generator=g).cuda()
    shared = ops.components_as_rows(inds, x)
    assert shared is not None and shared[0].shape[0] == rows * 3 ** inds and shared[0].shape[1] % 32 == 0
    for k in range(2):
        W = (torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5).cuda()
        y0 = ops.tensor_linear_fwd(inds, W, x, y_layout=ops.LAYOUT_COMP_CHAN)
        y1 = ops.tensor_linear_fwd(inds, W, x, y_layout=ops.LAYOUT_COMP_CHAN, x_rows=shared)
        assert torch.equal(y0, y1)
        _check(y1, lambda dt: OP.tensor_linear(inds, W.cpu().to(dt), x.cpu().to(dt)).reshape(
            rows, dim_out, 3 ** inds).transpose(1, 2), "shared rows per component")
    assert ops.components_as_rows(inds, x[:100].contiguous()) is None
    assert ops.components_as_rows(0, x) is None


def test_row_bounds_carried_as_factor_and_offset(ops):
    """ScaledBound: a chain of three layers that hands the first layer's row maxima on as (array, factor, offset)
    gives the float64 chain at the layer tolerance, the factors are upper bounds of what they stand for, and a
    negative factor is refused by the library."""
    g = torch.Generator().manual_seed(21)
    x = (torch.randn(3000, 128, generator=g) * 10.0 ** torch.randint(-3, 4, (3000, 1), generator=g).float()).cuda()
    Ws = [(torch.randn(256, 128, generator=g) / 128 ** 0.5).cuda(), (torch.randn(256, 256, generator=g) / 16).cuda(),
          (torch.randn(192, 256, generator=g) / 16).cuda()]
    bs = [torch.randn(256, generator=g).cuda() * 0.1, torch.randn(256, generator=g).cuda() * 0.1, None]
    bound = ops.ScaledBound(ops.row_absmax(x))
    h = x
    for k, (W, b) in enumerate(zip(Ws, bs)):
        l1, bmax = ops.linear_out_bound_factors(W, b)
        assert l1 >= float(W.abs().sum(1).amax()) and bmax >= (float(b.abs().amax()) if b is not None else 0.0)
        h_next = ops.tensor_linear_f16x2(W, h, bound, bias=b, act=ops.ACT_SILU if k < 2 else ops.ACT_NONE)
        assert bool((h_next.abs().amax(1, keepdim=True) <= bound.through(l1, bmax).tensor() * (1 + 1e-6)).all())
        h, bound = h_next, bound.through(l1, bmax)

    def chain(dt):
        t = x.cpu().to(dt)
        for k, (W, b) in enumerate(zip(Ws, bs)):
            t = torch.nn.functional.linear(t, W.cpu().to(dt), None if b is None else b.cpu().to(dt))
            t = torch.nn.functional.silu(t) if k < 2 else t
        return t
    _check(h, chain, "three layers on one array of row maxima")
    assert ops.linear_out_bound_factors(Ws[0], bs[0]) == ops.linear_out_bound_factors(Ws[0], bs[0])
    with torch.no_grad():
        Ws[0].mul_(3.0)
    assert ops.linear_out_bound_factors(Ws[0], bs[0])[0] > 2.9 * l1 * 0 + float(Ws[0].abs().sum(1).amax()) * 0.999
    with pytest.raises(RuntimeError, match="non-negative"):
        ops.tensor_linear_f16x2(Ws[1], h.new_zeros(300, 256), ops.ScaledBound(h.new_ones(300, 1), -1.0, 0.0))


def test_linear_out_bound_is_an_upper_bound(ops):
    g = torch.Generator().manual_seed(5)
    W = torch.randn(96, 64, generator=g).cuda()
    b = torch.randn(96, generator=g).cuda()
    x = torch.randn(500, 64, generator=g).cuda() * 3
    xb = ops.row_absmax(x)
    assert torch.equal(xb[:, 0], x.abs().amax(1))
    yb = ops.linear_out_bound(W, b, xb)
    y = torch.nn.functional.silu(torch.nn.functional.linear(x, W, b))
    assert bool((y.abs().amax(1, keepdim=True) <= yb).all())
    unit = ops.linear_out_bound(W, b, None)                      # inputs bounded by 1
    y1 = torch.nn.functional.linear(torch.rand(100, 64, device="cuda") * 2 - 1, W, b)
    assert unit.shape == (1, 1) and bool((y1.abs().amax() <= unit).all())
    assert ops.linear_out_bound(W, b, None) is unit                # cached per parameter version
    with torch.no_grad():
        W.mul_(2.0)
    assert float(ops.linear_out_bound(W, b, None)) > float(unit)  # recomputed after an in-place update


def test_packed_weight_cache_tracks_in_place_updates(ops):
    prev = ops.get_linear_mode()
    try:
        ops.set_linear_mode(1)
        W = torch.randn(128, 128, device="cuda")
        x = torch.randn(2048, 128, device="cuda")
        y1 = ops.tensor_linear_fwd(0, W, x)
        with torch.no_grad():
            W.mul_(2.0)
        y2 = ops.tensor_linear_fwd(0, W, x)
        torch.testing.assert_close(y2, 2 * y1, rtol=1e-5, atol=1e-5)
    finally:
        ops.set_linear_mode(prev)


def test_weight_written_behind_the_version_counter(pkg, ops):
    """`param.data.mul_()` changes a weight without touching its version counter: the caches cannot see it, and
    ops.invalidate_weight_caches() is the documented remedy (layer caches included)."""
    painn = importlib.import_module("learned-dynamics_amd.painn")
    torch.manual_seed(5)
    upd = painn.Update(64).cuda().eval()
    x_a, x_v = torch.randn(1, 700, 64).cuda(), torch.randn(1, 700, 64, 3).cuda()
    with torch.no_grad():
        upd(x_a, x_v)                                            # fills the caches
        for p in upd.parameters():
            p.data.mul_(1.25)
        ops.invalidate_weight_caches()
        got = upd(x_a, x_v)
        fresh = painn.Update(64).cuda().eval()
        fresh.load_state_dict(upd.state_dict())
        ref = fresh(x_a, x_v)
    for a, b in zip(got, ref):
        torch.testing.assert_close(a, b, rtol=0, atol=0)


def _segment_lengths(kind, n, g):
    if kind == "long":
        return torch.randint(40, 140, (n,), generator=g)
    if kind == "short":
        return torch.randint(0, 9, (n,), generator=g)
    if kind == "aligned":
        return torch.tensor([32, 64, 1, 31, 32, 0, 0, 96, 33, 31] * (n // 10))
    return torch.cat([torch.randint(0, 5, (n // 2,), generator=g), torch.randint(20, 300, (n - n // 2,), generator=g)])[
        torch.randperm(n, generator=g)]


@pytest.mark.parametrize("dim_in,dim_out,act,kind,want_rows", [(512, 512, 2, "long", False), (96, 256, 0, "short", True),
                                                               (256, 256, 1, "aligned", True), (64, 768, 2, "mixed", False)])
def test_linear_with_row_sums_in_the_epilogue(ops, dim_in, dim_out, act, kind, want_rows):
    """out[s] = scale * sum over the rows of segment s of act(x W^T + b), against the plain GEMM followed by
    the segment sum, and against float64; segments placed in every way relative to the kernel's 32-row blocks."""
    g = torch.Generator().manual_seed(dim_in + dim_out)
    n_seg = 300
    lengths = _segment_lengths(kind, n_seg, g)
    seg = torch.repeat_interleave(torch.arange(n_seg), lengths)
    rows = int(seg.numel())
    x = (torch.randn(rows, dim_in, generator=g) * (torch.rand(rows, 1, generator=g) * 3)).cuda()
    W = (torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5).cuda()
    b = torch.randn(dim_out, generator=g).cuda()
    row_ptr = ops.segment_row_ptr(seg.int().cuda(), n_seg)
    bound = ops.row_absmax(x)
    out, y = ops.tensor_linear_f16x2_rowsum(W, x, bound, row_ptr, seg.int().cuda(), n_seg, bias=b, act=act, scale=0.5,
                                            want_rows=want_rows)
    y_ref = ops.tensor_linear_f16x2(W, x, bound, bias=b, act=act)
    if want_rows:
        assert torch.equal(y, y_ref)          # the same accumulators through another epilogue
    else:
        assert y is None
    two_step = 0.5 * ops.segment_sum_csr(y_ref, row_ptr, n_seg)
    def ref(dt):
        z = x.cpu().to(dt) @ W.cpu().to(dt).T + b.cpu().to(dt)
        z = torch.nn.functional.silu(z) if act == 1 else (torch.nn.functional.leaky_relu(z, 0.1) if act == 2 else z)
        return 0.5 * torch.zeros(n_seg, dim_out, dtype=dt).index_add_(0, seg, z)

    _check(out, ref, f"row sums in the epilogue {dim_in}->{dim_out} {kind}")
    _check(two_step, ref, f"GEMM then segment sum {dim_in}->{dim_out} {kind}")
    assert not bool(out[(lengths == 0).cuda()].any())


@pytest.mark.parametrize("inds,rows,dim_in,dim_out", [(2, 8000, 16, 64), (1, 22000, 40, 96), (1, 30000, 64, 256), (1, 25000, 70, 64)])
def test_component_major_output_from_reference_layout_at_many_rows(ops, inds, rows, dim_in, dim_out):
    """x in the reference layout (rows, chan, 3..), y component-major (rows, 3^inds, chan_out): at many rows
    the dispatcher transposes x and uses the plain-row matrix path (K zero-padded to a multiple of 32).
    Against the einsum of extensions/tensor_ops/test.py:9-15 in float64, with accumulate."""
    T = 3 ** inds
    assert rows * T >= 65536
    g = torch.Generator().manual_seed(rows)
    x = torch.randn(rows, dim_in, *([3] * inds), generator=g).cuda()
    W = (torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5).cuda()
    y = ops.tensor_linear_fwd(inds, W, x, y_layout=ops.LAYOUT_COMP_CHAN)
    ref = lambda dt: torch.einsum("oi,bit->bto", W.cpu().to(dt), x.cpu().to(dt).reshape(rows, dim_in, T))
    assert y.shape == (rows, T, dim_out)
    _check(y, ref, f"component-major output, {rows} rows")
    y2 = ops.tensor_linear_fwd(inds, W, x, y_layout=ops.LAYOUT_COMP_CHAN, out=y.clone(), accumulate=True)
    _check(y2, lambda dt: y.cpu().to(dt) + ref(dt), f"component-major output, accumulate, {rows} rows")
    # the generic kernel, which serves fewer rows, on the first rows
    small = ops.tensor_linear_fwd(inds, W, x[:500].contiguous(), y_layout=ops.LAYOUT_COMP_CHAN)
    _check(small, lambda dt: ref(dt)[:500], "component-major output, generic kernel")


def test_linear_with_row_sums_edge_cases(ops):
    W = torch.randn(256, 64).cuda()
    row_ptr = torch.zeros(11, dtype=torch.int32, device="cuda")
    seg = torch.empty(0, dtype=torch.int32, device="cuda")
    out, y = ops.tensor_linear_f16x2_rowsum(W, torch.empty(0, 64, device="cuda"), torch.ones(1, 1, device="cuda"), row_ptr, seg,
                                            10, want_rows=True)
    assert out.shape == (10, 256) and not bool(out.any()) and y.shape == (0, 256)
    # one segment holding every row, fewer rows than a tile
    x = torch.randn(77, 64).cuda()
    seg = torch.zeros(77, dtype=torch.int32, device="cuda")
    row_ptr = torch.tensor([0, 77], dtype=torch.int32, device="cuda")
    out, _ = ops.tensor_linear_f16x2_rowsum(W, x, ops.row_absmax(x), row_ptr, seg, 1)
    _check(out, lambda dt: (x.cpu().to(dt) @ W.cpu().to(dt).T).sum(0, keepdim=True), "one segment of 77 rows")
    with pytest.raises(RuntimeError, match="multiple of 256"):
        ops.tensor_linear_f16x2_rowsum(W[:128].contiguous(), x, ops.row_absmax(x), row_ptr, seg, 1)


@pytest.mark.parametrize("inds", [0, 1, 2])
def test_plain_entry_point_through_ctypes(pkg, inds):
    """mg_tensor_linear called as a foreign caller would (raw pointers, element strides of W, the current stream):
    the transposed view of W, bias + SiLU for inds = 0, accumulation into y, and zero rows."""
    import ctypes
    L = importlib.import_module("learned-dynamics_amd._lib")
    lib = L.load()
    g = torch.Generator().manual_seed(40 + inds)
    Wt = torch.randn(48, 96, generator=g)                      # stored (dim_in, dim_out): W = Wt.t()
    x = torch.randn(33, 48, *([3] * inds), generator=g)
    bias = torch.randn(96, generator=g) if inds == 0 else None
    y0 = torch.randn(33, 96, *([3] * inds), generator=g)
    Wd, xd, yd = Wt.cuda(), x.cuda(), y0.cuda()
    bd = bias.cuda() if bias is not None else None
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    act = 1 if inds == 0 else 0
    L.check(lib.mg_tensor_linear(inds, Wd.data_ptr(), Wd.stride(1), Wd.stride(0), xd.data_ptr(), 33, 48, 96,
                                 bd.data_ptr() if bd is not None else None, act, 0, yd.data_ptr(), st))
    def ref(dt):
        lin = OP.tensor_linear(inds, Wt.t().to(dt), x.to(dt))
        return torch.nn.functional.silu(lin + bias.to(dt)) if inds == 0 else lin

    _check(yd, ref)
    L.check(lib.mg_tensor_linear(inds, Wd.data_ptr(), Wd.stride(1), Wd.stride(0), xd.data_ptr(), 33, 48, 96,
                                 None, 0, 1, yd.data_ptr(), st))
    _check(yd, lambda dt: ref(dt) + OP.tensor_linear(inds, Wt.t().to(dt), x.to(dt)))
    before = yd.clone()
    L.check(lib.mg_tensor_linear(inds, Wd.data_ptr(), Wd.stride(1), Wd.stride(0), xd.data_ptr(), 0, 48, 96,
                                 None, 0, 0, yd.data_ptr(), st))
    assert torch.equal(yd, before)


@pytest.mark.parametrize("span", [1e4, 1e6])
def test_linear_f16x2_in_row_dynamic_range_meeting_zero_weights(ops, span):
    """Inside ONE row: a few entries `span` times larger than the rest, and weights that are exactly zero on those
    entries, so the result is made of the small entries alone.  The row scale puts the row maximum M at 2^14..2^15
    and every entry is carried by two fp16 pieces with an absolute error of at most 2^-25 in scaled units, i.e.
    2^-39 M per term whatever the term's own size: the error bound is relative to the ROW, not to the term.
      span 1e4: the small terms still carry about 2^-26 relative error each: the rel 1e-5 / abs 1e-6 contract holds
                on the result itself;
      span 1e6: the bound 2^-39 M |w| sqrt(K) is about 1e-5 of a result of order one: the edge of the contract, and
                what this test pins is that bound (rows of the models carry activations and products of order one,
                their in-row spans stay far below 1e4)."""
    g = torch.Generator().manual_seed(int(span) % 97)
    rows, dim_in, dim_out = 4096, 512, 256
    x = torch.randn(rows, dim_in, generator=g)
    big = torch.zeros(dim_in, dtype=torch.bool)
    big[::37] = True
    x[:, big] *= span
    W = torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5
    W[:, big] = 0.0
    ref = x.double() @ W.double().t()
    y = ops.tensor_linear_f16x2(W.cuda(), x.cuda())
    small = x.clone()
    small[:, big] = 0.0
    ref32 = (small @ W.t()).double()                          # fp32 evaluation of the same sum (the zeros drop out exactly)
    e_ref = float((ref32 - ref).abs().max())
    err = (y.cpu().double() - ref).abs()
    contract = 1e-6 + 1e-5 * ref.abs() + 2 * e_ref            # the tolerance on the result, as everywhere else
    row_scale = (3 * 2.0 ** -39 * dim_in ** 0.5) * x.abs().amax(1, keepdim=True).double() * W.abs().amax(1).double()
    print(f"[f16x2 in-row span {span:g}] max err {float(err.max()):.3g}  e_ref {e_ref:.3g}  max row-scale bound "
          f"{float(row_scale.max()):.3g}  |ref| max {float(ref.abs().max()):.3g}")
    if span <= 1e4:
        assert bool((err <= contract).all()), (float(err.max()), e_ref)
    else:
        assert bool((err <= contract + row_scale).all()), (float(err.max()), e_ref)
        assert float(err.max()) < 3e-5 * float(ref.abs().max())


@pytest.mark.parametrize("inds,rows,dim_in,dim_out", [(0, 5000, 117, 210), (0, 70, 16, 512), (0, 1, 33, 31),
                                                      (0, 100003, 512, 384), (1, 3000, 48, 70), (2, 900, 20, 130),
                                                      (1, 300, 48, 70), (2, 100, 20, 130), (1, 8192, 64, 256),
                                                      (2, 4001, 16, 16), (1, 2000, 300, 64)])
def test_weight_gradient_against_float64(ops, inds, rows, dim_in, dim_out):
    """dW[o, i] = sum over rows and components of dy[r, o, t] x[r, i, t]: plain rows through the matrix cores (fp32
    ones where a dimension is not a multiple of 4 or the rows are few, else split fp16; tiles of 128 x 128 with ragged
    edges, row slices that do not divide the rows), tensor components transposed to plain rows for the matrix cores
    when there are at least 4096 of them and the channels fit 256, else through the vector kernel; slices are summed
    in a fixed order, so two runs agree bit for bit."""
    g = torch.Generator().manual_seed(rows + dim_in)
    comps = (3,) * inds
    x = torch.randn(rows, dim_in, *comps, generator=g).cuda()
    dy = torch.randn(rows, dim_out, *comps, generator=g).cuda()
    got = ops.tensor_linear_wgrad(inds, dy, x)
    want = torch.einsum("ro...,ri...->oi", dy.double(), x.double())
    fp32 = torch.einsum("ro...,ri...->oi", dy, x).double()
    scale = float(want.abs().max())
    err, err_ref = float((got.double() - want).abs().max()), float((fp32 - want).abs().max())
    assert err <= 1e-6 + 1e-5 * scale + 2 * err_ref, (err, err_ref, scale)
    assert torch.equal(ops.tensor_linear_wgrad(inds, dy, x), got)


@pytest.mark.parametrize("rows,dim_in,dim_out", [(4096, 64, 64), (5000, 68, 132), (40001, 512, 512), (33333, 128, 512),
                                                 (9000, 260, 64), (20011, 16, 512), (4100, 4, 8)])
@pytest.mark.parametrize("bounds", ["scanned", "row maxima", "loose"])
def test_weight_gradient_split_fp16(ops, rows, dim_in, dim_out, bounds):
    """Plain rows on the fp16 matrix cores with hi + lo operands: tiles with ragged edges, row slices that do not
    divide the rows, rows whose magnitudes span 2^12, the scales taken from the operands themselves, from row maxima
    or from a bound 1000 times too large; to the tolerance of the fp32 kernels, and the same bits on every run."""
    g = torch.Generator().manual_seed(rows + 3 * dim_in + dim_out)
    spread = torch.exp2(torch.randint(-12, 1, (rows, 1), generator=g).float())
    x = (torch.randn(rows, dim_in, generator=g) * spread).cuda()
    dy = (torch.randn(rows, dim_out, generator=g) * spread.flip(0) * 37.0).cuda()
    assert ops.get_linear_mode() == ops.LINEAR_F16X2
    kw = {}
    if bounds == "row maxima":
        kw = dict(dy_bound=ops.row_absmax(dy), x_bound=ops.row_absmax(x))
    elif bounds == "loose":
        kw = dict(dy_bound=dy.abs().max().reshape(1) * 1000.0, x_bound=x.abs().max().reshape(1) * 1000.0)
    got, got_b = ops.tensor_linear_wgrad(0, dy, x, want_bias=True, **kw)
    want_b = dy.double().sum(0)
    err_b, ref_b = float((got_b.double() - want_b).abs().max()), float((dy.sum(0).double() - want_b).abs().max())
    assert err_b <= 1e-6 + 1e-5 * float(want_b.abs().max()) + 2 * ref_b, (err_b, ref_b)
    want = dy.double().t() @ x.double()
    fp32 = (dy.t() @ x).double()
    scale = float(want.abs().max())
    err, err_ref = float((got.double() - want).abs().max()), float((fp32 - want).abs().max())
    print(f"[wgrad f16x2 {rows}x{dim_in}x{dim_out} {bounds}] err {err:.3g} fp32 err {err_ref:.3g} scale {scale:.3g}")
    assert err <= 1e-6 + 1e-5 * scale + 2 * err_ref, (err, err_ref, scale)
    assert torch.equal(ops.tensor_linear_wgrad(0, dy, x, **kw), got)
    # the fp32 matrix-core kernel on the same operands
    ops.set_linear_mode(ops.LINEAR_FP32_MFMA)
    try:
        plain = ops.tensor_linear_wgrad(0, dy, x)
    finally:
        ops.set_linear_mode(ops.LINEAR_F16X2)
    assert float((plain.double() - want).abs().max()) <= 1e-6 + 1e-5 * scale + 2 * err_ref
    assert not torch.equal(plain, got)          # (another kernel, another summation order)


def test_weight_gradient_at_the_edge_count_of_configs2(ops):
    """The split-fp16 weight gradient at the size training runs it at (1592454 edge rows, 512 x 512): against float64
    accumulated over row chunks on the device, with the error of torch's own fp32 product of the same operands as
    the yardstick; the bias gradient from the same pass; and the same bits on a second run."""
    rows, dim = 1592454, 512
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(rows, dim, device="cuda", generator=g)
    dy = torch.randn(rows, dim, device="cuda", generator=g) * torch.rand(rows, 1, device="cuda", generator=g)
    got, got_b = ops.tensor_linear_wgrad(0, dy, x, want_bias=True)
    want = torch.zeros(dim, dim, dtype=torch.float64, device="cuda")
    want_b = torch.zeros(dim, dtype=torch.float64, device="cuda")
    fp32 = torch.zeros(dim, dim, dtype=torch.float64, device="cuda")
    for lo in range(0, rows, 65536):
        a, b = dy[lo:lo + 65536], x[lo:lo + 65536]
        want += a.double().t() @ b.double()
        want_b += a.double().sum(0)
        fp32 += (a.t() @ b).double()
    scale = float(want.abs().max())
    err, err_ref = float((got.double() - want).abs().max()), float((fp32 - want).abs().max())
    print(f"[wgrad f16x2 {rows}x{dim}x{dim}] err {err:.3g}  chunked fp32 err {err_ref:.3g}  scale {scale:.3g}")
    assert err <= 1e-6 + 1e-5 * scale + 2 * err_ref, (err, err_ref, scale)
    assert float((got_b.double() - want_b).abs().max()) <= 1e-6 + 1e-5 * float(want_b.abs().max())
    again, again_b = ops.tensor_linear_wgrad(0, dy, x, want_bias=True)
    assert torch.equal(again, got) and torch.equal(again_b, got_b)

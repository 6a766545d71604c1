"""The PyTorch C++ binding (learned-dynamics_amd/csrc/torch_binding.cpp, built as managan_torch_ext.so): the functions
the reference exports from neighbour_grid_cuda, tensor_ops_cuda and codegen_tensops_cuda, with at::Tensor arguments.
Same kernels as the ctypes route, so results are compared bit for bit with it, tensor_linear (which the binding sends
to the fp32 matrix-core kernel) and its derivatives against the oracle; error texts as the reference's front ends."""
import importlib
import time

import numpy as np
import pytest
import torch

from oracle import neighbour as ON
from oracle import products as OP
from parity import assert_parity_of

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    return importlib.import_module("learned-dynamics_amd._lib").load_torch_ext()


def test_neighbour_functions_equal_the_ctypes_route_and_the_oracle(ext, ops):
    rng = np.random.default_rng(3)
    x = (rng.random((2, 900, 3)) * 30).astype(np.float32)
    xt = torch.from_numpy(x).cuda()
    src, dst, counts = ext.get_edges(64, 256, 6.0, 30.0, 30.0, 30.0, xt)
    s2, d2, c2 = ops.get_edges(64, 256, 6.0, 30.0, 30.0, 30.0, xt)
    assert src.dtype == torch.int32 and torch.equal(src, s2) and torch.equal(dst, d2) and torch.equal(counts, c2)
    ref = ON.edges(x, 6.0, (30.0, 30.0, 30.0))
    assert np.array_equal(ON.sorted_triples(src.cpu().numpy(), dst.cpu().numpy()), ON.sorted_triples(ref["src"], ref["dst"]))
    nb, cnt = ext.get_neighbours(64, 256, 6.0, 30.0, 30.0, 30.0, xt)
    nb2, cnt2 = ops.get_neighbours(64, 256, 6.0, 30.0, 30.0, 30.0, xt)
    assert torch.equal(cnt, cnt2)
    valid = torch.arange(256, device="cuda")[None, None, :] < cnt[..., None]
    assert torch.equal(nb[valid], nb2[valid])
    feat = torch.randn(2, 900, 7, device="cuda")
    on_edges = ext.edges_read(cnt, nb, feat)
    assert torch.equal(on_edges, ops.padded_edges_read(cnt, nb, feat))
    assert torch.equal(ext.edges_reduce(cnt, nb, on_edges), ops.padded_edges_reduce(cnt, nb, on_edges))
    # the reference's errors
    with pytest.raises(RuntimeError, match="Neighbour list overflow occurred. Try increasing neighboursmax."):
        ext.get_edges(64, 8, 6.0, 30.0, 30.0, 30.0, xt)
    with pytest.raises(RuntimeError, match="Cell list overflow occurred"):
        ext.get_edges(32, 256, 6.0, 30.0, 30.0, 30.0, torch.zeros(1, 100, 3, device="cuda"))
    with pytest.raises(RuntimeError, match="3\\*cutoff"):
        ext.get_edges(64, 256, 6.0, 12.0, 30.0, 30.0, xt)
    with pytest.raises(RuntimeError, match="x must be a CUDA tensor"):
        ext.get_edges(64, 256, 6.0, 30.0, 30.0, 30.0, xt.cpu())
    with pytest.raises(RuntimeError, match="x must be contiguous"):
        ext.get_edges(64, 256, 6.0, 30.0, 30.0, 30.0, xt[:, ::2])
    empty = ext.get_edges(64, 256, 6.0, 30.0, 30.0, 30.0, torch.zeros(0, 10, 3, device="cuda"))
    assert empty[0].numel() == 0 and empty[2].numel() == 0


@pytest.mark.parametrize("inds", [0, 1, 2])
def test_tensor_linear_and_its_derivatives(ext, inds):
    g = torch.Generator().manual_seed(20 + inds)
    W = torch.randn(40, 24, generator=g) / 24 ** 0.5
    x = torch.randn(5, 13, 24, *([3] * inds), generator=g)
    cot = torch.randn(5, 13, 40, *([3] * inds), generator=g)
    y = ext.tensor_linear(inds, W.cuda(), x.cuda())
    assert_parity_of(y, lambda dt: OP.tensor_linear(inds, W.to(dt), x.to(dt)), f"binding tensor_linear rank {inds}")
    # a transposed view of W costs nothing
    yt = ext.tensor_linear(inds, W.t().contiguous().cuda().t(), x.cuda())
    assert_parity_of(yt, lambda dt: OP.tensor_linear(inds, W.to(dt), x.to(dt)), "transposed weight")
    # first derivatives and the gradient of a gradient norm against autograd through the oracle in float64
    Wd, xd = W.double().requires_grad_(), x.double().requires_grad_()
    ref = torch.autograd.grad((OP.tensor_linear(inds, Wd, xd) * cot.double()).sum(), [Wd, xd], create_graph=True)
    ref2 = torch.autograd.grad(sum((r ** 2).sum() for r in ref), [Wd, xd])
    Wg, xg = W.cuda().requires_grad_(), x.cuda().requires_grad_()
    got = torch.autograd.grad((ext.tensor_linear(inds, Wg, xg) * cot.cuda()).sum(), [Wg, xg], create_graph=True)
    got2 = torch.autograd.grad(sum((t ** 2).sum() for t in got), [Wg, xg])
    for a, r in zip(list(got) + list(got2), list(ref) + list(ref2)):
        torch.testing.assert_close(a.detach().cpu().double(), r.detach(), rtol=1e-5, atol=2e-6 * float(r.abs().max()) + 1e-9)
    assert tuple(ext.tensor_linear(inds, W.cuda(), x[:0].cuda()).shape) == (0, 13, 40) + (3,) * inds
    with pytest.raises(RuntimeError, match="channel dim size mismatch for x"):
        ext.tensor_linear(0, W.cuda(), torch.randn(3, 5, device="cuda"))
    with pytest.raises(RuntimeError, match="up to 2"):
        ext.tensor_linear(3, W.cuda(), torch.randn(2, 24, 3, 3, 3, device="cuda"))
    with pytest.raises(RuntimeError, match="x must be contiguous"):
        ext.tensor_linear(0, W.cuda(), torch.randn(24, 3, device="cuda").t())


def test_bee_and_cow_equal_the_ctypes_route(ext, ops):
    g = torch.Generator().manual_seed(9)
    rows, chan = 77, 33
    l = [torch.randn(rows, chan, *([3] * k), generator=g).cuda() for k in range(3)]
    r = [torch.randn(rows, chan, *([3] * k), generator=g).cuda() for k in range(3)]
    ys = ext.bee_fwd_cuda(*l, *r)
    for a, b in zip(ys, ops.bee_fwd(*l, *r)):
        assert torch.equal(a, b)
    dys = [torch.randn_like(y) for y in ys]
    for a, b in zip(ext.bee_bwl_cuda(*r, *dys) + ext.bee_bwr_cuda(*l, *dys), ops.bee_bwl(*r, *dys) + ops.bee_bwr(*l, *dys)):
        assert torch.equal(a, b)
    for which, fwd, bwl, bwr in ((0, "cow_o0_fwd", "cow_o0_bwl", "cow_o0_bwr"), (1, "cow_o1_fwd", "cow_o1_bwl", "cow_o1_bwr")):
        out = getattr(ext, fwd + "_cuda")(l[0], l[1], r[0], r[1])
        for a, b in zip(out, getattr(ops, fwd)(l[0], l[1], r[0], r[1])):
            assert torch.equal(a, b)
        dy = [torch.randn_like(t) for t in out]
        for a, b in zip(getattr(ext, bwl + "_cuda")(r[0], r[1], *dy) + getattr(ext, bwr + "_cuda")(l[0], l[1], *dy),
                        getattr(ops, bwl)(r[0], r[1], *dy) + getattr(ops, bwr)(l[0], l[1], *dy)):
            assert torch.equal(a, b)
    with pytest.raises(RuntimeError, match="expected 13 output gradients"):
        ext.bee_bwl_cuda(*r, *dys[:12])
    with pytest.raises(RuntimeError, match="r_1 has wrong number of axes"):
        ext.bee_fwd_cuda(*l, r[0], r[0], r[2])
    with pytest.raises(RuntimeError, match="left and right operands must agree"):
        ext.bee_fwd_cuda(*l, *[t[:5].contiguous() for t in r])


def test_shims_are_the_binding_and_its_calls_cost_less_host_time(ext, pkg, ops):
    pkg.install_shims()
    import codegen_tensops_cuda
    import neighbour_grid_cuda
    import tensor_ops_cuda
    assert neighbour_grid_cuda.get_edges is ext.get_edges and codegen_tensops_cuda.bee_fwd_cuda is ext.bee_fwd_cuda
    W, x = torch.randn(64, 64, device="cuda"), torch.randn(256, 64, device="cuda")
    assert torch.equal(tensor_ops_cuda.tensor_linear(0, W, x), ext.tensor_linear(0, W, x))
    big = torch.randn(70000, 64, device="cuda")                        # the large-problem route: the Python operator
    assert_parity_of(tensor_ops_cuda.tensor_linear(0, W, big), lambda dt: big.cpu().to(dt) @ W.cpu().to(dt).T, "large route")

    def host_us(fn, n=300):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        dt = time.perf_counter() - t0                                  # issue time: the queue is never waited for
        torch.cuda.synchronize()
        return dt / n * 1e6

    with torch.no_grad():
        t_ext = host_us(lambda: ext.tensor_linear(0, W, x))
        t_py = host_us(lambda: ops.tensor_linear_fwd(0, W, x))
    print(f"[host time per call] tensor_linear 256 x 64 -> 64: binding {t_ext:.1f} us, ctypes route {t_py:.1f} us")
    assert t_ext < t_py


@pytest.mark.parametrize("inds", [(1, 1, 0), (0, 1, 1), (1, 1, 2), (2, 1, 1), (2, 2, 0)])
def test_tensor_prods_equals_the_ctypes_route_and_the_module_uses_it(ext, ops, inds):
    tp = importlib.import_module("learned-dynamics_amd.tensor_products")
    g = torch.Generator().manual_seed(77)
    mod = tp.TensorProds(*inds, 64, 64, 64, 64).cuda()
    lead = (3, 37)
    x_l = torch.randn(*lead, 64, *([3] * inds[0]), generator=g).cuda()
    x_r = torch.randn(*lead, 64, *([3] * inds[1]), generator=g).cuda()
    W_l, W_r, W_o = mod.lin_l.W.detach(), mod.lin_r.W.detach(), mod.lin_o.W.detach()
    assert ext.tensor_prods_supported(*inds, 64, 64, 64, 64) == ops.tensor_prods_supported(*inds, 64, 64, 64, 64)
    if not ext.tensor_prods_supported(*inds, 64, 64, 64, 64):
        pytest.skip("not a one-launch problem")
    y = ext.tensor_prods(*inds, W_l, W_r, W_o, x_l, x_r)
    assert y.shape == (*lead, 64, *([3] * inds[2]))
    assert torch.equal(y, ops.tensor_prods(*inds, W_l, W_r, W_o, x_l, x_r))
    with torch.no_grad():
        assert torch.equal(mod(x_l, x_r), y)
    # a weight that is a view with padded rows goes in as it is; one with a non-unit inner stride is copied
    wide = torch.zeros(64, 68, device="cuda")
    wide[:, :64] = W_l
    assert torch.equal(ext.tensor_prods(*inds, wide[:, :64], W_r, W_o, x_l, x_r), y)
    assert torch.equal(ext.tensor_prods(*inds, W_l.t().contiguous().t(), W_r, W_o, x_l, x_r), y)
    with pytest.raises(RuntimeError, match="shape mismatch"):
        ext.tensor_prods(*inds, W_l[:, :32], W_r, W_o, x_l, x_r)
    with pytest.raises(RuntimeError, match="do not broadcast"):
        ext.tensor_prods(*inds, W_l, W_r, W_o, x_l[:2], x_r)
    with pytest.raises(RuntimeError, match="float32 CUDA"):
        ext.tensor_prods(*inds, W_l, W_r, W_o, x_l.cpu(), x_r)

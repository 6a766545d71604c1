"""Gather / segment-sum kernels and the Graph helpers against the oracle."""
import importlib

import numpy as np
import pytest
import torch

from conftest import load_golden
from oracle import layers as OL

pytestmark = pytest.mark.gpu


def _random_sorted_index(n_rows, n_edges, seed, empty_rows=True):
    g = torch.Generator().manual_seed(seed)
    idx = torch.randint(0, n_rows, (n_edges,), generator=g)
    if empty_rows and n_rows > 4:
        idx[idx == 2] = 3
        idx[idx == n_rows - 1] = 0
    return torch.sort(idx).values


@pytest.mark.parametrize("feat_shape", [(), (1,), (4,), (3,), (128,), (128, 3), (64, 3, 3), (20, 3), (5,), (260,), (1030,)])
def test_segment_sum(ops, feat_shape):
    n_rows, n_edges = 300, 5000
    idx = _random_sorted_index(n_rows, n_edges, 1)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(n_edges, *feat_shape, generator=g)
    for dtype in (torch.int64, torch.int32):
        row_ptr = ops.segment_row_ptr(idx.to(dtype).cuda(), n_rows)
        counts = torch.bincount(idx, minlength=n_rows)
        assert torch.equal(torch.diff(row_ptr.cpu()).long(), counts)
    out = ops.segment_sum_csr(x.cuda(), row_ptr, n_rows)
    ref = torch.zeros(n_rows, *feat_shape).index_add_(0, idx, x)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5)


def test_segment_sum_long_rows(ops):
    idx = torch.cat([torch.zeros(3000, dtype=torch.long), torch.full((1,), 5), torch.full((2000,), 9)])
    x = torch.randn(idx.numel(), 384, generator=torch.Generator().manual_seed(3))
    row_ptr = ops.segment_row_ptr(idx.cuda(), 12)
    out = ops.segment_sum_csr(x.cuda(), row_ptr, 12)
    ref = torch.zeros(12, 384).index_add_(0, idx, x)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=2e-4)


@pytest.mark.parametrize("feat_shape", [(), (4,), (3,), (128, 3), (5,), (512,)])
def test_segment_sum_through_a_permutation(ops, feat_shape):
    """An unsorted index: rows summed in its stable sorted order through the permutation, bit for bit what gathering
    the rows into that order and summing them gives (the adjoint of edges_read_dst)."""
    n_rows, n_edges = 300, 5000
    g = torch.Generator().manual_seed(11)
    idx = torch.randint(0, n_rows, (n_edges,), generator=g)
    idx[idx == 7] = 8
    x = torch.randn(n_edges, *feat_shape, generator=g).cuda()
    perm = torch.sort(idx, stable=True).indices
    row_ptr = ops.segment_row_ptr(idx[perm].cuda(), n_rows)
    out = ops.segment_sum_csr(x, row_ptr, n_rows, perm=perm.to(torch.int32).cuda())
    two_step = ops.segment_sum_csr(ops.gather_rows(x, perm.cuda()), row_ptr, n_rows)
    assert torch.equal(out, two_step)
    ref = torch.zeros(n_rows, *feat_shape, dtype=torch.float64).index_add_(0, idx, x.cpu().double())
    torch.testing.assert_close(out.cpu().double(), ref, rtol=1e-5, atol=1e-5)


def test_segment_edge_cases(ops):
    row_ptr = ops.segment_row_ptr(torch.empty(0, dtype=torch.int64).cuda(), 7)
    assert row_ptr.tolist() == [0] * 8
    out = ops.segment_sum_csr(torch.empty(0, 5).cuda(), row_ptr, 7)
    assert torch.all(out == 0) and tuple(out.shape) == (7, 5)


@pytest.mark.parametrize("feat_shape", [(), (3,), (128,), (128, 3), (16, 3, 3), (7,)])
def test_gather(ops, feat_shape):
    g = torch.Generator().manual_seed(4)
    x = torch.randn(500, *feat_shape, generator=g)
    idx = torch.randint(0, 500, (3000,), generator=g)
    for dtype in (torch.int64, torch.int32):
        out = ops.gather_rows(x.cuda(), idx.to(dtype).cuda())
        assert torch.equal(out.cpu(), x[idx])


def test_graph_layers_golden(pkg):
    """The reference's self test (managan/graph_layers.py:80-122): degrees, the sum-of-products
    matrix 'calculated on paper', and the wrap bound."""
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    five = load_golden("graph_layers_five_points")
    box = tuple(five["box"])
    positions = torch.tensor(five["positions"], device="cuda")
    graph = gl.Graph.radius_graph(five["radius"], box, positions)
    assert torch.all(graph.src[1:] >= graph.src[:-1])
    assert graph.src.dtype == torch.int64 and graph.dst.dtype == torch.int64
    ones = torch.ones_like(graph.dst, dtype=torch.float)
    degrees = gl.edges_reduce_src(graph, ones)
    assert torch.allclose(degrees, torch.tensor(five["degrees"], device="cuda", dtype=torch.float))
    x = torch.arange(5, device="cuda").to(torch.float).repeat(4).reshape(1, 5, 4)
    s, d = gl.edges_read(graph, x)
    sumprod = gl.edges_reduce_src(graph, s * d)
    assert torch.allclose(sumprod, torch.tensor(five["sum_of_products"], device="cuda"))
    pos_src, pos_dst = gl.edges_read(graph, positions)
    delta = gl.boxwrap(torch.tensor(box, device="cuda"), pos_dst - pos_src)
    assert torch.all((delta ** 2).sum(-1) < five["wrapped_length_bound"] ** 2)
    assert torch.equal(delta, gl.edge_vectors(graph, positions, box))


def test_torch_scatter_shim(pkg):
    pkg.install_shims()
    from torch_scatter import segment_coo
    idx = _random_sorted_index(50, 700, 5).cuda()
    x = torch.randn(700, 16, 3, device="cuda")
    out = segment_coo(x, idx, dim_size=50)
    ref = torch.zeros(50, 16, 3).index_add_(0, idx.cpu(), x.cpu())
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5)


def test_gather_and_segment_sum_are_differentiable(pkg):
    """edges_read / edges_read_dst / edges_reduce_src against torch indexing and index_add_ under
    autograd, including a second derivative (the meanflow loss differentiates a jvp:
    archs/meanflow_painn8.py:274-282)."""
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    g = torch.Generator().manual_seed(11)
    B, N, E, C = 2, 40, 700, 6
    src = torch.sort(torch.randint(0, B * N, (E,), generator=g)).values
    dst = torch.randint(0, B * N, (E,), generator=g)
    graph = gl.Graph(src.cuda(), dst.cuda(), None, B, N)
    x = torch.randn(B, N, C, 3, generator=g)
    w_e = torch.randn(E, C, 3, generator=g)

    def model(x_node, gather_src_dst, reduce):
        xs, xd = gather_src_dst(x_node)
        m = xs * xd * w_e.to(x_node.device) + xd ** 3          # nonlinear in the gathered rows
        return (reduce(m) ** 2).sum()

    def ref_gather(x_node):
        flat = x_node.reshape(B * N, C, 3)
        return flat[src], flat[dst]

    def ref_reduce(m):
        return torch.zeros(B * N, C, 3, dtype=m.dtype).index_add_(0, src, m).reshape(B, N, C, 3)

    xr = x.clone().requires_grad_(True)
    loss_r = model(xr, ref_gather, ref_reduce)
    (gr,) = torch.autograd.grad(loss_r, xr, create_graph=True)
    (ggr,) = torch.autograd.grad((gr ** 2).sum(), xr)

    xg = x.cuda().requires_grad_(True)
    loss_g = model(xg, lambda t: gl.edges_read(graph, t), lambda m: gl.edges_reduce_src(graph, m))
    (gg,) = torch.autograd.grad(loss_g, xg, create_graph=True)
    (ggg,) = torch.autograd.grad((gg ** 2).sum(), xg)
    torch.testing.assert_close(loss_g.cpu(), loss_r, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(gg.detach().cpu(), gr.detach(), rtol=1e-4, atol=1e-4 * float(gr.detach().abs().max()))
    torch.testing.assert_close(ggg.cpu(), ggr, rtol=1e-4, atol=1e-4 * float(ggr.abs().max()))
    # the torch_scatter shim carries the same autograd
    pkg.install_shims()
    import torch_scatter
    e = torch.randn(E, 5, generator=g).cuda().requires_grad_(True)
    out = torch_scatter.segment_coo(e, src.cuda(), dim_size=B * N, reduce="sum")
    out.square().sum().backward()
    ref_e = torch.zeros(B * N, 5).index_add_(0, src, e.detach().cpu())
    torch.testing.assert_close(e.grad.cpu(), 2 * ref_e[src], rtol=1e-5, atol=1e-5)

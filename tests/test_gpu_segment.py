"""Gather / segment-sum kernels and the Graph helpers against the oracle."""
import importlib

import numpy as np
import pytest
import torch

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
    positions = torch.tensor([[[0., 0., -1.], [1., 0., 0.], [3., 0., 0.], [2., 1., 0.], [8., 0., 0.]]], device="cuda")
    graph = gl.Graph.radius_graph(2., (100., 100., 100.), positions)
    assert torch.all(graph.src[1:] >= graph.src[:-1])
    assert graph.src.dtype == torch.int64 and graph.dst.dtype == torch.int64
    ones = torch.ones_like(graph.dst, dtype=torch.float)
    degrees = gl.edges_reduce_src(graph, ones)
    assert torch.allclose(degrees, torch.tensor([[1., 3., 2., 2., 0.]], device="cuda"))
    x = torch.arange(5, device="cuda").to(torch.float).repeat(4).reshape(1, 5, 4)
    s, d = gl.edges_read(graph, x)
    sumprod = gl.edges_reduce_src(graph, s * d)
    expected = torch.tensor([[0., 0., 2., 6.], [20., 0., 6., 8.], [18., 12., 0., 2.], [14., 12., 4., 0.],
                             [0., 0., 0., 0.]], device="cuda")[None]
    assert torch.allclose(sumprod, expected)
    pos_src, pos_dst = gl.edges_read(graph, positions)
    delta = gl.boxwrap(torch.tensor((100., 100., 100.), device="cuda"), pos_dst - pos_src)
    assert torch.all((delta ** 2).sum(-1) < 2.001 ** 2)
    assert torch.equal(delta, gl.edge_vectors(graph, positions, (100., 100., 100.)))


def test_torch_scatter_shim(pkg):
    pkg.install_shims()
    from torch_scatter import segment_coo
    idx = _random_sorted_index(50, 700, 5).cuda()
    x = torch.randn(700, 16, 3, device="cuda")
    out = segment_coo(x, idx, dim_size=50)
    ref = torch.zeros(50, 16, 3).index_add_(0, idx.cpu(), x.cpu())
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5)

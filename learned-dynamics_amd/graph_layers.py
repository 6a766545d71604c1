"""Graph container and the gather / segment-sum / boxwrap helpers, mirroring
managan/graph_layers.py of the reference (same names, arguments and error
behaviour) on top of the HIP kernels.

Differences that do not change results: the Graph also keeps the int32 index
arrays and the CSR row_ptr the neighbour search produced, so gathers and
segment sums run on them directly; rows are exact-size (the celllist_max /
neighbours_max caps are only used to raise the reference's overflow errors).

Gathers and segment sums are differentiable (each is the other's adjoint, and the
adjoints are expressed with the same two autograd functions, so second derivatives
as taken by torch.autograd.functional.jvp(create_graph=True) work too).
"""
import torch

from . import ops


class Graph:
    """Batch of graphs with the same number of nodes each; edges are stored flat
    and index into a dimension of size batch*nodes.  src must be non-decreasing.
    (managan/graph_layers.py:9-24)"""

    def __init__(self, src, dst, edge_indices, batch, nodes, row_ptr=None, cell_order=None):
        self.src32 = src.to(torch.int32).contiguous()
        self.dst32 = dst.to(torch.int32).contiguous()
        self.src = src.to(torch.int64)
        self.dst = dst.to(torch.int64)
        self.edge_indices = edge_indices
        self.batch = batch
        self.nodes = nodes
        self._row_ptr = row_ptr
        self.cell_order = cell_order   # int32 atom ids in cell order, or None (radius graphs only)
        self._by_src = None
        self._by_dst = None

    @property
    def by_src(self):
        if self._by_src is None:
            self._by_src = _SortedIndex(self.src32, self.batch * self.nodes, row_ptr=self.row_ptr, is_sorted=True)
        return self._by_src

    @property
    def by_dst(self):
        if self._by_dst is None:
            self._by_dst = _SortedIndex(self.dst32, self.batch * self.nodes)
        return self._by_dst

    @property
    def row_ptr(self):
        if self._row_ptr is None:
            self._row_ptr = ops.segment_row_ptr(self.src32, self.batch * self.nodes)
        return self._row_ptr

    @property
    def degree(self):
        """Edges per node as a float32 column (nodes, 1): what a per-edge bias sums to.  Formed once per graph, except
        for a capacity-sized graph, whose row pointer is rewritten in place by every search of a captured rollout."""
        rp = self.row_ptr
        if getattr(self, "padded", False):
            return (rp[1:] - rp[:-1]).to(torch.float32)[:, None]
        if getattr(self, "_degree", None) is None:
            self._degree = (rp[1:] - rp[:-1]).to(torch.float32)[:, None]
        return self._degree

    @staticmethod
    def radius_graph(r0, box, pos, celllist_max=32, neighbours_max=64):
        """Nodes are connected if they are within r0 of each other under periodic
        boundary conditions given by box (3 floats).  pos: (batch, nodes, 3).
        (managan/graph_layers.py:25-34)"""
        batch, nodes, three = pos.shape
        assert three == 3
        assert torch.all(~torch.isnan(pos)), "some positions are NaN!"
        src, dst, edge_indices, row_ptr, order = ops.get_edges(celllist_max, neighbours_max, r0, *box, pos,
                                                               return_row_ptr=True, return_order=True)
        ans = Graph(src, dst, edge_indices, batch, nodes, row_ptr=row_ptr, cell_order=order)
        setattr(ans, "box", box)
        return ans


class _SortedIndex:
    """An index along dim 0 together with what its adjoint needs: the permutation that sorts it
    and the CSR row pointer of the sorted index.  For a sorted index the permutation is None."""

    def __init__(self, index32, n_rows, row_ptr=None, is_sorted=False):
        self.index = index32
        self.n_rows = n_rows
        self._row_ptr = row_ptr
        self._perm = None
        self.is_sorted = is_sorted

    @property
    def perm(self):
        if self.is_sorted:
            return None
        if self._perm is None:
            # stable sort by destination: index plumbing, done once per graph and only when a
            # gradient through a gather-by-dst is asked for
            self._perm = torch.sort(self.index.long(), stable=True).indices.to(torch.int32).contiguous()
        return self._perm

    @property
    def row_ptr(self):
        if self._row_ptr is None:
            # integer gather (a float32 detour would round node ids above 2^24)
            idx = self.index if self.is_sorted else self.index[self.perm.long()]
            self._row_ptr = ops.segment_row_ptr(idx.contiguous(), self.n_rows)
        return self._row_ptr


class _Gather(torch.autograd.Function):
    """x[index] along dim 0; adjoint: sum of the gradient rows that share an index
    (edges_read / edges_read_dst of managan/graph_layers.py:37-52 rely on torch indexing for this)."""

    @staticmethod
    def forward(ctx, x, sidx):
        ctx.sidx = sidx
        return ops.gather_rows(x.contiguous(), sidx.index)

    @staticmethod
    def jvp(ctx, x_t, _):
        return _Gather.apply(x_t, ctx.sidx)

    @staticmethod
    def backward(ctx, dy):
        return _ScatterSum.apply(dy, ctx.sidx), None


class _ScatterSum(torch.autograd.Function):
    """out[r] = sum of the rows e with index[e] = r; adjoint: a gather
    (torch_scatter.segment_coo at managan/graph_layers.py:54-59 for a sorted index)."""

    @staticmethod
    def forward(ctx, x_edge, sidx):
        ctx.sidx = sidx
        # (an unsorted index: the rows are read in its sorted order through the permutation)
        return ops.segment_sum_csr(x_edge.contiguous(), sidx.row_ptr, sidx.n_rows, perm=sidx.perm)

    @staticmethod
    def jvp(ctx, x_t, _):
        return _ScatterSum.apply(x_t, ctx.sidx)

    @staticmethod
    def backward(ctx, dy):
        return _Gather.apply(dy, ctx.sidx), None


def _flat_nodes(graph, x_node):
    b, n, *rest = x_node.shape
    assert b == graph.batch and n == graph.nodes
    return x_node.reshape(graph.batch * graph.nodes, *rest).contiguous()


def edges_read(graph: Graph, x_node: torch.Tensor):
    """x_node: (batch, nodes, ...) -> (x_src, x_dst), each (edges, ...)."""
    flat = _flat_nodes(graph, x_node)
    return _Gather.apply(flat, graph.by_src), _Gather.apply(flat, graph.by_dst)


def edges_read_dst(graph: Graph, x_node: torch.Tensor):
    """x_node: (batch, nodes, ...) -> x_dst: (edges, ...)."""
    return _Gather.apply(_flat_nodes(graph, x_node), graph.by_dst)


def edges_reduce_src(graph: Graph, x_edge: torch.Tensor):
    """Sum edge data onto the src node of each edge.  x_edge: (edges, ...)."""
    ans = _ScatterSum.apply(x_edge, graph.by_src)
    return ans.reshape(graph.batch, graph.nodes, *ans.shape[1:])


def segment_sum(x_edge, index, dim_size):
    """segment_coo(x_edge, index, dim_size=dim_size, reduce='sum') for a sorted index."""
    index = index.contiguous()
    sidx = _SortedIndex(index if index.dtype == torch.int32 else index.to(torch.int32), dim_size,
                        row_ptr=ops.segment_row_ptr(index, dim_size), is_sorted=True)
    return _ScatterSum.apply(x_edge, sidx)


def boxwrap(box: torch.Tensor, delta_pos: torch.Tensor):
    """Wrap a position difference to the shortest periodic image.  box: (3), delta_pos: (..., 3)."""
    return (delta_pos + 0.5 * box) % box - 0.5 * box


def edge_vectors(graph: Graph, pos: torch.Tensor, box, want_shift=False):
    """r_ij = boxwrap(box, pos[dst] - pos[src]) in one kernel (what graph_setup computes with
    two gathers and a wrap, archs/meanflow_painn8.py:167-172), optionally with the int8
    periodic-image shift of every edge."""
    flat = pos.reshape(graph.batch * graph.nodes, 3).contiguous()
    return ops.edge_vectors(flat, graph.src32, graph.dst32, box, want_shift=want_shift)


def graph_setup(r0, box, pos, neighbours_max=64, celllist_max=32):
    graph = Graph.radius_graph(r0, box, pos, celllist_max=celllist_max, neighbours_max=neighbours_max)
    return graph, edge_vectors(graph, pos, box)


def graph_setup_capacity(r0, box, pos, capacity, buffers=None):
    """graph_setup without the device->host copy of the edge count: the edge arrays hold `capacity` edges, of which
    the first E (graph.stats[0], on the device) are the graph; row_ptr is exact.  Nothing in it synchronises, so the
    call can be recorded into a HIP graph together with the layers (pass the `buffers` of an earlier call,
    graph.buffers, so that a replay writes into the same memory).  Entries of src / dst past E are valid but
    meaningless node indices: only kernels that walk the edges through row_ptr may be used on such a graph
    (graph.padded is True); per-edge tensors such as r_ij have `capacity` rows.
    When the graph has more than `capacity` edges the result is the graph cut at `capacity` edges: the edges that do
    not fit are dropped and row_ptr / edge counts are lowered to the capacity on the device, so nothing reads past
    the arrays; graph.stats[0] keeps the true count and graph.stats[3] has bit 1 set.  The count stays on the device
    inside a capture, so read graph.stats after the replay to know whether a result is that of the whole graph."""
    out = ops.neighbour_edges(pos.contiguous(), r0, box, capacity, out=buffers)
    batch, nodes = int(pos.shape[0]), int(pos.shape[1])
    graph = Graph(out["src"], out["dst"], out["edge_counts"], batch, nodes, row_ptr=out["row_ptr"],
                  cell_order=out["order"])
    graph.box = box
    graph.padded = True
    graph.stats = out["stats"]
    graph.buffers = out
    return graph, edge_vectors(graph, pos, box)


def expand_graph(graph: Graph, new_batch: int):
    assert graph.batch == 1, "Graph to be expanded should have batch size 1"
    offs = graph.nodes * torch.arange(new_batch, device=graph.src.device)[:, None]
    src = (graph.src[None].expand(new_batch, -1) + offs).flatten()
    dst = (graph.dst[None].expand(new_batch, -1) + offs).flatten()
    return Graph(src, dst, None, new_batch, graph.nodes)

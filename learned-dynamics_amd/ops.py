"""Torch-facing operators over the C ABI.

Each function validates its arguments the way the reference's C++ front ends
do (device, contiguity, rank and per-axis size checks, same messages), allocates
the outputs with torch, and enqueues the HIP kernels on the current torch
stream through libmanagan_hip.so.  Nothing here computes on the CPU or with
torch kernels: if the library is missing, importing this module fails.
"""
import contextlib
import ctypes
import weakref

import torch

from . import _lib as L

_lib = L.load()

BEE_ORDER = ("000", "110", "220", "011", "101", "121", "211", "022", "202", "112", "222", "111", "212")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


class _AlreadyCurrent:
    """A context that does nothing: the device asked for is the current one."""

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_ALREADY_CURRENT = _AlreadyCurrent()


def _on(device):
    """`with _on(t.device):` makes t's device current for the allocations and launches inside, like torch.cuda.device,
    without that context manager's bookkeeping when the device is current already (every call on a one-GPU host)."""
    if _raw_device is not None and (device.index is None or device.index == _raw_device()):
        return _ALREADY_CURRENT
    return torch.cuda.device(device)


def _stream():
    """The current HIP stream of the current device as a pointer argument."""
    if _raw_stream is not None and _raw_device is not None:     # same value as below, without building Stream objects
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


CONCURRENT_MAX_ROWS = 16384      # above this many rows a kernel fills the chip by itself
_side_streams = {}


def concurrent(fns, rows=0):
    """Results of independent callables.  With few rows (a single small system) each kernel of a layer occupies a
    fraction of the chip for a few microseconds, so independent pieces of a layer (the input linears of the three
    ranks, the three output kernels, the norms) are enqueued on side streams between a fork event and join events and
    overlap on the GPU when the launches are being captured into a HIP graph; with many rows, one callable or eager
    execution they simply run in turn.  Every side stream starts after
    everything enqueued so far on the current stream and the current stream continues after all of them, so sections
    are totally ordered among each other, memory handed between them needs no extra bookkeeping, and a HIP graph
    capture records the fork and join as dependencies.  Default stream priority throughout."""
    fns = list(fns)
    # eager launches of such small kernels are bound by the host, which the events would only slow down further: the
    # overlap is for captured graphs
    if len(fns) < 2 or rows > CONCURRENT_MAX_ROWS or not torch.cuda.is_current_stream_capturing():
        return [f() for f in fns]
    main = torch.cuda.current_stream()
    key = main.device.index
    pool = _side_streams.setdefault(key, [])
    while len(pool) < len(fns) - 1:
        pool.append(torch.cuda.Stream(device=main.device))
    fork = torch.cuda.Event()
    fork.record(main)
    outs = [None] * len(fns)
    joins = []
    for k in range(1, len(fns)):
        side = pool[k - 1]
        side.wait_event(fork)
        with torch.cuda.stream(side):
            outs[k] = fns[k]()
            done = torch.cuda.Event()
            done.record(side)
        joins.append(done)
    outs[0] = fns[0]()
    for done in joins:
        main.wait_event(done)
    return outs


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _check_input(t, name, dtype=torch.float32):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dtype != dtype:
        raise RuntimeError(f"expected scalar type {str(dtype).replace('torch.', '').capitalize()} "
                           f"but found {str(t.dtype).replace('torch.', '')} for {name}")


# --------------------------------------------------------------------- stage A
_edge_count_hint = {}      # (batch, nodes, cutoff, box) -> edge count of the last search of that shape
_pinned_pool = []          # statistics words free for the next search
_pinned_abandoned = []     # words of searches that were dropped unread: a kernel may still be about to write them


def _pinned_stats():
    """Four int32 words of pinned host memory (device-visible at the same address), reused between searches.  The
    words are never handed back to the allocator: a search that is dropped before its statistics were read leaves
    them on a list that is recycled after a device synchronisation."""
    if not _pinned_pool and len(_pinned_abandoned) >= 64:
        torch.cuda.synchronize()
        _pinned_pool.extend(_pinned_abandoned)
        del _pinned_abandoned[:]
    return _pinned_pool.pop() if _pinned_pool else torch.empty(4, dtype=torch.int32, pin_memory=True)


class NeighbourSearch:
    """Result of the count phase; `fill()` writes the edges."""

    def __init__(self, x, cutoff, box):
        _check_input(x, "x")
        if x.dim() != 3 or x.size(2) != 3:
            raise RuntimeError("x must have shape (batch, nodes, 3)")
        self.x = x
        self.batch, self.nodes = int(x.size(0)), int(x.size(1))
        self.cutoff = float(cutoff)
        self.box = tuple(float(b) for b in box)
        nbytes = ctypes.c_size_t(0)
        L.check(_lib.mg_neighbour_workspace_bytes(self.batch, self.nodes, self.cutoff, *self.box,
                                                  ctypes.byref(nbytes)))
        dev = x.device
        with _on(dev):
            self.workspace = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
            self.row_ptr = torch.empty(self.batch * self.nodes + 1, dtype=torch.int32, device=dev)
            self.edge_counts = torch.empty(self.batch, dtype=torch.int32, device=dev)
            # The four statistics go to pinned host memory, which the GPU writes directly: the host needs the edge
            # count to size src / dst, and polling four words that the scan kernel stores as soon as it knows them
            # costs a few microseconds where a device->host copy with its synchronisation costs about twenty.
            self.stats = _pinned_stats()
            self._stats_np = self.stats.numpy()
            self._stats_np[:] = -1                     # (never a valid value: the kernels store counts and flags)
            L.check(_lib.mg_neighbour_count(_p(x), self.batch, self.nodes, self.cutoff, *self.box,
                                            _p(self.workspace), self.workspace.numel(), _p(self.row_ptr),
                                            _p(self.edge_counts), _p(self.stats), _stream()))
        self._host_stats = None

    def host_stats(self):
        """(E, max atoms per cell, max degree, overflow flag), read from the pinned words the kernels write; falls
        back to a stream synchronisation if they have not all arrived after a bounded number of polls."""
        if self._host_stats is None:
            st = self._stats_np
            for _ in range(20000):
                if st.min() >= 0:
                    break
            else:
                torch.cuda.current_stream(self.x.device).synchronize()
            self._host_stats = tuple(int(v) for v in st)
            _pinned_pool.append(self.stats)            # every word has arrived: nothing will write them again
            self.stats = torch.tensor(self._host_stats, dtype=torch.int32)
            self._stats_np = None
            if min(self._host_stats) < 0:
                raise RuntimeError("the neighbour search did not report its statistics")
            if self._host_stats[3]:
                raise RuntimeError("edge count does not fit int32")
        return self._host_stats

    def __del__(self):
        if getattr(self, "_stats_np", None) is not None:
            _pinned_abandoned.append(self.stats)

    def fill(self, n_edges=None):
        """src, dst of exactly E edges.  With n_edges the caller fixes the capacity (edges beyond a capacity below E
        are dropped, never written).  Otherwise the edge count comes from the device, and the wait for it is taken off
        the critical path: the fill pass is queued at once into arrays sized from an estimate (the edge count of the
        last search of this shape, else the mean density, plus a margin), the count is read afterwards, and the
        first E entries are returned; only when the estimate was too small is the pass run again at the exact size."""
        dev = self.x.device
        if n_edges is not None or self._host_stats is not None:
            E = self.host_stats()[0] if n_edges is None else int(n_edges)
            with _on(dev):
                src = torch.empty(E, dtype=torch.int32, device=dev)
                dst = torch.empty(E, dtype=torch.int32, device=dev)
            return self.fill_into(src, dst)
        key = (self.batch, self.nodes, self.cutoff, self.box)
        hint = _edge_count_hint.get(key)
        if hint is None:
            volume = self.box[0] * self.box[1] * self.box[2]
            hint = 1.5 * self.batch * self.nodes * (self.nodes / volume) * 4.18879 * self.cutoff ** 3
        capacity = min(int(1.125 * hint) + 4096, 2 ** 31 - 1)
        with _on(dev):
            src = torch.empty(capacity, dtype=torch.int32, device=dev)
            dst = torch.empty(capacity, dtype=torch.int32, device=dev)
        self.fill_into(src, dst)
        E = self.host_stats()[0]
        if len(_edge_count_hint) > 256:
            _edge_count_hint.clear()
        _edge_count_hint[key] = E
        if E <= capacity:
            return src[:E], dst[:E]
        return self.fill(E)

    def fill_into(self, src, dst):
        """Write the edges into caller-owned int32 arrays whose common length is the capacity; no host
        synchronisation.  `stats[0]` (device) holds the true edge count for the caller to compare."""
        _check_input(src, "src", torch.int32)
        _check_input(dst, "dst", torch.int32)
        if src.numel() != dst.numel():
            raise RuntimeError("src and dst must have the same length")
        with _on(self.x.device):
            L.check(_lib.mg_neighbour_fill(_p(self.workspace), self.workspace.numel(), self.batch, self.nodes,
                                           self.cutoff, *self.box, _p(self.row_ptr), int(src.numel()), _p(src),
                                           _p(dst), _stream()))
        return src, dst


    def cell_order(self):
        """int32 (batch*nodes): atom ids in cell order (a cache-friendly row order for the edge kernels)."""
        dev = self.x.device
        with _on(dev):
            order = torch.empty(self.batch * self.nodes, dtype=torch.int32, device=dev)
            L.check(_lib.mg_neighbour_cell_order(_p(self.workspace), self.workspace.numel(), self.batch, self.nodes,
                                                 self.cutoff, *self.box, _p(order), _stream()))
        return order


def neighbour_edges(x, cutoff, box, capacity, out=None):
    """Radius graph into arrays of `capacity` edges without reading the edge count back: one enqueue, no host
    synchronisation (recordable into a HIP graph once `out` holds the buffers of an earlier call).
    Returns dict(src, dst, row_ptr, edge_counts, stats, workspace, order); stats[0] (device) is the true edge count,
    edges beyond the capacity are dropped; order is the cell order of the atoms."""
    _check_input(x, "x")
    if x.dim() != 3 or x.size(2) != 3:
        raise RuntimeError("x must have shape (batch, nodes, 3)")
    B, N = int(x.size(0)), int(x.size(1))
    box = tuple(float(b) for b in box)
    dev = x.device
    with _on(dev):
        if out is None:
            nbytes = ctypes.c_size_t(0)
            L.check(_lib.mg_neighbour_workspace_bytes(B, N, float(cutoff), *box, ctypes.byref(nbytes)))
            out = dict(workspace=torch.empty(nbytes.value, dtype=torch.uint8, device=dev),
                       row_ptr=torch.empty(B * N + 1, dtype=torch.int32, device=dev),
                       edge_counts=torch.empty(B, dtype=torch.int32, device=dev),
                       stats=torch.empty(4, dtype=torch.int32, device=dev),
                       # zeros: entries past the edge count are never written by the search and must stay valid
                       # node indices for kernels that run over the whole capacity
                       src=torch.zeros(int(capacity), dtype=torch.int32, device=dev),
                       dst=torch.zeros(int(capacity), dtype=torch.int32, device=dev),
                       order=torch.empty(B * N, dtype=torch.int32, device=dev))
        L.check(_lib.mg_neighbour_edges(_p(x), B, N, float(cutoff), *box, _p(out["workspace"]), out["workspace"].numel(),
                                        _p(out["row_ptr"]), _p(out["edge_counts"]), _p(out["stats"]),
                                        int(out["src"].numel()), _p(out["src"]), _p(out["dst"]), _stream()))
        L.check(_lib.mg_neighbour_cell_order(_p(out["workspace"]), out["workspace"].numel(), B, N, float(cutoff), *box,
                                             _p(out["order"]), _stream()))
    return out


def _check_caps(search, listmax, neighboursmax):
    """The reference's overflow errors, in the reference's order
    (extensions/neighbour_grid/neighbour_grid_kern.cu:195-217)."""
    _, max_cell, max_deg, _ = search.host_stats()
    if max_cell > listmax:
        raise RuntimeError("Cell list overflow occurred. Trying increasing listmax.")
    if listmax not in (32, 64, 128, 256):
        raise RuntimeError("expected listmax to be one of 32, 64, 128, 256. other values not supported!")
    if max_deg > neighboursmax:
        raise RuntimeError("Neighbour list overflow occurred. Try increasing neighboursmax.")


def get_edges(listmax, neighboursmax, cutoff, box_x, box_y, box_z, x, return_row_ptr=False, return_order=False):
    """(src int32[E], dst int32[E], edgeCounts int32[B]); extensions/neighbour_grid/neighbour_grid.cpp:170-195."""
    search = NeighbourSearch(x, cutoff, (box_x, box_y, box_z))
    src, dst = search.fill()                       # queued before the statistics are read (see fill)
    _check_caps(search, listmax, neighboursmax)
    out = (src, dst, search.edge_counts)
    if return_row_ptr:
        out = out + (search.row_ptr,)
    if return_order:
        out = out + (search.cell_order(),)
    return out


def get_neighbours(listmax, neighboursmax, cutoff, box_x, box_y, box_z, x):
    """(neighbours int32[B,N,neighboursmax], counts int32[B,N]); neighbour_grid.cpp:59-103."""
    search = NeighbourSearch(x, cutoff, (box_x, box_y, box_z))
    _check_caps(search, listmax, neighboursmax)
    _, dst = search.fill()
    B, N = search.batch, search.nodes
    with _on(x.device):
        neighbours = torch.empty(B, N, neighboursmax, dtype=torch.int32, device=x.device)
        counts = torch.empty(B, N, dtype=torch.int32, device=x.device)
        L.check(_lib.mg_neighbour_pad(_p(search.row_ptr), _p(dst), B, N, neighboursmax, _p(neighbours),
                                      _p(counts), _stream()))
    return neighbours, counts


def wrap_cells(cutoff, box, x):
    _check_input(x, "x")
    B, N = int(x.size(0)), int(x.size(1))
    with _on(x.device):
        w = torch.empty_like(x)
        cell = torch.empty(B, N, dtype=torch.int32, device=x.device)
        L.check(_lib.mg_neighbour_wrap_cells(_p(x), B, N, float(cutoff), *[float(b) for b in box], _p(w),
                                             _p(cell), _stream()))
    return w, cell


def padded_edges_read(counts, neighbours, x):
    _check_input(counts, "neighbourCounts", torch.int32)
    _check_input(neighbours, "neighbours", torch.int32)
    _check_input(x, "x")
    if counts.dim() != 2:
        raise RuntimeError("neighbourCounts must have shape (batch, nodes)")
    if neighbours.dim() != 3:
        raise RuntimeError("neighbourCounts must have shape (batch, nodes, neighboursmax)")
    if x.dim() != 3:
        raise RuntimeError("x must have shape (batch, nodes, chan)")
    B, N = counts.shape
    if not (B == neighbours.size(0) == x.size(0)):
        raise RuntimeError("batch dimension of all tensors must match")
    if not (N == neighbours.size(1) == x.size(1)):
        raise RuntimeError("node dimension of all tensors must match")
    nmax, chan = int(neighbours.size(2)), int(x.size(2))
    with _on(x.device):
        out = torch.empty(B, N, nmax, chan, dtype=torch.float32, device=x.device)
        L.check(_lib.mg_padded_edges_read(_p(counts), _p(neighbours), _p(x), B, N, nmax, chan, _p(out), _stream()))
    return out


def padded_edges_reduce(counts, neighbours, x):
    _check_input(counts, "neighbourCounts", torch.int32)
    _check_input(neighbours, "neighbours", torch.int32)
    _check_input(x, "x")
    if counts.dim() != 2:
        raise RuntimeError("neighbourCounts must have shape (batch, nodes)")
    if neighbours.dim() != 3:
        raise RuntimeError("neighbours must have shape (batch, nodes, neighboursmax)")
    if x.dim() != 4:
        raise RuntimeError("x must have shape (batch, nodes, neighboursmax, chan)")
    B, N = counts.shape
    if not (B == neighbours.size(0) == x.size(0)):
        raise RuntimeError("batch dimension of all tensors must match")
    if not (N == neighbours.size(1) == x.size(1)):
        raise RuntimeError("node dimension of all tensors must match")
    nmax = int(neighbours.size(2))
    if nmax != x.size(2):
        raise RuntimeError("neighboursmax dimension must match between neighbours and x")
    chan = int(x.size(3))
    with _on(x.device):
        out = torch.empty(B, N, chan, dtype=torch.float32, device=x.device)
        L.check(_lib.mg_padded_edges_reduce(_p(counts), _p(x), B, N, nmax, chan, _p(out), _stream()))
    return out


def edge_vectors(pos, src, dst, box, want_shift=False):
    """r_ij = boxwrap(box, pos[dst] - pos[src]) (E,3) and optionally the int8 image shift."""
    _check_input(pos, "pos")
    _check_input(src, "src", torch.int32)
    _check_input(dst, "dst", torch.int32)
    E = int(src.numel())
    with _on(pos.device):
        r = torch.empty(E, 3, dtype=torch.float32, device=pos.device)
        shift = torch.empty(E, 3, dtype=torch.int8, device=pos.device) if want_shift else None
        L.check(_lib.mg_edge_vectors(_p(pos), _p(src), _p(dst), E, *[float(b) for b in box], _p(r), _p(shift),
                                     _stream()))
    return (r, shift) if want_shift else r


# --------------------------------------------------------------------- stage C
def segment_row_ptr(index, n_rows):
    if index.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("index must be int32 or int64")
    _check_input(index, "index", index.dtype)
    with _on(index.device):
        row_ptr = torch.empty(n_rows + 1, dtype=torch.int32, device=index.device)
        L.check(_lib.mg_segment_row_ptr(_p(index), int(index.dtype == torch.int64), int(index.numel()), int(n_rows),
                                        _p(row_ptr), _stream()))
    return row_ptr


def segment_sum_csr(x_edge, row_ptr, n_rows, perm=None):
    """out[r] = sum of x_edge[row_ptr[r]:row_ptr[r+1]]; trailing dims kept.  perm (int32, one entry per edge): the rows
    are taken in the order x_edge[perm] without copying them into it."""
    _check_input(x_edge, "x_edge")
    _check_input(row_ptr, "row_ptr", torch.int32)
    if perm is not None:
        _check_input(perm, "perm", torch.int32)
        if perm.numel() != x_edge.size(0):
            raise RuntimeError("perm must have one entry per edge")
    rest = tuple(x_edge.shape[1:])
    feat = 1
    for d in rest:
        feat *= int(d)
    with _on(x_edge.device):
        out = torch.empty((n_rows,) + rest, dtype=torch.float32, device=x_edge.device)
        L.check(_lib.mg_segment_sum_csr_perm(_p(x_edge), _p(perm), _p(row_ptr), int(n_rows), feat, _p(out), _stream()))
    return out


def gather_rows(x, index):
    """x[index] along dim 0 for a contiguous float32 x."""
    _check_input(x, "x")
    if index.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("index must be int32 or int64")
    _check_input(index, "index", index.dtype)
    rest = tuple(x.shape[1:])
    feat = 1
    for d in rest:
        feat *= int(d)
    E = int(index.numel())
    with _on(x.device):
        out = torch.empty((E,) + rest, dtype=torch.float32, device=x.device)
        L.check(_lib.mg_gather_rows(_p(x), _p(index), int(index.dtype == torch.int64), E, int(x.size(0)), feat,
                                    _p(out), _stream()))
    return out


# --------------------------------------------------------------------- stage B
def _rows_chan(tensors_by_rank, names):
    """Shape checks of the fused product ops: exactly (R,C), (R,C,3), (R,C,3,3), all R and C equal."""
    rows = chan = None
    for t, name, rank in zip(tensors_by_rank, names, (0, 1, 2) * 5):
        _check_input(t, name)
        if t.dim() != 2 + rank:
            raise RuntimeError(f"{name} has wrong number of axes")
        for ax in range(rank):
            if t.size(2 + ax) != 3:
                raise RuntimeError(f"{name} must have size 3 on tensor axes")
        if rows is None:
            rows, chan = int(t.size(0)), int(t.size(1))
        if t.size(0) != rows:
            raise RuntimeError(f"{name} batch size mismatch")
        if t.size(1) != chan:
            raise RuntimeError(f"{name} channel size mismatch")
    return rows, chan


def _shape(rows, chan, rank):
    return (rows, chan) + (3,) * rank


def bee_fwd(l_0, l_1, l_2, r_0, r_1, r_2):
    rows, chan = _rows_chan((l_0, l_1, l_2), ("l_0", "l_1", "l_2"))
    rows2, chan2 = _rows_chan((r_0, r_1, r_2), ("r_0", "r_1", "r_2"))
    if rows2 != rows or chan2 != chan:
        raise RuntimeError("left and right operands must agree on batch and channel sizes")
    dev = l_0.device
    with _on(dev):
        ys = [torch.empty(_shape(rows, chan, int(lab[2])), dtype=torch.float32, device=dev) for lab in BEE_ORDER]
        arr = L.PtrArray13(*[y.data_ptr() for y in ys])
        L.check(_lib.mg_bee_fwd(_p(l_0), _p(l_1), _p(l_2), _p(r_0), _p(r_1), _p(r_2), rows, chan,
                                ctypes.byref(arr), _stream()))
    return ys


def _bee_bwd(side, o_0, o_1, o_2, dys):
    rows, chan = _rows_chan((o_0, o_1, o_2), ("x_0", "x_1", "x_2"))
    if len(dys) != 13:
        raise RuntimeError("expected 13 output gradients")
    for dy, lab in zip(dys, BEE_ORDER):
        _check_input(dy, f"dy_{lab}")
        if tuple(dy.shape) != _shape(rows, chan, int(lab[2])):
            raise RuntimeError(f"dy_{lab} has wrong shape")
    dev = o_0.device
    with _on(dev):
        d = [torch.empty(_shape(rows, chan, k), dtype=torch.float32, device=dev) for k in range(3)]
        arr = L.PtrArray13(*[dy.data_ptr() for dy in dys])
        L.check(_lib.mg_bee_bwd(side, _p(o_0), _p(o_1), _p(o_2), ctypes.byref(arr), rows, chan, _p(d[0]),
                                _p(d[1]), _p(d[2]), _stream()))
    return d


def bee_edge_filters_fwd(enc, rh):
    """(phi_v, phi_d) = (enc[..., None] * rh[:, None, :], enc[..., None, None] * rh[:, None, None, :] * rh[:, None, :, None])
    for enc (E, chan) and rh (E, 3) (archs/diffuser_atoms15.py:240-243), one kernel."""
    _check_input(enc, "enc")
    _check_input(rh, "rh")
    E, chan = int(enc.size(0)), int(enc.size(1))
    if enc.dim() != 2 or tuple(rh.shape) != (E, 3):
        raise RuntimeError("expected enc (E, chan) and rh (E, 3)")
    with _on(enc.device):
        phi_v = torch.empty(E, chan, 3, dtype=torch.float32, device=enc.device)
        phi_d = torch.empty(E, chan, 3, 3, dtype=torch.float32, device=enc.device)
        L.check(_lib.mg_bee_edge_filters_fwd(_p(enc), _p(rh), E, chan, _p(phi_v), _p(phi_d), _stream()))
    return phi_v, phi_d


def bee_edge_filters_bwd(enc, rh, g_v, g_d):
    """(d_enc, d_rh): the adjoint of bee_edge_filters_fwd."""
    for t, name in ((enc, "enc"), (rh, "rh"), (g_v, "g_v"), (g_d, "g_d")):
        _check_input(t, name)
    E, chan = int(enc.size(0)), int(enc.size(1))
    if tuple(rh.shape) != (E, 3) or tuple(g_v.shape) != (E, chan, 3) or tuple(g_d.shape) != (E, chan, 3, 3):
        raise RuntimeError("expected rh (E, 3), g_v (E, chan, 3), g_d (E, chan, 3, 3)")
    with _on(enc.device):
        d_enc, d_rh = torch.empty_like(enc), torch.empty_like(rh)
        L.check(_lib.mg_bee_edge_filters_bwd(_p(enc), _p(rh), _p(g_v), _p(g_d), E, chan, _p(d_enc), _p(d_rh), _stream()))
    return d_enc, d_rh


SILU_MAX_ORDER = 4


def silu_order(z, order, mul=None):
    """SiLU^(order)(z), elementwise, times mul if given (same shape); order 0 .. SILU_MAX_ORDER."""
    _check_input(z, "z")
    if mul is not None:
        _check_input(mul, "mul")
        if mul.shape != z.shape:
            raise RuntimeError("mul must have the shape of z")
    if not 0 <= int(order) <= SILU_MAX_ORDER:
        raise RuntimeError(f"silu_order: order must be in 0..{SILU_MAX_ORDER}")
    with _on(z.device):
        out = torch.empty_like(z)
        L.check(_lib.mg_silu_order(_p(z), _p(mul) if mul is not None else None, z.numel(), int(order), _p(out), _stream()))
    return out


def bee_indexed_supported(chan):
    return bool(_lib.mg_bee_indexed_supported(int(chan)))


def bee_fwd_indexed(l_0, l_1, l_2, l_index, r_0, r_1, r_2):
    """bee_fwd with the left operands given per node: product row e reads row l_index[e] (int32) of l_*."""
    n_l, chan = _rows_chan((l_0, l_1, l_2), ("l_0", "l_1", "l_2"))
    rows, chan2 = _rows_chan((r_0, r_1, r_2), ("r_0", "r_1", "r_2"))
    _check_input(l_index, "l_index", torch.int32)
    if chan2 != chan or l_index.numel() != rows:
        raise RuntimeError("operands must agree on the channel size and l_index must have one entry per row")
    dev = r_0.device
    with _on(dev):
        ys = [torch.empty(_shape(rows, chan, int(lab[2])), dtype=torch.float32, device=dev) for lab in BEE_ORDER]
        arr = L.PtrArray13(*[y.data_ptr() for y in ys])
        L.check(_lib.mg_bee_fwd_indexed(_p(l_0), _p(l_1), _p(l_2), _p(l_index), n_l, _p(r_0), _p(r_1), _p(r_2), rows,
                                        chan, ctypes.byref(arr), _stream()))
    return ys


def bee_bwd_indexed(side, o_0, o_1, o_2, o_index, dys, dy_index, rows):
    """bee_bwl (side 0) / bee_bwr (side 1) for `rows` product rows, with the other side's operands read through
    o_index (or None: one row per product row) and every output gradient that does not have `rows` rows read through
    dy_index (gradients of products that were summed over the edges of a node)."""
    n_o, chan = _rows_chan((o_0, o_1, o_2), ("x_0", "x_1", "x_2"))
    if len(dys) != 13:
        raise RuntimeError("expected 13 output gradients")
    if o_index is None and n_o != rows:
        raise RuntimeError("operands without an index need one row per product row")
    mask, dy_rows = 0, 0
    for k, (dy, lab) in enumerate(zip(dys, BEE_ORDER)):
        _check_input(dy, f"dy_{lab}")
        if tuple(dy.shape[1:]) != _shape(rows, chan, int(lab[2]))[1:]:
            raise RuntimeError(f"dy_{lab} has wrong shape")
        if dy.size(0) != rows:
            if dy_index is None or (dy_rows and dy.size(0) != dy_rows):
                raise RuntimeError(f"dy_{lab} has {dy.size(0)} rows for {rows} product rows")
            mask |= 1 << k
            dy_rows = int(dy.size(0))
    for idx, name in ((o_index, "o_index"), (dy_index, "dy_index")):
        if idx is not None:
            _check_input(idx, name, torch.int32)
            if idx.numel() != rows:
                raise RuntimeError(f"{name} must have one entry per product row")
    dev = o_0.device
    with _on(dev):
        d = [torch.empty(_shape(rows, chan, k), dtype=torch.float32, device=dev) for k in range(3)]
        arr = L.PtrArray13(*[dy.data_ptr() for dy in dys])
        L.check(_lib.mg_bee_bwd_indexed(side, _p(o_0), _p(o_1), _p(o_2), _p(o_index), n_o, ctypes.byref(arr),
                                        _p(dy_index), dy_rows, mask, int(rows), chan, _p(d[0]), _p(d[1]), _p(d[2]),
                                        _stream()))
    return d


def bee_bwl(r_0, r_1, r_2, *dys):
    return _bee_bwd(0, r_0, r_1, r_2, dys)


def bee_bwr(l_0, l_1, l_2, *dys):
    return _bee_bwd(1, l_0, l_1, l_2, dys)


def _cow_inputs(l_0, l_1, r_0, r_1):
    rows, chan = _rows_chan((l_0, l_1), ("l_0", "l_1"))
    rows2, chan2 = _rows_chan((r_0, r_1), ("r_0", "r_1"))
    if rows2 != rows or chan2 != chan:
        raise RuntimeError("left and right operands must agree on batch and channel sizes")
    return rows, chan


def cow_o0_fwd(l_0, l_1, r_0, r_1):
    rows, chan = _cow_inputs(l_0, l_1, r_0, r_1)
    dev = l_0.device
    with _on(dev):
        y0 = torch.empty(rows, chan, dtype=torch.float32, device=dev)
        y1 = torch.empty(rows, chan, dtype=torch.float32, device=dev)
        L.check(_lib.mg_cow_o0_fwd(_p(l_0), _p(l_1), _p(r_0), _p(r_1), rows, chan, _p(y0), _p(y1), _stream()))
    return [y0, y1]


def cow_o1_fwd(l_0, l_1, r_0, r_1):
    rows, chan = _cow_inputs(l_0, l_1, r_0, r_1)
    dev = l_0.device
    with _on(dev):
        ys = [torch.empty(rows, chan, 3, dtype=torch.float32, device=dev) for _ in range(3)]
        L.check(_lib.mg_cow_o1_fwd(_p(l_0), _p(l_1), _p(r_0), _p(r_1), rows, chan, _p(ys[0]), _p(ys[1]),
                                   _p(ys[2]), _stream()))
    return ys


def _cow_bwd(which, side, o_0, o_1, dys):
    rows, chan = _rows_chan((o_0, o_1), ("x_0", "x_1"))
    ranks = (0, 0) if which == 0 else (1, 1, 1)
    if len(dys) != len(ranks):
        raise RuntimeError("wrong number of output gradients")
    for k, (dy, rk) in enumerate(zip(dys, ranks)):
        _check_input(dy, f"dy[{k}]")
        if tuple(dy.shape) != _shape(rows, chan, rk):
            raise RuntimeError(f"dy[{k}] has wrong shape")
    dev = o_0.device
    with _on(dev):
        d0 = torch.empty(rows, chan, dtype=torch.float32, device=dev)
        d1 = torch.empty(rows, chan, 3, dtype=torch.float32, device=dev)
        if which == 0:
            L.check(_lib.mg_cow_o0_bwd(side, _p(o_0), _p(o_1), _p(dys[0]), _p(dys[1]), rows, chan, _p(d0), _p(d1),
                                       _stream()))
        else:
            L.check(_lib.mg_cow_o1_bwd(side, _p(o_0), _p(o_1), _p(dys[0]), _p(dys[1]), _p(dys[2]), rows, chan,
                                       _p(d0), _p(d1), _stream()))
    return [d0, d1]


def cow_o0_bwl(r_0, r_1, *dys):
    return _cow_bwd(0, 0, r_0, r_1, dys)


def cow_o0_bwr(l_0, l_1, *dys):
    return _cow_bwd(0, 1, l_0, l_1, dys)


def cow_o1_bwl(r_0, r_1, *dys):
    return _cow_bwd(1, 0, r_0, r_1, dys)


def cow_o1_bwr(l_0, l_1, *dys):
    return _cow_bwd(1, 1, l_0, l_1, dys)


# ---------------------------------------------------------------- Ant16
def _ant16_check(x_0, x_1, x_2, pairs):
    """Shape checks of ant16_o*_cuda (extensions/codegen_tensops/codegen_tensops.cpp:610-660), same messages."""
    for t, nm in ((x_0, "x_0"), (x_1, "x_1"), (x_2, "x_2")):
        if t is not None:
            _check_input(t, nm)
    batch = None
    dims = [None, None, None]
    for k, (t, nm) in enumerate(((x_0, "x_0"), (x_1, "x_1"), (x_2, "x_2"))):
        if t is None:
            continue
        if t.dim() != 2 + k:
            raise RuntimeError(f"{nm} has wrong number of axes")
        if batch is None:
            batch = int(t.size(0))
        elif t.size(0) != batch:
            raise RuntimeError(f"{nm}: expected axis 0 to have size batch")
        dims[k] = int(t.size(1))
        for ax in range(2, 2 + k):
            if t.size(ax) != 3:
                raise RuntimeError(f"{nm}: expected axis {ax} to have size 3")
    dim_l = None
    for lab, P, left in pairs:
        _check_input(P, f"P_{lab}")
        _check_input(left, f"left_{lab}")
        rl, rr, ro = int(lab[0]), int(lab[1]), int(lab[2])
        if P.dim() != 3:
            raise RuntimeError(f"P_{lab} has wrong number of axes")
        if P.size(0) != dims[ro]:
            raise RuntimeError(f"P_{lab}: expected axis 0 to have size dim_{ro}")
        if dim_l is None:
            dim_l = int(P.size(1))
        elif P.size(1) != dim_l:
            raise RuntimeError(f"P_{lab}: expected axis 1 to have size dim_l")
        if P.size(2) != dims[rr]:
            raise RuntimeError(f"P_{lab}: expected axis 2 to have size dim_{rr}")
        if left.dim() != 2 + rl:
            raise RuntimeError(f"left_{lab} has wrong number of axes")
        if left.size(0) != batch:
            raise RuntimeError(f"left_{lab}: expected axis 0 to have size batch")
        if left.size(1) != dim_l:
            raise RuntimeError(f"left_{lab}: expected axis 1 to have size dim_l")
        for ax in range(2, 2 + rl):
            if left.size(ax) != 3:
                raise RuntimeError(f"left_{lab}: expected axis {ax} to have size 3")
    return batch, dims, dim_l


def _ant16(rank_o, x_0, x_1, x_2, pairs):
    """y (rows, dim_o, (3,)^rank_o) = sum over the given (label, P, left) of the Ant16 contraction."""
    batch, dims, dim_l = _ant16_check(x_0, x_1, x_2, pairs)
    dev = pairs[0][1].device
    n = len(pairs)
    labels = (ctypes.c_int * n)(*[BEE_ORDER.index(lab) for lab, _, _ in pairs])
    Ps = (ctypes.c_void_p * n)(*[P.data_ptr() for _, P, _ in pairs])
    lefts = (ctypes.c_void_p * n)(*[left.data_ptr() for _, _, left in pairs])
    with _on(dev):
        y = torch.empty(_shape(batch, dims[rank_o], rank_o), dtype=torch.float32, device=dev)
        if batch > 0:
            L.check(_lib.mg_ant16_fwd(rank_o, n, labels, Ps, lefts, _p(x_0), _p(x_1), _p(x_2), batch,
                                      dims[0] or 0, dims[1] or 0, dims[2] or 0, dim_l, 0, _p(y), _stream()))
    return y


def ant16_o0(x_0, x_1, x_2, P_000, left_000, P_110, left_110, P_220, left_220):
    return [_ant16(0, x_0, x_1, x_2, [("000", P_000, left_000), ("110", P_110, left_110), ("220", P_220, left_220)])]


def ant16_o1(x_0, x_1, x_2, P_011, left_011, P_101, left_101, P_121, left_121, P_211, left_211):
    return [_ant16(1, x_0, x_1, x_2, [("011", P_011, left_011), ("101", P_101, left_101), ("121", P_121, left_121),
                                      ("211", P_211, left_211)])]


def ant16_o2(x_0, x_1, x_2, P_022, left_022, P_202, left_202, P_112, left_112, P_222, left_222):
    return [_ant16(2, x_0, x_1, x_2, [("022", P_022, left_022), ("202", P_202, left_202), ("112", P_112, left_112),
                                      ("222", P_222, left_222)])]


def ant16_oc(x_1, x_2, P_111, left_111, P_212, left_212):
    """The two chiral products: (y_1c, y_2c).  x_2 only fixes dim_2 (rank-2 output channels)."""
    return [_ant16(1, None, x_1, x_2, [("111", P_111, left_111)]),
            _ant16(2, None, x_1, x_2, [("212", P_212, left_212)])]


def _ant16_dims(pairs_P):
    """(dim_0, dim_1, dim_2, dim_l) from the shapes of the P of some product types (label, P)."""
    dims, dim_l = [0, 0, 0], 0
    for lab, P in pairs_P:
        if P.dim() != 3:
            raise RuntimeError(f"P_{lab} has wrong number of axes")
        for k, size in ((int(lab[2]), int(P.size(0))), (int(lab[1]), int(P.size(2)))):
            if dims[k] not in (0, size):
                raise RuntimeError(f"P_{lab}: channel counts of rank {k} disagree")
            dims[k] = size
        if dim_l not in (0, int(P.size(1))):
            raise RuntimeError(f"P_{lab}: expected axis 1 to have size dim_l")
        dim_l = int(P.size(1))
    return dims, dim_l


def ant16_grad_x(rank_r, dys, terms):
    """Gradient for x_{rank_r} of the Ant16 contraction: sum over `terms` = [(label, P, left)] whose right operand
    has that rank of  dx[b,j,X] = sum_{o,i} P[o,i,j] C_X(left[b,i,:], dy[b,o,:]); dys = (dy_0, dy_1, dy_2), entries
    the terms do not use may be None (ant16_o*_backward_cuda, extensions/codegen_tensops/codegen_tensops.cpp:669-821)."""
    terms = [(lab, P.contiguous(), left.contiguous()) for lab, P, left in terms]
    dys = [None if d is None else d.contiguous() for d in dys]
    dims, dim_l = _ant16_dims([(lab, P) for lab, P, _ in terms])
    batch = int(terms[0][2].size(0))
    dev = terms[0][1].device
    n = len(terms)
    for lab, P, left in terms:
        if int(lab[1]) != rank_r:
            raise RuntimeError(f"product {lab} has no right operand of rank {rank_r}")
        dy = dys[int(lab[2])]
        if dy is None or tuple(dy.shape) != _shape(batch, dims[int(lab[2])], int(lab[2])):
            raise RuntimeError(f"dy_{lab[2]}: expected shape {_shape(batch, dims[int(lab[2])], int(lab[2]))}")
        if tuple(left.shape) != _shape(batch, dim_l, int(lab[0])):
            raise RuntimeError(f"left_{lab}: expected shape {_shape(batch, dim_l, int(lab[0]))}")
    labels = (ctypes.c_int * n)(*[BEE_ORDER.index(lab) for lab, _, _ in terms])
    Ps = (ctypes.c_void_p * n)(*[P.data_ptr() for _, P, _ in terms])
    lefts = (ctypes.c_void_p * n)(*[left.data_ptr() for _, _, left in terms])
    with _on(dev):
        dx = torch.empty(_shape(batch, dims[rank_r], rank_r), dtype=torch.float32, device=dev)
        if dx.numel() > 0:
            L.check(_lib.mg_ant16_grad_x(rank_r, n, labels, Ps, lefts, _p(dys[0]), _p(dys[1]), _p(dys[2]), batch,
                                         dims[0], dims[1], dims[2], dim_l, 0, _p(dx), _stream()))
    return dx


def _ant16_one(label, P, x, dy, left=None):
    rl, rr, ro = (int(c) for c in label)
    batch = int(dy.size(0))
    dims = [0, 0, 0]
    dims[ro] = int(dy.size(1))
    if dims[rr] not in (0, int(x.size(1))):
        raise RuntimeError(f"x_{rr} and dy_{ro} of product {label} disagree on the channel count of rank {rr}")
    dims[rr] = int(x.size(1))
    if tuple(x.shape) != _shape(batch, dims[rr], rr):
        raise RuntimeError(f"x_{rr}: expected shape {_shape(batch, dims[rr], rr)}")
    if tuple(dy.shape) != _shape(batch, dims[ro], ro):
        raise RuntimeError(f"dy_{ro}: expected shape {_shape(batch, dims[ro], ro)}")
    if P is not None:
        dim_l = int(P.size(1))
        if tuple(P.shape) != (dims[ro], dim_l, dims[rr]):
            raise RuntimeError(f"P_{label}: expected shape {(dims[ro], dim_l, dims[rr])}")
    else:
        dim_l = int(left.size(1))
        if tuple(left.shape) != _shape(batch, dim_l, rl):
            raise RuntimeError(f"left_{label}: expected shape {_shape(batch, dim_l, rl)}")
    return batch, dims, dim_l


def ant16_grad_left(label, P, x, dy):
    """dleft[b,i,L] = sum_{o,j} P[o,i,j] C_L(x[b,j,:], dy[b,o,:]) of one product type
    (ant16_o*_backleft_cuda, extensions/codegen_tensops/codegen_tensops.cpp:892-1070)."""
    P, x, dy = P.contiguous(), x.contiguous(), dy.contiguous()
    batch, dims, dim_l = _ant16_one(label, P, x, dy)
    with _on(P.device):
        dleft = torch.empty(_shape(batch, dim_l, int(label[0])), dtype=torch.float32, device=P.device)
        if dleft.numel() > 0:
            L.check(_lib.mg_ant16_grad_left(BEE_ORDER.index(label), _p(P), _p(x), _p(dy), batch, dims[0], dims[1],
                                            dims[2], dim_l, _p(dleft), _stream()))
    return dleft


def ant16_grad_weight(label, left, x, dy):
    """dP[o,i,j] = sum_{b,O} dy[b,o,O] C_O(left[b,i,:], x[b,j,:]) of one product type; the rows are reduced in slices
    that are added in order, so the result is the same on every run
    (ant16_o*_wtsback_cuda, extensions/codegen_tensops/codegen_tensops.cpp:1142-1325)."""
    left, x, dy = left.contiguous(), x.contiguous(), dy.contiguous()
    batch, dims, dim_l = _ant16_one(label, None, x, dy, left=left)
    dim_r, dim_o = dims[int(label[1])], dims[int(label[2])]
    with _on(left.device):
        dP = torch.empty(dim_o, dim_l, dim_r, dtype=torch.float32, device=left.device)
        if dP.numel() > 0:
            nbytes = ctypes.c_size_t(0)
            L.check(_lib.mg_ant16_grad_weight_workspace_bytes(batch, dim_o, dim_l, dim_r, ctypes.byref(nbytes)))
            ws = torch.empty(nbytes.value, dtype=torch.uint8, device=left.device)
            L.check(_lib.mg_ant16_grad_weight(BEE_ORDER.index(label), _p(left), _p(x), _p(dy), batch, dims[0], dims[1],
                                              dims[2], dim_l, _p(ws), _p(dP), _stream()))
    return dP


def tensor_prod_bare(inds_l, inds_r, inds_o, x_l, x_r):
    """TensorProdBare.forward for operands (..., chan, (3,)^inds); leading dims must agree."""
    _check_input(x_l, "x_l")
    _check_input(x_r, "x_r")
    lead_l = tuple(x_l.shape[:x_l.dim() - inds_l])
    lead_r = tuple(x_r.shape[:x_r.dim() - inds_r])
    if lead_l != lead_r:
        raise RuntimeError(f"operands do not broadcast: {tuple(x_l.shape)} vs {tuple(x_r.shape)}")
    if tuple(x_l.shape[x_l.dim() - inds_l:]) != (3,) * inds_l or tuple(x_r.shape[x_r.dim() - inds_r:]) != (3,) * inds_r:
        raise RuntimeError("tensor axes must have size 3")
    n = 1
    for d in lead_l:
        n *= int(d)
    with _on(x_l.device):
        y = torch.empty(lead_l + (3,) * inds_o, dtype=torch.float32, device=x_l.device)
        L.check(_lib.mg_tensor_prod_bare(inds_l, inds_r, inds_o, _p(x_l), _p(x_r), n, 1, _p(y), _stream()))
    return y


def tensor_prods_supported(inds_l, inds_r, inds_o, dim_l, dim_r, rank, dim_o):
    """Whether tensor_prods (the one-launch TensorProds) takes this problem."""
    return bool(_lib.mg_tensor_prods_supported(inds_l, inds_r, inds_o, dim_l, dim_r, rank, dim_o))


def tensor_prods(inds_l, inds_r, inds_o, W_l, W_r, W_o, x_l, x_r):
    """lin_o(prod(lin_l(x_l), lin_r(x_r))) in one launch (managan/tensor_products.py:109-121); x: (..., dim, (3,)^inds),
    weights (out, in) with unit stride along a row."""
    for t, nm in ((W_l, "W_l"), (W_r, "W_r"), (W_o, "W_o"), (x_l, "x_l"), (x_r, "x_r")):
        if not t.is_cuda or t.dtype != torch.float32:
            raise RuntimeError(f"{nm} must be a float32 CUDA tensor")
    x_l, x_r = x_l.contiguous(), x_r.contiguous()
    lead = tuple(x_l.shape[:x_l.dim() - inds_l - 1])
    if lead != tuple(x_r.shape[:x_r.dim() - inds_r - 1]):
        raise RuntimeError(f"operands do not broadcast: {tuple(x_l.shape)} vs {tuple(x_r.shape)}")
    rank, dim_l = (int(v) for v in W_l.shape)
    dim_o = int(W_o.shape[0])
    dim_r = int(W_r.shape[1])
    if tuple(x_l.shape[len(lead):]) != (dim_l,) + (3,) * inds_l or tuple(x_r.shape[len(lead):]) != (dim_r,) + (3,) * inds_r \
            or int(W_r.shape[0]) != rank or int(W_o.shape[1]) != rank:
        raise RuntimeError("shape mismatch between weights and operands")
    Ws = [W if W.stride(1) == 1 and W.stride(0) % 4 == 0 and W.data_ptr() % 16 == 0 else W.contiguous() for W in (W_l, W_r, W_o)]
    rows = 1
    for d in lead:
        rows *= int(d)
    with _on(x_l.device):
        y = torch.empty(lead + (dim_o,) + (3,) * inds_o, dtype=torch.float32, device=x_l.device)
        L.check(_lib.mg_tensor_prods(inds_l, inds_r, inds_o, _p(Ws[0]), Ws[0].stride(0), _p(Ws[1]), Ws[1].stride(0),
                                     _p(Ws[2]), Ws[2].stride(0), _p(x_l), _p(x_r), rows, dim_l, dim_r, rank, dim_o,
                                     _p(y), _stream()))
    return y


def tensor_prods_avd(a, v_l, v_r):
    """(v_l . v_r, a v_r, v_l (x) v_r) in one pass; a: (..., C), v: (..., C, 3)."""
    for t, nm in ((a, "a"), (v_l, "v_l"), (v_r, "v_r")):
        _check_input(t, nm)
    if tuple(v_l.shape) != tuple(a.shape) + (3,) or tuple(v_r.shape) != tuple(v_l.shape):
        raise RuntimeError("shape mismatch")
    n = int(a.numel())
    dev = a.device
    with _on(dev):
        y0 = torch.empty_like(a)
        y1 = torch.empty_like(v_l)
        y2 = torch.empty(tuple(v_l.shape) + (3,), dtype=torch.float32, device=dev)
        L.check(_lib.mg_tensor_prods_avd(_p(a), _p(v_l), _p(v_r), n, 1, _p(y0), _p(y1), _p(y2), _stream()))
    return y0, y1, y2


ACT_NONE, ACT_SILU, ACT_LEAKY = 0, 1, 2
LINEAR_FP32_MFMA, LINEAR_BF16X3, LINEAR_F16X2 = 0, 1, 2


def set_linear_mode(mode):
    """0: fp32 MFMA; 1: bf16x3-split operands on the bf16 MFMA (fp32-class accuracy, faster);
    2 (default): two-piece fp16 split with per-row scales where the layer shape allows (a few fp32
    ulps per product, half the matrix work of mode 1), mode 1 elsewhere."""
    L.check(_lib.mg_set_linear_mode(int(mode)))


def get_linear_mode():
    return int(_lib.mg_get_linear_mode())


_cache_epoch = 0


def invalidate_weight_caches():
    """Forget everything kept per weight tensor (pre-split planes, norms, permuted / padded / concatenated copies, here
    and in the layers).  The caches notice a new tensor object and an in-place update through the tensor itself (its
    version counter); a write that bypasses the counter (`param.data.mul_(...)`, a raw pointer) needs this call."""
    global _cache_epoch
    _cache_epoch += 1


def tensor_version(t):
    """t's version counter (with the epoch of invalidate_weight_caches in the high bits), or -1 for an inference
    tensor, which has none: a result cached for -1 is never reused."""
    return -1 if t.is_inference() else (_cache_epoch << 40) | t._version


def stamp(tensors, keep_unversioned=False):
    """What a cache of something computed from these tensors compares: objects, versions, addresses.  With an inference
    tensor among them (no version counter) the stamp equals no other, so the cached value is rebuilt; with
    keep_unversioned such a tensor is stamped by object, address and the epoch of invalidate_weight_caches instead
    (for decisions that are expensive to re-make and that a caller who writes such tensors in place can reset)."""
    st = tuple((id(t), tensor_version(t), t.data_ptr()) for t in tensors)
    if all(v[1] >= 0 for v in st):
        return st
    return tuple((i, v if v >= 0 else -1 - _cache_epoch, p) for i, v, p in st) if keep_unversioned else (object(),)


@contextlib.contextmanager
def derived_tensors():
    """For tensors computed from parameters and kept across calls: nothing recorded for autograd, and ordinary tensors
    (with the version counter the caches check) also when the caller runs under torch.inference_mode()."""
    with torch.inference_mode(False), torch.no_grad():
        yield


_packed_cache = {}


def _packed(W, kind):
    """Pre-split planes of W for the packed GEMM entry points.  Cached per tensor OBJECT (weak
    reference) and version counter, so parameters are packed once and re-packed after an in-place
    update; a new tensor that happens to reuse a freed address never hits a stale entry.  A view
    (the transposed weight of every input-gradient GEMM is a fresh view object of the parameter) is
    cached under the tensor it is a view of, with its offset, shape and strides."""
    owner = W._base if W._base is not None else W
    key = (id(owner), kind, int(W.storage_offset()), tuple(W.shape), tuple(W.stride()))
    hit = _packed_cache.get(key)
    version = tensor_version(owner)
    if hit is not None and version >= 0 and hit[0]() is owner and hit[1] == version and hit[2] == owner.data_ptr():
        return hit[3]
    dim_out, dim_in = int(W.size(0)), int(W.size(1))
    nbytes = ctypes.c_size_t(0)
    size_fn, pack_fn = ((_lib.mg_linear_packed_weight_bytes, _lib.mg_linear_pack_weight) if kind == "bf16x3" else
                        (_lib.mg_linear_f16x2_packed_weight_bytes, _lib.mg_linear_f16x2_pack_weight))
    L.check(size_fn(dim_in, dim_out, ctypes.byref(nbytes)))
    with _on(W.device):
        packed = torch.empty(nbytes.value, dtype=torch.uint8, device=W.device)
        L.check(pack_fn(_p(W), int(W.stride(0)), int(W.stride(1)), dim_in, dim_out, _p(packed), _stream()))
    if len(_packed_cache) > 4096:
        _packed_cache.clear()
    # the entry (and the device memory of its planes) goes when the tensor it was packed from does
    _packed_cache[key] = (weakref.ref(owner, lambda _, key=key: _packed_cache.pop(key, None)),
                          version, owner.data_ptr(), packed)
    return packed


_padded_cache = {}


def zero_padded_columns(W, k_pad):
    """W (dim_out, dim_in) with zero columns appended up to k_pad; cached per parameter object and version."""
    if int(W.size(1)) == k_pad:
        return W
    key = (id(W), k_pad)
    hit = _padded_cache.get(key)
    if hit is not None and hit[0]() is W and hit[1] == tensor_version(W) >= 0 and hit[2] == W.data_ptr():
        return hit[3]
    with derived_tensors():
        Wp = torch.nn.functional.pad(W.detach(), (0, k_pad - int(W.size(1)))).contiguous()
    if len(_padded_cache) > 256:
        _padded_cache.clear()
    _padded_cache[key] = (weakref.ref(W), tensor_version(W), W.data_ptr(), Wp)
    return Wp


def packed_weight(W):
    """bf16x3 planes of W for mg_tensor_linear_packed."""
    return _packed(W, "bf16x3")


def packed_weight_f16x2(W):
    """fp16 hi/lo planes + per-row inverse scales of W for mg_tensor_linear_f16x2."""
    return _packed(W, "f16x2")


def row_absmax(x):
    """(rows, dim) -> (rows, 1): max_i |x[r, i]|, the row bounds mg_tensor_linear_f16x2 scales by."""
    _check_input(x, "x")
    if x.dim() != 2:
        raise RuntimeError("x must have two dims")
    with _on(x.device):
        out = torch.empty(x.size(0), 1, dtype=torch.float32, device=x.device)
        L.check(_lib.mg_row_absmax(_p(x), int(x.size(0)), int(x.size(1)), _p(out), _stream()))
    return out


def linear_f64(W, bias, x, act=ACT_NONE):
    """act(x W^T + bias) in float64 arithmetic: W (dim_out, dim_in) and bias float32 parameters, x (rows, dim_in) and
    the result float64.  For measuring approximations of a float32 MLP against exact arithmetic, not a compute path."""
    _check_input(W, "W")
    _check_input(x, "x", torch.float64)
    if bias is not None:
        _check_input(bias, "bias")
    if x.dim() != 2 or W.dim() != 2 or W.size(1) != x.size(1) or (bias is not None and bias.numel() != W.size(0)):
        raise RuntimeError("linear_f64: x (rows, dim_in), W (dim_out, dim_in), bias (dim_out)")
    with _on(x.device):
        y = torch.empty(x.size(0), W.size(0), dtype=torch.float64, device=x.device)
        L.check(_lib.mg_linear_f64(_p(W), _p(bias) if bias is not None else None, _p(x), int(x.size(0)),
                                   int(W.size(1)), int(W.size(0)), int(act), _p(y), _stream()))
    return y


_bound_cache = {}


def linear_in_unit_bound(device):
    """(1, 1) bound for inputs whose entries are at most 1 in magnitude (sines, cosines, one-hots)."""
    key = ("unit", str(device))
    hit = _bound_cache.get(key)
    if hit is None:
        hit = _bound_cache[key] = torch.ones(1, 1, dtype=torch.float32, device=device)
    return hit


def linear_out_bound(W, bias, in_bound):
    """Upper bound of |act(x W^T + bias)| per row, given upper bounds in_bound ((rows, 1) or (1, 1);
    None: entries of x are at most 1 in magnitude) of |x| per row, for any act with |act(z)| <= |z|
    (identity, SiLU, LeakyReLU):  |y[r, o]| <= in_bound[r] * max_o sum_i |W[o, i]| + max_o |bias[o]|.
    The two weight norms are cached per parameter object and version (device tensors; no host
    synchronisation).  These bounds feed mg_tensor_linear_f16x2, whose accuracy does not depend on
    how tight they are as long as they stay within a factor 2^14 of the true row maxima."""
    if isinstance(in_bound, ScaledBound):
        return in_bound.through(*linear_out_bound_factors(W, bias))
    if in_bound is None:
        in_bound = linear_in_unit_bound(W.device)
    key = ("norms", id(W), id(bias))
    hit = _bound_cache.get(key)
    w_ver, b_ver = tensor_version(W), (tensor_version(bias) if bias is not None else 0)
    if (hit is None or min(w_ver, b_ver) < 0 or hit[0]() is not W or hit[1] != w_ver
            or (bias is not None and (hit[2]() is not bias or hit[3] != b_ver))):
        with derived_tensors():
            l1 = W.detach().abs().sum(dim=1).amax().reshape(1, 1)
            bmax = bias.detach().abs().amax().reshape(1, 1) if bias is not None else torch.zeros_like(l1)
        hit = (weakref.ref(W), w_ver, weakref.ref(bias) if bias is not None else None, b_ver, l1, bmax, {})
        if len(_bound_cache) > 1024:
            _bound_cache.clear()
        _bound_cache[key] = hit
    l1, bmax, per_input = hit[4], hit[5], hit[6]
    if in_bound.numel() == 1:
        # a constant input bound (cached tensor object) gives a constant output bound: computed once
        memo = per_input.get(id(in_bound))
        if memo is not None and memo[0]() is in_bound:
            return memo[1]
        out = torch.addcmul(bmax, in_bound.reshape(1, 1), l1)
        if len(per_input) > 16:
            per_input.clear()
        per_input[id(in_bound)] = (weakref.ref(in_bound), out)
        return out
    if in_bound.dim() == 2 and in_bound.size(1) > 1:           # partial maxima per row: the largest counts
        in_bound = in_bound.amax(dim=1, keepdim=True)
    return torch.addcmul(bmax, in_bound.reshape(-1, 1), l1)


_factor_cache = {}


def linear_out_bound_factors(W, bias):
    """(max_o sum_i |W[o, i]|, max_o |bias[o]|) as host floats: |act(x W^T + bias)| <= |x|max * first + second.
    Read back once per version of the parameters (one host synchronisation then, none afterwards)."""
    key = (id(W), id(bias))
    hit = _factor_cache.get(key)
    w_ver, b_ver = tensor_version(W), (tensor_version(bias) if bias is not None else 0)
    if (hit is None or min(w_ver, b_ver) < 0 or hit[0]() is not W or hit[1] != w_ver
            or (bias is not None and (hit[2]() is not bias or hit[3] != b_ver))):
        with derived_tensors():
            both = torch.stack([W.detach().abs().sum(dim=1).amax(),
                                bias.detach().abs().amax() if bias is not None else W.new_zeros(())]).tolist()
        # a little above the float32 value: the product with a row maximum must not round below the true bound
        hit = (weakref.ref(W), w_ver, weakref.ref(bias) if bias is not None else None, b_ver,
               both[0] * (1.0 + 1e-6), both[1] * (1.0 + 1e-6))
        if len(_factor_cache) > 1024:
            _factor_cache.clear()
        _factor_cache[key] = hit
    return hit[4], hit[5]


def f16x2_supported(rows, dim_in, dim_out, x):
    return dim_in % 32 == 0 and dim_in >= 64 and dim_out >= 8 and rows >= 256 and x.data_ptr() % 16 == 0


class ScaledBound:
    """Row bounds given as mul * base + add: base (rows, parts) row maxima as some kernel emitted them, mul and add host
    floats.  A chain of layers whose bounds follow from the weight norms (linear_out_bound_factors) carries one array
    this way, without a launch per layer to update it; tensor() forms the array for a consumer that wants one."""
    __slots__ = ("base", "mul", "add")

    def __init__(self, base, mul=1.0, add=0.0):
        self.base, self.mul, self.add = base, float(mul), float(add)

    def through(self, l1, bmax):
        """The bound after a linear layer with these norms (and any act with |act(z)| <= |z|)."""
        return ScaledBound(self.base, self.mul * l1, self.add * l1 + bmax)

    def tensor(self):
        b = self.base if self.base.size(1) == 1 else self.base.amax(dim=1, keepdim=True)
        return b * self.mul + self.add


def tensor_linear_f16x2(W, x, x_rowmax=None, bias=None, act=ACT_NONE, out=None, accumulate=False, out_comps=1,
                        want_rowmax=False, rows_per_bound=1):
    """y = act(x W^T + bias) for plain rows x (rows, dim_in) through the two-piece fp16 split.
    x_rowmax (rows, parts), or (1, parts) for one bound shared by all rows: upper bounds of the
    row maxima of |x| (None: computed here), or a ScaledBound of such an array.
    Returns y, or (y, y_rowmax) with want_rowmax=True."""
    bound_mul, bound_add = 1.0, 0.0
    if isinstance(x_rowmax, ScaledBound):
        x_rowmax, bound_mul, bound_add = x_rowmax.base, x_rowmax.mul, x_rowmax.add
    _check_input(x, "x")
    if x.dim() != 2 or W.dim() != 2 or x.size(1) != W.size(1):
        raise RuntimeError("expected x (rows, dim_in) and W (dim_out, dim_in)")
    rows, dim_in, dim_out = int(x.size(0)), int(W.size(1)), int(W.size(0))
    if x_rowmax is None:
        x_rowmax = row_absmax(x)
    _check_input(x_rowmax, "x_rowmax")
    if x_rowmax.dim() != 2 or (x_rowmax.size(0) != 1 and x_rowmax.size(0) * rows_per_bound != rows):
        raise RuntimeError("x_rowmax must be (rows / rows_per_bound, parts) or (1, parts)")
    rowmax_stride = int(x_rowmax.size(1)) if x_rowmax.size(0) > 1 or rows == rows_per_bound else 0
    if bias is not None:
        _check_input(bias, "bias")
        if bias.numel() != dim_out:
            raise RuntimeError("bias size mismatch")
    if rows % out_comps != 0:
        raise RuntimeError("rows must be a multiple of out_comps")
    y_shape = [rows, dim_out] if out_comps == 1 else [rows // out_comps, dim_out, out_comps]
    with _on(x.device):
        if out is None:
            y = torch.empty(y_shape, dtype=torch.float32, device=x.device)
        else:
            _check_input(out, "out")
            if out.numel() != rows * dim_out:
                raise RuntimeError("out has wrong size")
            y = out
        ymax = None
        if want_rowmax:
            if out_comps != 1:
                raise RuntimeError("row maxima are only produced for out_comps == 1")
            parts = int(_lib.mg_tensor_linear_f16x2_rowmax_parts(rows, dim_in, dim_out))
            ymax = torch.empty(rows, parts, dtype=torch.float32, device=x.device)
        L.check(_lib.mg_tensor_linear_f16x2_scaled_bound(
            _p(packed_weight_f16x2(W)), _p(x), _p(x_rowmax), int(x_rowmax.size(1)), rowmax_stride, int(rows_per_bound),
            rows, dim_in, dim_out, _p(bias), int(act), int(bool(accumulate)), int(out_comps), _p(y), _p(ymax),
            bound_mul, bound_add, _stream()))
    return (y, ymax) if want_rowmax else y


LAYOUT_CHAN_COMP, LAYOUT_COMP_CHAN = 0, 1


def components_as_rows(inds, x):
    """x (..., dim_in, (3,)^inds) in the reference's layout -> (x2, x2max): one plain GEMM row per (row, component)
    with the channels zero-padded to a power of two, and the row maxima of |x2| -- what tensor_linear_fwd forms for
    itself when it sends such an input through the split-fp16 path, for callers that apply several weights to the same
    x (x_rows= of tensor_linear_fwd).  None when that path would not be taken for this input."""
    _check_input(x, "x")
    if inds < 1 or inds > 2 or x.dim() < 1 + inds:
        return None
    T = 3 ** inds
    dim_in = int(x.size(x.dim() - 1 - inds))
    rows = x.numel() // (dim_in * T) if dim_in else 0
    k_pad = (dim_in + 31) // 32 * 32
    if get_linear_mode() != LINEAR_F16X2 or rows * T < 32768 or k_pad > 256 or k_pad & (k_pad - 1):
        return None
    with _on(x.device):
        x2 = torch.empty(rows * T, k_pad, dtype=torch.float32, device=x.device)
        x2max = torch.empty(rows * T, 1, dtype=torch.float32, device=x.device)
        L.check(_lib.mg_components_to_rows(_p(x), rows, dim_in, T, k_pad, _p(x2), _p(x2max), _stream()))
    return x2, x2max


def tensor_linear_fwd(inds, W, x, bias=None, act=ACT_NONE, out=None, accumulate=False,
                      x_layout=LAYOUT_CHAN_COMP, y_layout=LAYOUT_CHAN_COMP, row_bound=None, rows_per_bound=1,
                      want_rowmax=False, x_rows=None):
    """y[..., o, t] = act(sum_i W[o, i] x[..., i, t] + bias[o]); W may have any strides.
    Layout 0 stores a tensor as (..., chan, (3,)^inds) like the reference; layout 1 is
    component-major (..., 3^inds, chan), the layout the fused edge kernels read and write.
    row_bound ((rows of the GEMM) / rows_per_bound, parts): upper bounds of the row maxima of |x| from
    the kernel that produced x, used by the split-fp16 matrix path instead of a pass over x.
    want_rowmax: return (y, rowmax) with rowmax ((GEMM rows), parts) partial row maxima of |y| when the kernel
    that ran can emit them (plain-row output through the split-fp16 path), else (y, None).
    x_rows: components_as_rows(inds, x) of this same x, if the caller has it (None is allowed)."""
    if not W.is_cuda:
        raise RuntimeError("W must be a CUDA tensor")
    _check_input(x, "x")
    if W.dtype != torch.float32:
        raise RuntimeError("W must be float32")
    if W.dim() != 2:
        raise RuntimeError("expected W to be a matrix (2 dims)")
    if inds > 2 or inds < 0:
        raise RuntimeError("tensor_linear currently only supports a number of indices up to 2. "
                           "go edit the code to add more (easy with copy/paste).")
    dim_out, dim_in = int(W.size(0)), int(W.size(1))
    T = 3 ** inds
    if x_layout == LAYOUT_CHAN_COMP:
        batch_dims = x.dim() - (1 + inds)
        if batch_dims < 0:
            raise RuntimeError("x has too few dims")
        if x.size(batch_dims) != dim_in:
            raise RuntimeError("channel dim size mismatch for x")
        for i in range(batch_dims + 1, batch_dims + inds + 1):
            if x.size(i) != 3:
                raise RuntimeError("expected tensor index dim to be 3d for input x")
    else:
        batch_dims = x.dim() - 2
        if batch_dims < 0 or x.size(-1) != dim_in or x.size(-2) != T:
            raise RuntimeError("component-major x must have shape (..., 3^inds, dim_in)")
    lead = [int(d) for d in x.shape[:batch_dims]]
    rows = 1
    for d in lead:
        rows *= d
    y_shape = lead + ([dim_out] + [3] * inds if y_layout == LAYOUT_CHAN_COMP else [T, dim_out])
    if bias is not None:
        _check_input(bias, "bias")
        if bias.numel() != dim_out:
            raise RuntimeError("bias size mismatch")
    with _on(x.device):
        if out is None:
            y = torch.empty(y_shape, dtype=torch.float32, device=x.device)
        else:
            _check_input(out, "out")
            if list(out.shape) != y_shape:
                raise RuntimeError("out has wrong shape")
            y = out
        plain_rows = inds == 0 or x_layout == LAYOUT_COMP_CHAN
        mode = get_linear_mode()
        wide = (plain_rows and dim_in % 32 == 0 and dim_in >= 64 and dim_out >= 64 and rows * T >= 1024
                and x.data_ptr() % 16 == 0)
        out_comps = 1 if (inds == 0 or y_layout == LAYOUT_COMP_CHAN) else T
        ymax = None

        def rowmax_buffer(k_in):
            if not (want_rowmax and out_comps == 1 and not accumulate):
                return None
            parts = int(_lib.mg_tensor_linear_f16x2_rowmax_parts(rows * T, k_in, dim_out))
            return torch.empty(rows * T, parts, dtype=torch.float32, device=x.device)
        if (mode == LINEAR_F16X2 and inds > 0 and x_layout == LAYOUT_CHAN_COMP and rows * T >= 32768 and dim_out >= 64
                and row_bound is None and (y_layout == LAYOUT_COMP_CHAN or not (want_rowmax or accumulate or bias is not None
                                                                                or act != ACT_NONE))):
            # (row, chan, comp) -> (row, comp, chan) rows (K zero-padded to a multiple of 32), then the plain-row
            # matrix path: its component-major output is written at the full store rate, which the generic
            # kernel's layout mapping is not; with the reference's output layout its component epilogue still
            # beats the generic kernel (61 against 104 us for 16384 x 128 x 3 -> 384)
            k_pad = (dim_in + 31) // 32 * 32
            if x_rows is not None and tuple(x_rows[0].shape) == (rows * T, k_pad):
                x2, x2max = x_rows
            elif k_pad <= 256 and k_pad & (k_pad - 1) == 0:
                # transposition, padding and the row maxima in one pass
                x2 = torch.empty(rows * T, k_pad, dtype=torch.float32, device=x.device)
                x2max = torch.empty(rows * T, 1, dtype=torch.float32, device=x.device)
                L.check(_lib.mg_components_to_rows(_p(x), rows, dim_in, T, k_pad, _p(x2), _p(x2max), _stream()))
            else:
                xt = x.reshape(rows, dim_in, T).transpose(1, 2)
                xt = torch.nn.functional.pad(xt, (0, k_pad - dim_in)) if k_pad != dim_in else xt.contiguous()
                x2 = xt.reshape(rows * T, k_pad)
                x2max = row_absmax(x2)
            Wp = zero_padded_columns(W, k_pad)
            ymax = rowmax_buffer(k_pad)
            L.check(_lib.mg_tensor_linear_f16x2(_p(packed_weight_f16x2(Wp)), _p(x2), _p(x2max), 1, 1, 1,
                                                rows * T, k_pad, dim_out, _p(bias), int(act), int(bool(accumulate)),
                                                out_comps, _p(y), _p(ymax), _stream()))
        elif (plain_rows and mode == LINEAR_F16X2 and f16x2_supported(rows * T, dim_in, dim_out, x)):
            x2 = x.reshape(rows * T, dim_in)
            if row_bound is None:
                row_bound, rows_per_bound = row_absmax(x2), 1
            elif row_bound.dim() != 2 or row_bound.size(0) * rows_per_bound != rows * T:
                raise RuntimeError("row_bound must be (rows / rows_per_bound, parts)")
            ymax = rowmax_buffer(dim_in)
            L.check(_lib.mg_tensor_linear_f16x2(_p(packed_weight_f16x2(W)), _p(x2), _p(row_bound),
                                                int(row_bound.size(1)), int(row_bound.size(1)), int(rows_per_bound),
                                                rows * T,
                                                dim_in, dim_out, _p(bias), int(act), int(bool(accumulate)),
                                                out_comps, _p(y), _p(ymax), _stream()))
        elif wide and mode == LINEAR_BF16X3:
            L.check(_lib.mg_tensor_linear_packed(_p(packed_weight(W)), _p(x), rows * T, dim_in, dim_out, _p(bias),
                                                 int(act), int(bool(accumulate)), out_comps, _p(y), _stream()))
        else:
            L.check(_lib.mg_tensor_linear_layout(inds, _p(W), int(W.stride(0)), int(W.stride(1)), _p(x), rows,
                                                 dim_in, dim_out, _p(bias), int(act), int(bool(accumulate)),
                                                 int(x_layout), int(y_layout), _p(y), _stream()))
    return (y, ymax) if want_rowmax else y


def tensor_linear_wgrad(inds, dy, x, dy_bound=None, x_bound=None, want_bias=False):
    """dW[o, i] = sum over rows and components of dy[.., o, :] x[.., i, :].  Plain rows (inds = 0) of the sizes
    mg_tensor_linear_wgrad_f16x2 takes go through it while the linear mode is the split-fp16 one; dy_bound / x_bound
    (float tensors of any shape whose largest magnitude bounds |dy| / |x|, e.g. row maxima that the caller already
    holds) save it a pass over the operand.  want_bias (inds = 0): returns (dW, db) with db[o] = sum over rows of
    dy[.., o], from the same pass where the kernel offers it."""
    _check_input(dy, "dy")
    _check_input(x, "x")
    if want_bias and inds != 0:
        raise RuntimeError("the bias gradient is defined for plain rows only")
    batch_dims = x.dim() - (1 + inds)
    dim_in, dim_out = int(x.size(batch_dims)), int(dy.size(batch_dims))
    rows = 1
    for i in range(batch_dims):
        rows *= int(x.size(i))
    with _on(x.device):
        dW = torch.empty(dim_out, dim_in, dtype=torch.float32, device=x.device)
        db = None
        nbytes = ctypes.c_size_t(0)

        def workspace(n_rows, n_in, n_out):
            L.check(_lib.mg_tensor_linear_wgrad_workspace_bytes(n_rows, n_in, n_out, ctypes.byref(nbytes)))
            return torch.empty(nbytes.value, dtype=torch.uint8, device=x.device)
        if (inds == 0 and get_linear_mode() == LINEAR_F16X2 and x.data_ptr() % 16 == 0 and dy.data_ptr() % 16 == 0
                and _lib.mg_tensor_linear_wgrad_f16x2_supported(rows, dim_in, dim_out)):
            for b, name in ((dy_bound, "dy_bound"), (x_bound, "x_bound")):
                if b is not None:
                    _check_input(b, name)
            if want_bias:
                db = torch.empty(dim_out, dtype=torch.float32, device=x.device)
            ws = workspace(rows, dim_in, dim_out)
            L.check(_lib.mg_tensor_linear_wgrad_f16x2(
                _p(dy), _p(x), _p(dy_bound), 0 if dy_bound is None else dy_bound.numel(),
                _p(x_bound), 0 if x_bound is None else x_bound.numel(), rows, dim_in, dim_out, _p(ws), _p(dW), _p(db),
                _stream()))
        elif (inds > 0 and get_linear_mode() == LINEAR_F16X2 and rows * 3 ** inds >= 4096
              and max(dim_in, dim_out) <= 256):
            # (row, chan, comp) -> one plain row per (row, comp), channels zero-padded to a power of two: the sum over
            # rows and components is then the plain-row weight gradient, on the matrix cores; the transposition
            # also yields the row maxima the kernel scales by
            T = 3 ** inds

            def as_rows(t, dim):
                pad = max(32, 1 << (dim - 1).bit_length())
                out = torch.empty(rows * T, pad, dtype=torch.float32, device=t.device)
                bound = torch.empty(rows * T, 1, dtype=torch.float32, device=t.device)
                L.check(_lib.mg_components_to_rows(_p(t), rows, dim, T, pad, _p(out), _p(bound), _stream()))
                return out, bound, pad
            dy2, dy2_bound, o_pad = as_rows(dy, dim_out)
            x2, x2_bound, i_pad = as_rows(x, dim_in)
            ws = workspace(rows * T, i_pad, o_pad)
            dW_pad = dW if (o_pad, i_pad) == (dim_out, dim_in) else torch.empty(o_pad, i_pad, dtype=torch.float32,
                                                                                device=x.device)
            L.check(_lib.mg_tensor_linear_wgrad_f16x2(_p(dy2), _p(x2), _p(dy2_bound), rows * T, _p(x2_bound), rows * T,
                                                      rows * T, i_pad, o_pad, _p(ws), _p(dW_pad), None, _stream()))
            if dW_pad is not dW:
                dW = dW_pad[:dim_out, :dim_in].contiguous()
        else:
            ws = workspace(rows, dim_in, dim_out)
            L.check(_lib.mg_tensor_linear_wgrad(inds, _p(dy), _p(x), rows, dim_in, dim_out, _p(ws), _p(dW), _stream()))
            if want_bias:
                db = dy.reshape(-1, dim_out).sum(0)
    return (dW, db) if want_bias else dW


# ------------------------------------------------- bf16-storage configuration
def _check_bf16(t, name):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if t.dtype != torch.bfloat16:
        raise RuntimeError(f"{name} must be bfloat16")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def tensor_linear_bf16(W, x, bias=None, act=ACT_NONE, out=None, accumulate=False, out_comps=1,
                       out_dtype=torch.bfloat16):
    """y = act(bias + x W^T) on bf16 storage: x (rows, dim_in) bfloat16, W (dim_out, dim_in) float32
    parameter (split once, 16 significand bits used), fp32 accumulation, y bfloat16 or float32.
    out_comps = T > 1 treats consecutive groups of T rows as the components of one row and writes
    y as (rows / T, dim_out, T)."""
    _check_bf16(x, "x")
    if W.dim() != 2 or W.dtype != torch.float32 or not W.is_cuda:
        raise RuntimeError("W must be a float32 CUDA matrix")
    if x.dim() != 2 or x.size(1) != W.size(1):
        raise RuntimeError("x must have shape (rows, dim_in)")
    rows, dim_in, dim_out = int(x.size(0)), int(W.size(1)), int(W.size(0))
    if dim_in % 32:
        raise RuntimeError("dim_in must be a multiple of 32 on the bf16 path")
    if rows % out_comps:
        raise RuntimeError("rows must be a multiple of out_comps")
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_contiguous() or bias.numel() != dim_out):
        raise RuntimeError("bias must be a contiguous float32 tensor of dim_out elements")
    shape = (rows, dim_out) if out_comps == 1 else (rows // out_comps, dim_out, out_comps)
    with _on(x.device):
        if out is None:
            if accumulate:
                raise RuntimeError("accumulate needs out")
            out = torch.empty(shape, dtype=out_dtype, device=x.device)
        elif tuple(out.shape) != shape or not out.is_contiguous() or out.dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError("out has the wrong shape, dtype or layout")
        L.check(_lib.mg_tensor_linear_bf16(_p(packed_weight(W)), _p(x), rows, dim_in, dim_out,
                                           _p(bias) if bias is not None else None, int(act), int(bool(accumulate)),
                                           int(out_comps), int(out.dtype == torch.bfloat16), _p(out), _stream()))
    return out


def bee_message_bf16(row_ptr, dst, rhat, enc, La, Lv, Ld, enc_W, enc_b, node_order=None):
    """bee_message on bf16 storage: La (N,chan), Lv (N,3,chan), Ld (N,9,chan) bfloat16 ->
    P0 (E,3,chan), S1 (N,3,5,chan), S2 (N,9,5,chan) bfloat16."""
    for t, nm in ((La, "La"), (Lv, "Lv"), (Ld, "Ld")):
        _check_bf16(t, nm)
    for t, nm in ((rhat, "rhat"), (enc, "enc"), (enc_W, "enc_W"), (enc_b, "enc_b")):
        _check_input(t, nm)
    N, chan = int(La.size(0)), int(La.size(1))
    E = int(dst.numel())
    if tuple(Lv.shape) != (N, 3, chan) or tuple(Ld.shape) != (N, 9, chan):
        raise RuntimeError("Lv, Ld must be (nodes, 3, chan), (nodes, 9, chan)")
    if tuple(rhat.shape) != (E, 3) or tuple(enc.shape) != (E, 8) or tuple(enc_W.shape) != (chan, 8):
        raise RuntimeError("rhat (E,3), enc (E,8), enc_W (chan,8) expected")
    if row_ptr.dtype != torch.int32 or dst.dtype != torch.int32 or row_ptr.numel() != N + 1:
        raise RuntimeError("row_ptr (nodes+1) and dst must be int32")
    if node_order is not None and (node_order.dtype != torch.int32 or node_order.numel() != N):
        raise RuntimeError("node_order must be int32 with one entry per node")
    with _on(La.device):
        P0 = torch.empty(E, 3, chan, dtype=torch.bfloat16, device=La.device)
        S1 = torch.empty(N, 3, 5, chan, dtype=torch.bfloat16, device=La.device)
        S2 = torch.empty(N, 9, 5, chan, dtype=torch.bfloat16, device=La.device)
        L.check(_lib.mg_bee_message_bf16(_p(row_ptr), _p(dst), _p(node_order) if node_order is not None else None,
                                         N, E, _p(rhat), _p(enc), _p(La), _p(Lv), _p(Ld), chan, _p(enc_W),
                                         _p(enc_b), _p(P0), _p(S1), _p(S2), _stream()))
    return P0, S1, S2


def bee_node_products(l0, l1, l2, r0, r1, r2, want_node_max=False):
    """The 13 products on node rows in component-major layout (float32 or bfloat16 storage):
    l0/r0 (N,chan), l1/r1 (N,3,chan), l2/r2 (N,9,chan) -> P0 (N,3,chan), P1 (N,3,5,chan), P2 (N,9,5,chan)
    (+ node_max (N, chan/64): partial maxima of all products per node, float32 operands with
    chan % 64 == 0 only; None otherwise)."""
    bf = l0.dtype == torch.bfloat16
    for t, nm in ((l0, "l0"), (l1, "l1"), (l2, "l2"), (r0, "r0"), (r1, "r1"), (r2, "r2")):
        (_check_bf16 if bf else _check_input)(t, nm)
    N, chan = int(l0.size(0)), int(l0.size(1))
    for t, comps in ((l0, None), (r0, None), (l1, 3), (r1, 3), (l2, 9), (r2, 9)):
        want = (N, chan) if comps is None else (N, comps, chan)
        if tuple(t.shape) != want:
            raise RuntimeError("operands must be (nodes, chan), (nodes, 3, chan), (nodes, 9, chan)")
    with _on(l0.device):
        P0 = torch.empty(N, 3, chan, dtype=l0.dtype, device=l0.device)
        P1 = torch.empty(N, 3, 5, chan, dtype=l0.dtype, device=l0.device)
        P2 = torch.empty(N, 9, 5, chan, dtype=l0.dtype, device=l0.device)
        node_max = None
        if bf:
            L.check(_lib.mg_bee_node_products_bf16(N, chan, _p(l0), _p(l1), _p(l2), _p(r0), _p(r1), _p(r2), _p(P0),
                                                   _p(P1), _p(P2), _stream()))
        else:
            if want_node_max and chan % 64 == 0:
                node_max = torch.empty(N, chan // 64, dtype=torch.float32, device=l0.device)
            L.check(_lib.mg_bee_node_products(N, chan, _p(l0), _p(l1), _p(l2), _p(r0), _p(r1), _p(r2), _p(P0), _p(P1),
                                              _p(P2), _p(node_max), _stream()))
    return (P0, P1, P2, node_max) if want_node_max else (P0, P1, P2)


def bf16_rowsum_supported(rows, dim_in, dim_out):
    return dim_out % 128 == 0 and dim_in % 32 == 0 and rows >= 4096


def tensor_linear_bf16_rowsum(W, x, row_ptr, seg, n_out, bias=None, act=ACT_NONE, scale=1.0, want_rows=False):
    """(out, y): out (n_out, dim_out) float32 = scale * sum over the rows of each segment of the bfloat16-rounded
    act(bias + W x[r]); y (rows, dim_out) bfloat16 with want_rows, else None.  x (rows, dim_in) bfloat16 sorted by
    segment: seg (rows,) int32 ascending, row_ptr its CSR form."""
    _check_bf16(x, "x")
    _check_input(W, "W")
    for t, nm in ((row_ptr, "row_ptr"), (seg, "seg")):
        _check_input(t, nm, torch.int32)
    if x.dim() != 2 or W.dim() != 2 or x.size(1) != W.size(1):
        raise RuntimeError("x must have shape (rows, dim_in) and W (dim_out, dim_in)")
    rows, dim_in, dim_out = int(x.size(0)), int(W.size(1)), int(W.size(0))
    if seg.numel() != rows or row_ptr.numel() != n_out + 1:
        raise RuntimeError("seg must have one entry per row and row_ptr n_out + 1 entries")
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_contiguous() or bias.numel() != dim_out):
        raise RuntimeError("bias must be a contiguous float32 tensor of dim_out elements")
    nbytes = ctypes.c_size_t(0)
    L.check(_lib.mg_tensor_linear_bf16_rowsum_workspace_bytes(rows, dim_out, ctypes.byref(nbytes)))
    with _on(x.device):
        out = torch.empty(n_out, dim_out, dtype=torch.float32, device=x.device)
        y = torch.empty(rows, dim_out, dtype=torch.bfloat16, device=x.device) if want_rows else None
        work = torch.empty(nbytes.value // 4, dtype=torch.float32, device=x.device)
        L.check(_lib.mg_tensor_linear_bf16_rowsum(_p(packed_weight(W)), _p(x), rows, dim_in, dim_out, _p(bias), int(act),
                                                  _p(row_ptr), _p(seg), int(n_out), float(scale), _p(work), _p(y),
                                                  _p(out), _stream()))
    return out, y


def mlp_chain_bf16_supported(rows, dim_in, dim_psi, hidden):
    return dim_psi == 128 and hidden == 256 and dim_in % 32 == 0 and rows >= 4096


def mlp_chain_bf16(Y, x, W1, b1, W2, b2, row_ptr, seg, n_out, act=ACT_LEAKY):
    """(sum_psi (n_out, 128), sum_h2 (n_out, 256)) float32: the sums over the rows of each segment of the
    bfloat16-rounded psi = Y x and h2 = act(b2 + W2 act(b1 + W1 psi)), every layer rounded to bfloat16 as
    tensor_linear_bf16 stores it, in one kernel that writes no per-row tensor.  x (rows, dim_in) bfloat16 sorted
    by segment (seg ascending, row_ptr its CSR form); Y (128, dim_in), W1 (256, 128), W2 (256, 256) float32."""
    _check_bf16(x, "x")
    for t, nm in ((Y, "Y"), (W1, "W1"), (W2, "W2"), (b1, "b1"), (b2, "b2")):
        _check_input(t, nm)
    for t, nm in ((row_ptr, "row_ptr"), (seg, "seg")):
        _check_input(t, nm, torch.int32)
    rows, dim_in = int(x.size(0)), int(x.size(1))
    if (x.dim() != 2 or tuple(Y.shape) != (128, dim_in) or tuple(W1.shape) != (256, 128) or tuple(W2.shape) != (256, 256)
            or b1.numel() != 256 or b2.numel() != 256 or dim_in % 32):
        raise RuntimeError("mlp_chain_bf16: x (rows, dim_in), Y (128, dim_in), W1 (256, 128), W2 (256, 256) expected")
    if seg.numel() != rows or row_ptr.numel() != n_out + 1:
        raise RuntimeError("seg must have one entry per row and row_ptr n_out + 1 entries")
    nbytes = ctypes.c_size_t(0)
    L.check(_lib.mg_mlp_chain_bf16_workspace_bytes(rows, ctypes.byref(nbytes)))
    with _on(x.device):
        s_psi = torch.empty(n_out, 128, dtype=torch.float32, device=x.device)
        s_h = torch.empty(n_out, 256, dtype=torch.float32, device=x.device)
        work = torch.empty(nbytes.value // 4, dtype=torch.float32, device=x.device)
        L.check(_lib.mg_mlp_chain_bf16(_p(x), rows, dim_in, _p(packed_weight(Y)),
                                       _p(packed_weight(_operand_order_columns(W1))), _p(b1),
                                       _p(packed_weight(_operand_order_columns(W2))), _p(b2), int(act), _p(row_ptr),
                                       _p(seg), int(n_out), _p(work), _p(s_psi), _p(s_h), _stream()))
    return s_psi, s_h


def tens_group_norm_bf16_supported(comps, chan):
    return chan % 8 == 0 and comps * chan <= 4608


def tens_group_norm_bf16(y, batch, groups, gamma, eps, res=None):
    """TensGroupNorm on a component-major bf16 storage tensor y (batch * nodes, comps, chan) or (batch * nodes, chan):
    gamma * y / sqrt(eps + second moment of the group over nodes, components and the group's channels) (+ res)."""
    _check_bf16(y, "y")
    _check_input(gamma, "gamma")
    if res is not None:
        _check_bf16(res, "res")
        if res.shape != y.shape:
            raise RuntimeError("res must have the shape of y")
    rows, chan = int(y.size(0)), int(y.size(-1))
    comps = 1 if y.dim() == 2 else int(y.size(1))
    if rows % batch or gamma.numel() != chan:
        raise RuntimeError("rows must be a multiple of batch and gamma must have chan entries")
    nbytes = ctypes.c_size_t(0)
    L.check(_lib.mg_tens_group_norm_bf16_scratch_bytes(int(batch), int(groups), ctypes.byref(nbytes)))
    with _on(y.device):
        out = torch.empty_like(y)
        scratch = torch.empty((nbytes.value + 7) // 8, dtype=torch.float64, device=y.device)
        L.check(_lib.mg_tens_group_norm_bf16(_p(y), _p(res), int(batch), rows // batch, comps, chan, int(groups), float(eps),
                                             _p(gamma), _p(scratch), _p(out), _stream()))
    return out


def segment_sum_csr_bf16(x_edge, row_ptr, n_rows, scale=1.0):
    """scale * (sum of the bfloat16 edge rows of each CSR row), fp32 accumulation, bfloat16 result."""
    _check_bf16(x_edge, "x_edge")
    if x_edge.dim() != 2 or x_edge.size(1) % 4:
        raise RuntimeError("x_edge must be (edges, feat) with feat a multiple of 4")
    if row_ptr.dtype != torch.int32 or row_ptr.numel() != n_rows + 1:
        raise RuntimeError("row_ptr must be int32 with n_rows + 1 entries")
    feat = int(x_edge.size(1))
    with _on(x_edge.device):
        out = torch.empty(n_rows, feat, dtype=torch.bfloat16, device=x_edge.device)
        L.check(_lib.mg_segment_sum_csr_bf16(_p(x_edge), _p(row_ptr), int(n_rows), feat, float(scale), _p(out),
                                             _stream()))
    return out


# ----------------------------------------------------------------------- PaiNN
def painn_radial_encode(r_ij, n, rmax):
    """radial_encode of archs/meanflow_painn8.py:25-35: (E,3) -> (E,n)."""
    _check_input(r_ij, "r_ij")
    if r_ij.dim() != 2 or r_ij.size(1) != 3:
        raise RuntimeError("r_ij must have shape (edges, 3)")
    E = int(r_ij.size(0))
    with _on(r_ij.device):
        out = torch.empty(E, n, dtype=torch.float32, device=r_ij.device)
        L.check(_lib.mg_painn_radial_encode(_p(r_ij), E, int(n), float(rmax), _p(out), _stream()))
    return out


def painn_radial_linear_supported(n, dim_out):
    """Shapes the fused encode + first-layer kernel takes."""
    g = dim_out // 4
    return n <= 32 and dim_out % 4 == 0 and 1 <= g <= 256 and 256 % g == 0


def painn_radial_linear(r_ij, n, rmax, W, bias=None, act=ACT_NONE):
    """act(bias + radial_encode(r_ij, n, rmax) @ W.T) without writing the encoding
    (archs/meanflow_painn8.py:25-35 into the first layer of mlp_dist, :38-51)."""
    _check_input(r_ij, "r_ij")
    if r_ij.dim() != 2 or r_ij.size(1) != 3:
        raise RuntimeError("r_ij must have shape (edges, 3)")
    if W.dim() != 2 or W.size(1) != n:
        raise RuntimeError("W must have shape (dim_out, n)")
    if W.dtype != torch.float32 or not W.is_cuda:
        raise RuntimeError("W must be a float32 CUDA tensor")
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_cuda or not bias.is_contiguous()
                             or bias.numel() != W.size(0)):
        raise RuntimeError("bias must be a contiguous float32 CUDA tensor of dim_out elements")
    E, O = int(r_ij.size(0)), int(W.size(0))
    with _on(r_ij.device):
        y = torch.empty(E, O, dtype=torch.float32, device=r_ij.device)
        L.check(_lib.mg_painn_radial_linear(_p(r_ij), E, int(n), float(rmax), _p(W), W.stride(0), W.stride(1),
                                            _p(bias) if bias is not None else None, O, int(act), _p(y), _stream()))
    return y


def painn_combine_supported(n):
    return bool(_lib.mg_painn_combine_supported(int(n)))


def _combine_inputs(dist, actv, v, direction, node):
    for t, name in ((dist, "dist"), (actv, "actv"), (v, "v"), (direction, "direction")):
        _check_input(t, name)
    E, n = int(dist.size(0)), int(v.size(1))
    rows = int(v.size(0))
    if node is None:
        if rows != E:
            raise RuntimeError("without an index v needs one row per edge")
    else:
        _check_input(node, "node", torch.int32)
        if node.numel() != E:
            raise RuntimeError("node must have one entry per edge")
    if v.dim() != 3 or v.size(2) != 3 or tuple(dist.shape) != (E, 4 * n) or tuple(actv.shape) != (rows, 4 * n) \
            or tuple(direction.shape) != (E, 3):
        raise RuntimeError("expected dist (E, 4n), actv (rows, 4n), v (rows, n, 3), direction (E, 3)")
    return E, n, rows


def painn_combine_fwd(dist, actv, v, direction, node=None, terms=15):
    """m = v p[:, :n] + (v x direction) p[:, n:2n] + direction p[:, 2n:3n], a = p[:, 3n:] with p = dist * actv
    (archs/meanflow_painn8.py:94-100), in one pass.  node (int32, one per edge): actv and v hold one row per node and
    edge e reads row node[e] (the reference's edges_read_dst folded in).  terms: mask of the four terms that take part
    (15: all; include/managan_hip.h)."""
    E, n, rows = _combine_inputs(dist, actv, v, direction, node)
    with _on(v.device):
        m = torch.empty(E, n, 3, dtype=torch.float32, device=v.device)
        a = torch.empty(E, n, dtype=torch.float32, device=v.device)
        L.check(_lib.mg_painn_combine_fwd(_p(dist), _p(actv), _p(v), _p(direction), _p(node), rows, E, n, int(terms),
                                          _p(m), _p(a), _stream()))
    return m, a


def painn_combine_fwd_rows(dist, actv, v, direction, node, row_ptr, n_out_rows, terms=15):
    """painn_combine_fwd with m and a summed over the edges of each CSR row inside the kernel (edges sorted by the row,
    row_ptr (n_out_rows + 1) int32): (out_v (n_out_rows, n, 3), out_a (n_out_rows, n))."""
    E, n, rows = _combine_inputs(dist, actv, v, direction, node)
    _check_input(row_ptr, "row_ptr", torch.int32)
    if row_ptr.numel() != n_out_rows + 1:
        raise RuntimeError("row_ptr must have n_out_rows + 1 entries")
    with _on(v.device):
        out_v = torch.empty(n_out_rows, n, 3, dtype=torch.float32, device=v.device)
        out_a = torch.empty(n_out_rows, n, dtype=torch.float32, device=v.device)
        L.check(_lib.mg_painn_combine_fwd_rows(_p(dist), _p(actv), _p(v), _p(direction), _p(node), rows, _p(row_ptr),
                                               int(n_out_rows), E, n, int(terms), _p(out_v), _p(out_a), _stream()))
    return out_v, out_a


def painn_combine_bwd(dist, actv, v, direction, dm, da, node=None, grad_row=None, terms=15, want=(True, True, True, True)):
    """Gradients of painn_combine_fwd's four inputs from those of its outputs; those of actv and v per edge
    ((E, 4n), (E, n, 3)) also when the inputs are per node.  grad_row (int32, one per edge): dm and da hold one row per
    node and edge e takes row grad_row[e] (the adjoint of summing m and a over the edges of a source node)."""
    E, n, rows = _combine_inputs(dist, actv, v, direction, node)
    _check_input(dm, "dm")
    _check_input(da, "da")
    g_rows = E
    if grad_row is not None:
        _check_input(grad_row, "grad_row", torch.int32)
        g_rows = int(dm.size(0))
        if grad_row.numel() != E:
            raise RuntimeError("grad_row must have one entry per edge")
    if tuple(dm.shape) != (g_rows, n, 3) or tuple(da.shape) != (g_rows, n):
        raise RuntimeError("expected dm (rows, n, 3) and da (rows, n)")
    with _on(v.device):
        # (want: which of the four gradients to compute; the others come back as None)
        d_dist = torch.empty_like(dist) if want[0] else None
        d_actv = torch.empty(E, 4 * n, dtype=torch.float32, device=v.device) if want[1] else None
        dv = torch.empty(E, n, 3, dtype=torch.float32, device=v.device) if want[2] else None
        d_dir = torch.empty_like(direction) if want[3] else None
        L.check(_lib.mg_painn_combine_bwd(_p(dist), _p(actv), _p(v), _p(direction), _p(node), rows, _p(dm), _p(da),
                                          _p(grad_row), g_rows, E, n, int(terms), _p(d_dist), _p(d_actv), _p(dv),
                                          _p(d_dir), _stream()))
    return d_dist, d_actv, dv, d_dir


def painn_combine_bwd_grid(table, period, d, actv, v, direction, dm, da, node, grad_row, terms=15,
                           want=(True, True, True, True)):
    """painn_combine_bwd with the filter of edge e interpolated from `table` (rows, 4n) at the length d[e] inside the
    kernel (the backward pass of a message whose forward pass was painn_table_message: no (E, 4n) filter is kept).
    actv (nodes, 4n) and v (nodes, n, 3) are read at node[e], dm and da at grad_row[e]."""
    for t, name in ((table, "table"), (d, "d"), (actv, "actv"), (v, "v"), (direction, "direction"), (dm, "dm"), (da, "da")):
        _check_input(t, name)
    _check_input(node, "node", torch.int32)
    _check_input(grad_row, "grad_row", torch.int32)
    E, n, rows = int(d.numel()), int(v.size(1)), int(v.size(0))
    if tuple(table.shape[1:]) != (4 * n,) or tuple(actv.shape) != (rows, 4 * n) or tuple(v.shape) != (rows, n, 3):
        raise RuntimeError("expected table (grid rows, 4n), actv (rows, 4n), v (rows, n, 3)")
    if tuple(direction.shape) != (E, 3) or node.numel() != E or grad_row.numel() != E:
        raise RuntimeError("expected direction (edges, 3) and one index entry per edge")
    g_rows = int(dm.size(0))
    if tuple(dm.shape) != (g_rows, n, 3) or tuple(da.shape) != (g_rows, n):
        raise RuntimeError("expected dm (rows, n, 3) and da (rows, n)")
    with _on(v.device):
        d_dist = torch.empty(E, 4 * n, dtype=torch.float32, device=v.device) if want[0] else None
        d_actv = torch.empty(E, 4 * n, dtype=torch.float32, device=v.device) if want[1] else None
        dv = torch.empty(E, n, 3, dtype=torch.float32, device=v.device) if want[2] else None
        d_dir = torch.empty_like(direction) if want[3] else None
        L.check(_lib.mg_painn_combine_bwd_grid(_p(table), int(table.size(0)), float(period), _p(d), _p(actv), _p(v),
                                               _p(direction), _p(node), rows, _p(dm), _p(da), _p(grad_row), g_rows, E, n,
                                               int(terms), _p(d_dist), _p(d_actv), _p(dv), _p(d_dir), _stream()))
    return d_dist, d_actv, dv, d_dir


def painn_combine_bwd_rows(dist, actv, v, direction, dm, da, row_ptr, order, grad_row, terms=15,
                           want=(True, True, True, True), table=None, period=None, d=None):
    """The gradients of painn_combine_fwd's inputs for actv (rows, 4n) and v (rows, n, 3) read per edge at one row,
    with those two gradients summed per row inside the kernel: (d_dist (E, 4n), d_actv (rows, 4n), dv (rows, n, 3),
    d_dir (E, 3)).  (row_ptr, order): the CSR of the edges by the row they read (order None: edges sorted by it).
    dm, da are read at grad_row[e] (None: at e).  The filter: dist (E, 4n), or dist None and table (grid rows, 4n),
    period, d (E): interpolated inside the kernel."""
    grid = dist is None
    for t, name in ((actv, "actv"), (v, "v"), (direction, "direction"), (dm, "dm"), (da, "da")):
        _check_input(t, name)
    _check_input(row_ptr, "row_ptr", torch.int32)
    if order is not None:
        _check_input(order, "order", torch.int32)
    if grad_row is not None:
        _check_input(grad_row, "grad_row", torch.int32)
    E, n, rows = int(direction.size(0)), int(v.size(1)), int(v.size(0))
    if grid:
        _check_input(table, "table")
        _check_input(d, "d")
        if table.dim() != 2 or table.size(1) != 4 * n or d.numel() != E:
            raise RuntimeError("expected table (grid rows, 4n) and d (edges)")
    else:
        _check_input(dist, "dist")
        if tuple(dist.shape) != (E, 4 * n):
            raise RuntimeError("expected dist (edges, 4n)")
    if tuple(actv.shape) != (rows, 4 * n) or tuple(v.shape) != (rows, n, 3) or tuple(direction.shape) != (E, 3):
        raise RuntimeError("expected actv (rows, 4n), v (rows, n, 3), direction (edges, 3)")
    if row_ptr.numel() != rows + 1 or (order is not None and order.numel() != E) or \
            (grad_row is not None and grad_row.numel() != E):
        raise RuntimeError("expected row_ptr (rows + 1) and one entry per edge in order / grad_row")
    g_rows = int(dm.size(0))
    if tuple(dm.shape) != (g_rows, n, 3) or tuple(da.shape) != (g_rows, n) or (grad_row is None and g_rows != E):
        raise RuntimeError("expected dm (rows, n, 3) and da (rows, n)")
    with _on(v.device):
        d_dist = torch.empty(E, 4 * n, dtype=torch.float32, device=v.device) if want[0] else None
        d_actv = torch.empty(rows, 4 * n, dtype=torch.float32, device=v.device) if want[1] else None
        dv = torch.empty(rows, n, 3, dtype=torch.float32, device=v.device) if want[2] else None
        d_dir = torch.empty_like(direction) if want[3] else None
        L.check(_lib.mg_painn_combine_bwd_rows(_p(dist), _p(table) if grid else None, int(table.size(0)) if grid else 0,
                                               float(period) if grid else 0.0, _p(d) if grid else None, _p(actv), _p(v),
                                               _p(direction), _p(row_ptr), _p(order), rows, _p(dm), _p(da), _p(grad_row),
                                               g_rows, E, n, int(terms), _p(d_dist), _p(d_actv), _p(dv), _p(d_dir), _stream()))
    return d_dist, d_actv, dv, d_dir


def painn_table_interp_supported(table_rows, cols):
    return bool(_lib.mg_painn_table_interp_supported(int(table_rows), int(cols)))


def _table_inputs(table, d):
    _check_input(table, "table")
    _check_input(d, "d")
    if table.dim() != 2 or d.dim() != 1:
        raise RuntimeError("expected table (rows, cols) and d (edges)")
    return int(table.size(0)), int(table.size(1)), int(d.numel())


def painn_table_interp_fwd(table, d, period, order=0):
    """(edges, cols): the grid `table` of a function of period `period`, interpolated at the lengths d (4-point
    Lagrange, as the inference kernels do); order 1 .. 3: the interpolant's derivative of that order in d."""
    rows, cols, E = _table_inputs(table, d)
    with _on(d.device):
        out = torch.empty(E, cols, dtype=torch.float32, device=d.device)
        L.check(_lib.mg_painn_table_interp_fwd(_p(table), rows, cols, float(period), _p(d), E, int(order), _p(out),
                                               _stream()))
    return out


def painn_table_sorted_edges(d, table_rows, period):
    """(perm, bucket_ptr): the edges in the order of a stable sort by the grid row below their length, and the row
    pointer of the sorted rows: what painn_table_interp_bwd sums by."""
    _check_input(d, "d")
    E = int(d.numel())
    with _on(d.device):
        bucket = torch.empty(E, dtype=torch.int32, device=d.device)
        L.check(_lib.mg_painn_table_buckets(_p(d), E, int(table_rows), float(period), _p(bucket), _stream()))
        ordered, perm = torch.sort(bucket, stable=True)
    return perm.to(torch.int32).contiguous(), segment_row_ptr(ordered.contiguous(), int(table_rows))


def painn_table_interp_bwd(g, table, d, period, perm, bucket_ptr, want_length_grad=True, order=0, table_rows=None):
    """(d_table, dd): the gradients of painn_table_interp_fwd's table and lengths for the output gradient g.
    table may be None when only d_table is wanted (table_rows then gives the grid's size)."""
    _check_input(d, "d")
    _check_input(g, "g")
    if table is not None:
        rows, cols, E = _table_inputs(table, d)
    else:
        rows, cols, E = int(table_rows), int(g.size(1)), int(d.numel())
        if want_length_grad:
            raise RuntimeError("the length gradient needs the table")
    _check_input(perm, "perm", torch.int32)
    _check_input(bucket_ptr, "bucket_ptr", torch.int32)
    if tuple(g.shape) != (E, cols) or perm.numel() != E or bucket_ptr.numel() != rows + 1:
        raise RuntimeError("expected g (edges, cols), perm (edges), bucket_ptr (rows + 1)")
    with _on(d.device):
        nbytes = ctypes.c_size_t(0)
        L.check(_lib.mg_painn_table_interp_bwd_workspace_bytes(rows, cols, ctypes.byref(nbytes)))
        ws = torch.empty(nbytes.value, dtype=torch.uint8, device=d.device)
        d_table = torch.empty(rows, cols, dtype=torch.float32, device=d.device)
        dd = torch.empty_like(d) if want_length_grad else None
        L.check(_lib.mg_painn_table_interp_bwd(_p(g), _p(table), rows, cols, float(period), _p(d), _p(perm),
                                               _p(bucket_ptr), E, int(order), _p(ws), _p(d_table), _p(dd), _stream()))
    return d_table, dd


def painn_message(row_ptr, dst, r_ij, filt, actv, x_v, epsilon, res_a=None, res_v=None, node_order=None):
    """Fused gather-product-scatter of the PaiNN message (archs/meanflow_painn8.py:91-100).
    filt (E,4n), actv (nodes,4n), x_v (nodes,n,3) -> out_a (nodes,n), out_v (nodes,n,3).
    node_order (int32, nodes): processing order of the rows (does not change the results)."""
    _check_input(row_ptr, "row_ptr", torch.int32)
    _check_input(dst, "dst", torch.int32)
    for t, nm in ((r_ij, "r_ij"), (filt, "filt"), (actv, "actv"), (x_v, "x_v")):
        _check_input(t, nm)
    n_nodes, n = int(x_v.size(0)), int(x_v.size(1))
    E = int(dst.numel())
    if tuple(x_v.shape) != (n_nodes, n, 3):
        raise RuntimeError("x_v must have shape (nodes, n, 3)")
    if tuple(actv.shape) != (n_nodes, 4 * n):
        raise RuntimeError("actv must have shape (nodes, 4n)")
    if tuple(filt.shape) != (E, 4 * n):
        raise RuntimeError("filt must have shape (edges, 4n)")
    if tuple(r_ij.shape) != (E, 3):
        raise RuntimeError("r_ij must have shape (edges, 3)")
    if row_ptr.numel() != n_nodes + 1:
        raise RuntimeError("row_ptr must have nodes+1 entries")
    for t, nm, shape in ((res_a, "res_a", (n_nodes, n)), (res_v, "res_v", (n_nodes, n, 3))):
        if t is not None:
            _check_input(t, nm)
            if tuple(t.shape) != shape:
                raise RuntimeError(f"{nm} has wrong shape")
    if node_order is not None:
        _check_input(node_order, "node_order", torch.int32)
        if node_order.numel() != n_nodes:
            raise RuntimeError("node_order must have one entry per node")
    dev = x_v.device
    with _on(dev):
        out_a = torch.empty(n_nodes, n, dtype=torch.float32, device=dev)
        out_v = torch.empty(n_nodes, n, 3, dtype=torch.float32, device=dev)
        L.check(_lib.mg_painn_message(_p(row_ptr), _p(dst), _p(node_order), n_nodes, E, _p(r_ij), _p(filt), _p(actv), _p(x_v), n,
                                      float(epsilon), _p(res_a), _p(res_v), _p(out_a), _p(out_v), _stream()))
    return out_a, out_v


def painn_table_message(row_ptr, dst, r_ij, table, period, actv, x_v, epsilon, res_a=None, res_v=None, node_order=None):
    """painn_message with the per-edge filter interpolated from `table` (rows, 4n): the filter as a function of
    the edge length at d = k * period / rows (rows a power of two; the function has period `period`)."""
    _check_input(row_ptr, "row_ptr", torch.int32)
    _check_input(dst, "dst", torch.int32)
    for t, nm in ((r_ij, "r_ij"), (table, "table"), (actv, "actv"), (x_v, "x_v")):
        _check_input(t, nm)
    n_nodes, n = int(x_v.size(0)), int(x_v.size(1))
    E = int(dst.numel())
    if tuple(x_v.shape) != (n_nodes, n, 3):
        raise RuntimeError("x_v must have shape (nodes, n, 3)")
    if tuple(actv.shape) != (n_nodes, 4 * n):
        raise RuntimeError("actv must have shape (nodes, 4n)")
    if table.dim() != 2 or table.size(1) != 4 * n:
        raise RuntimeError("table must have shape (rows, 4n)")
    if tuple(r_ij.shape) != (E, 3):
        raise RuntimeError("r_ij must have shape (edges, 3)")
    if row_ptr.numel() != n_nodes + 1:
        raise RuntimeError("row_ptr must have nodes+1 entries")
    for t, nm, shape in ((res_a, "res_a", (n_nodes, n)), (res_v, "res_v", (n_nodes, n, 3))):
        if t is not None:
            _check_input(t, nm)
            if tuple(t.shape) != shape:
                raise RuntimeError(f"{nm} has wrong shape")
    if node_order is not None:
        _check_input(node_order, "node_order", torch.int32)
        if node_order.numel() != n_nodes:
            raise RuntimeError("node_order must have one entry per node")
    dev = x_v.device
    with _on(dev):
        out_a = torch.empty(n_nodes, n, dtype=torch.float32, device=dev)
        out_v = torch.empty(n_nodes, n, 3, dtype=torch.float32, device=dev)
        L.check(_lib.mg_painn_table_message(_p(row_ptr), _p(dst), _p(node_order), n_nodes, E, _p(r_ij), _p(table),
                                            int(table.size(0)), float(period), _p(actv), _p(x_v), n, float(epsilon),
                                            _p(res_a), _p(res_v), _p(out_a), _p(out_v), _stream()))
    return out_a, out_v


PAINN_SLICE = 16              # channels per slice of painn_table_message_sliced
PAINN_SLICED_MAX_ROWS = 512   # table rows that fit in LDS beside a slice's 64 columns


def painn_slice_permutation(n, device):
    """Column order of actv for painn_table_message_sliced: position (s, k, c) of (n / 16, 4, 16) holds column
    k n + 16 s + c."""
    s, k, c = torch.meshgrid(torch.arange(n // PAINN_SLICE), torch.arange(4), torch.arange(PAINN_SLICE), indexing="ij")
    return (k * n + PAINN_SLICE * s + c).reshape(-1).to(device)


def painn_edge_records(r_ij, table_rows, period, epsilon):
    """(edges, 8): per edge the first of its four grid rows, the interpolation weights and the direction, for
    painn_table_message_sliced."""
    _check_input(r_ij, "r_ij")
    E = int(r_ij.size(0))
    if tuple(r_ij.shape) != (E, 3):
        raise RuntimeError("r_ij must have shape (edges, 3)")
    with _on(r_ij.device):
        rec = torch.empty(E, 8, dtype=torch.float32, device=r_ij.device)
        L.check(_lib.mg_painn_edge_records(_p(r_ij), E, int(table_rows), float(period), float(epsilon), _p(rec), _stream()))
    return rec


def painn_table_message_sliced(row_ptr, dst, r_ij, table, period, actv_sliced, x_v, epsilon, res_a=None, res_v=None,
                               node_order=None, records=None):
    """painn_table_message with the table held in LDS (at most 512 rows, n a multiple of 16) and actv given with its
    columns in the order of painn_slice_permutation.  records: painn_edge_records(r_ij, rows, period, epsilon) if the
    caller keeps them (they depend on the edges, not on the features)."""
    _check_input(row_ptr, "row_ptr", torch.int32)
    _check_input(dst, "dst", torch.int32)
    for t, nm in ((r_ij, "r_ij"), (table, "table"), (actv_sliced, "actv_sliced"), (x_v, "x_v")):
        _check_input(t, nm)
    n_nodes, n = int(x_v.size(0)), int(x_v.size(1))
    E = int(dst.numel())
    if tuple(x_v.shape) != (n_nodes, n, 3):
        raise RuntimeError("x_v must have shape (nodes, n, 3)")
    if tuple(actv_sliced.shape) != (n_nodes, 4 * n):
        raise RuntimeError("actv_sliced must have shape (nodes, 4n)")
    if table.dim() != 2 or table.size(1) != 4 * n:
        raise RuntimeError("table must have shape (rows, 4n)")
    if tuple(r_ij.shape) != (E, 3):
        raise RuntimeError("r_ij must have shape (edges, 3)")
    if row_ptr.numel() != n_nodes + 1:
        raise RuntimeError("row_ptr must have nodes+1 entries")
    for t, nm, shape in ((res_a, "res_a", (n_nodes, n)), (res_v, "res_v", (n_nodes, n, 3))):
        if t is not None:
            _check_input(t, nm)
            if tuple(t.shape) != shape:
                raise RuntimeError(f"{nm} has wrong shape")
    if node_order is not None:
        _check_input(node_order, "node_order", torch.int32)
        if node_order.numel() != n_nodes:
            raise RuntimeError("node_order must have one entry per node")
    rows = int(table.size(0))
    if rows < 4 or rows > PAINN_SLICED_MAX_ROWS or rows & (rows - 1):
        raise RuntimeError(f"table rows must be a power of two in 4..{PAINN_SLICED_MAX_ROWS} (got {rows})")
    if records is None:
        records = painn_edge_records(r_ij, rows, period, epsilon)
    else:
        _check_input(records, "records")
        if tuple(records.shape) != (E, 8):
            raise RuntimeError("records must have shape (edges, 8)")
    dev = x_v.device
    with _on(dev):
        out_a = torch.empty(n_nodes, n, dtype=torch.float32, device=dev)
        out_v = torch.empty(n_nodes, n, 3, dtype=torch.float32, device=dev)
        L.check(_lib.mg_painn_table_message_sliced(_p(row_ptr), _p(dst), _p(node_order), n_nodes, E, _p(records),
                                                   _p(table), rows, _p(actv_sliced), _p(x_v), n, _p(res_a), _p(res_v),
                                                   _p(out_a), _p(out_v), _stream()))
    return out_a, out_v


def bee_products_linear_supported(n_nodes, chan):
    # below a few thousand nodes the fused kernels (a workgroup walks the whole reduction dimension, building its
    # operand from cache reads) are bound by that chain's latency: products kernel + three plain GEMMs are faster
    return get_linear_mode() == LINEAR_F16X2 and chan % 32 == 0 and chan >= 32 and n_nodes >= 8192


def bee_products_linear(rank_o, W, l0, l1, l2, r0, r1, r2, node_bound):
    """y (nodes, dim_out, (3,)^rank_o) = sum over the product types of output rank rank_o of Y_lab p_lab(l, r), with
    W = [Y_lab ...] concatenated along the input axis in the order 000 110 220 / 011 101 121 211 111 /
    022 202 112 222 212.  l_k, r_k component-major (nodes, 3^k, chan) ((nodes, chan) for k = 0); node_bound (nodes,):
    upper bound of every |product component| of the node."""
    for t, nm in ((W, "W"), (l0, "l0"), (l1, "l1"), (l2, "l2"), (r0, "r0"), (r1, "r1"), (r2, "r2"), (node_bound, "node_bound")):
        _check_input(t, nm)
    N, chan = int(l0.size(0)), int(l0.size(1))
    for t, comps in ((l0, None), (r0, None), (l1, 3), (r1, 3), (l2, 9), (r2, 9)):
        if tuple(t.shape) != ((N, chan) if comps is None else (N, comps, chan)):
            raise RuntimeError("operands must be (nodes, chan), (nodes, 3, chan), (nodes, 9, chan)")
    n_types = 3 if rank_o == 0 else 5
    if W.dim() != 2 or int(W.size(1)) != n_types * chan:
        raise RuntimeError(f"W must be (dim_out, {n_types} * chan)")
    if node_bound.numel() != N:
        raise RuntimeError("node_bound must have one entry per node")
    dim_out = int(W.size(0))
    k_order = 1 if (rank_o == 2 and dim_out <= 64) else 0
    if k_order:
        W = _channel_block_major_columns(W, n_types, chan)
    with _on(l0.device):
        y = torch.empty((N, dim_out) + (3,) * rank_o, dtype=torch.float32, device=l0.device)
        L.check(_lib.mg_bee_products_linear(int(rank_o), _p(l0), _p(l1), _p(l2), _p(r0), _p(r1), _p(r2), _p(node_bound),
                                            N, chan, _p(packed_weight_f16x2(W)), k_order, dim_out, _p(y), _stream()))
    return y


_reordered_cache = {}


def _channel_block_major_columns(W, n_types, chan):
    """W (dim_out, n_types * chan) with its columns reordered from (type, channel) to (channel block of 32, type,
    channel in block); cached per tensor object and version."""
    key = (id(W), n_types, chan)
    hit = _reordered_cache.get(key)
    if hit is not None and hit[0]() is W and hit[1] == tensor_version(W) >= 0 and hit[2] == W.data_ptr():
        return hit[3]
    with derived_tensors():
        Wr = (W.detach().reshape(W.shape[0], n_types, chan // 32, 32).permute(0, 2, 1, 3)
              .reshape(W.shape[0], n_types * chan).contiguous())
    if len(_reordered_cache) > 256:
        _reordered_cache.clear()
    _reordered_cache[key] = (weakref.ref(W), tensor_version(W), W.data_ptr(), Wr)
    return Wr


def f16x2_rowsum_supported(rows, dim_in, dim_out, x):
    """The GEMM whose epilogue sums the rows of each segment: 256-column tiles, and enough rows to fill the chip."""
    return (get_linear_mode() == LINEAR_F16X2 and dim_out % 256 == 0 and dim_in % 32 == 0 and dim_in >= 64
            and rows >= 4096 and x.data_ptr() % 16 == 0)


def tensor_linear_f16x2_rowsum(W, x, x_bound, row_ptr, seg, n_out, bias=None, act=ACT_NONE, scale=1.0, want_rows=False):
    """(out, y): out[s] = scale * sum over the rows r of segment s of act(bias + W x[r]) (n_out, dim_out); y is the
    per-row result (rows, dim_out) when want_rows is set, else None.  Rows are sorted by segment: seg (rows,) int32
    ascending, row_ptr its CSR form.  x_bound: (rows, parts) or (1, parts) upper bounds of the row maxima of |x|, or
    a ScaledBound of such an array."""
    bound_mul, bound_add = 1.0, 0.0
    if isinstance(x_bound, ScaledBound):
        x_bound, bound_mul, bound_add = x_bound.base, x_bound.mul, x_bound.add
    for t, nm in ((W, "W"), (x, "x"), (x_bound, "x_bound")):
        _check_input(t, nm)
    for t, nm in ((row_ptr, "row_ptr"), (seg, "seg")):
        _check_input(t, nm, torch.int32)
    if x.dim() != 2 or W.dim() != 2 or x.size(1) != W.size(1):
        raise RuntimeError("x must have shape (rows, dim_in) and W (dim_out, dim_in)")
    rows, dim_in, dim_out = int(x.size(0)), int(W.size(1)), int(W.size(0))
    if seg.numel() != rows or row_ptr.numel() != n_out + 1:
        raise RuntimeError("seg must have one entry per row and row_ptr n_out + 1 entries")
    if x_bound.dim() != 2 or x_bound.size(0) not in (1, rows) or not 1 <= x_bound.size(1) <= 64:
        raise RuntimeError("x_bound must be (rows, parts) or (1, parts) with 1..64 parts")
    if bias is not None:
        _check_input(bias, "bias")
        if bias.numel() != dim_out:
            raise RuntimeError("bias must have dim_out elements")
    dev = x.device
    nbytes = ctypes.c_size_t(0)
    L.check(_lib.mg_tensor_linear_f16x2_rowsum_workspace_bytes(rows, dim_out, ctypes.byref(nbytes)))
    with _on(dev):
        out = torch.empty(n_out, dim_out, dtype=torch.float32, device=dev)
        y = torch.empty(rows, dim_out, dtype=torch.float32, device=dev) if want_rows else None
        work = torch.empty(nbytes.value // 4, dtype=torch.float32, device=dev)
        stride = 0 if x_bound.size(0) == 1 else int(x_bound.size(1))
        L.check(_lib.mg_tensor_linear_f16x2_rowsum_scaled_bound(
            _p(packed_weight_f16x2(W)), _p(x), _p(x_bound), int(x_bound.size(1)), stride, rows, dim_in, dim_out,
            _p(bias), int(act), _p(row_ptr), _p(seg), int(n_out), float(scale), _p(work), _p(y), _p(out),
            bound_mul, bound_add, _stream()))
    return out, y


def painn_filter_hidden_supported(n_rbf, hidden, n_edges):
    """First two filter layers in one kernel: 16 radial functions, hidden width 256 or 512."""
    return get_linear_mode() == LINEAR_F16X2 and n_rbf == 16 and hidden in (256, 512) and n_edges >= 1024


_chunk_perm_cache = {}


def _operand_order_columns(W):
    """W (dim_out, dim_in) with the input channels of every group of 32 reordered to the accumulator order of the
    matrix core (position 16 g + p holds channel 8 (p / 4) + 4 g + p % 4); cached per tensor object and version."""
    key = id(W)
    hit = _chunk_perm_cache.get(key)
    if hit is not None and hit[0]() is W and hit[1] == tensor_version(W) >= 0 and hit[2] == W.data_ptr():
        return hit[3]
    pos = torch.arange(32, device=W.device)
    g, p = pos // 16, pos % 16
    src = 8 * (p // 4) + 4 * g + p % 4
    cols = (torch.arange(0, W.shape[1], 32, device=W.device)[:, None] + src[None, :]).reshape(-1)
    with derived_tensors():
        Wr = W.detach()[:, cols].contiguous()
    if len(_chunk_perm_cache) > 256:
        _chunk_perm_cache.clear()
    _chunk_perm_cache[key] = (weakref.ref(W), tensor_version(W), W.data_ptr(), Wr)
    return Wr


def painn_filter_hidden(r_ij, rmax, W1, b1, W2, b2, h1_bound):
    """SiLU(b2 + W2 SiLU(b1 + W1 radial_encode(r_ij, 16, rmax))) (edges, hidden) without storing the first layer's
    output.  h1_bound: (1, 1) upper bound of the first layer's output (linear_out_bound(W1, b1, None))."""
    for t, nm in ((r_ij, "r_ij"), (W2, "W2"), (b2, "b2"), (h1_bound, "h1_bound")):
        _check_input(t, nm)
    if not W1.is_cuda or W1.dtype != torch.float32 or W1.dim() != 2 or W1.size(1) != 16:
        raise RuntimeError("W1 must be a float32 CUDA matrix (hidden, 16)")
    hidden = int(W1.size(0))
    if tuple(W2.shape) != (hidden, hidden) or b2.numel() != hidden or (b1 is not None and b1.numel() != hidden):
        raise RuntimeError("W2 must be (hidden, hidden), b1 and b2 (hidden,)")
    if r_ij.dim() != 2 or r_ij.size(1) != 3:
        raise RuntimeError("r_ij must have shape (edges, 3)")
    if b1 is not None:
        _check_input(b1, "b1")
    E = int(r_ij.size(0))
    with _on(r_ij.device):
        y = torch.empty(E, hidden, dtype=torch.float32, device=r_ij.device)
        L.check(_lib.mg_painn_filter_hidden(_p(r_ij), E, float(rmax), _p(W1), int(W1.stride(0)), int(W1.stride(1)),
                                            _p(b1), _p(packed_weight_f16x2(_operand_order_columns(W2))), _p(b2), hidden,
                                            _p(h1_bound), _p(y), _stream()))
    return y


def painn_filter_message_supported(n, hidden, n_edges):
    """The fused filter + message kernel: channel blocks of 64, a hidden width the matrix path tiles, and
    enough edges to fill the chip with 256-edge tiles."""
    return (get_linear_mode() == LINEAR_F16X2 and n % 64 == 0 and hidden % 32 == 0 and hidden >= 64
            and n_edges >= 1024)


def painn_filter_permutation(n, device):
    """Order of the 4n filter columns in the fused kernel's packed weight: (channel block of 64, k, channel
    in block).  perm[p] is the filter column k n + c that packed row p holds."""
    c = torch.arange(n, device=device)
    k = torch.arange(4, device=device)
    col = (k[None, :, None] * n + (c.reshape(n // 64, 1, 64)))     # (blocks, 4, 64)
    return col.reshape(-1)


def painn_filter_message(W3_perm, bias3_perm, h, h_bound, row_ptr, src, dst, r_ij, actv, x_v, epsilon,
                         res_a=None, res_v=None):
    """painn_message(filt = h @ W3.T + bias3, ...) without storing filt.  W3_perm / bias3_perm: W3 / bias3 with
    rows in painn_filter_permutation order; h (edges, hidden); h_bound (edges, parts) or (1, parts): upper
    bounds of the row maxima of |h|."""
    for t, nm in ((W3_perm, "W3_perm"), (bias3_perm, "bias3_perm"), (h, "h"), (h_bound, "h_bound"), (r_ij, "r_ij"),
                  (actv, "actv"), (x_v, "x_v")):
        _check_input(t, nm)
    for t, nm in ((row_ptr, "row_ptr"), (src, "src"), (dst, "dst")):
        _check_input(t, nm, torch.int32)
    n_nodes, n = int(x_v.size(0)), int(x_v.size(1))
    E, hidden = int(h.size(0)), int(h.size(1))
    if tuple(x_v.shape) != (n_nodes, n, 3):
        raise RuntimeError("x_v must have shape (nodes, n, 3)")
    if tuple(actv.shape) != (n_nodes, 4 * n):
        raise RuntimeError("actv must have shape (nodes, 4n)")
    if tuple(W3_perm.shape) != (4 * n, hidden) or tuple(bias3_perm.shape) != (4 * n,):
        raise RuntimeError("W3_perm must have shape (4n, hidden) and bias3_perm (4n,)")
    if tuple(r_ij.shape) != (E, 3) or src.numel() != E or dst.numel() != E:
        raise RuntimeError("r_ij, src and dst must have one row per edge")
    if row_ptr.numel() != n_nodes + 1:
        raise RuntimeError("row_ptr must have nodes+1 entries")
    if h_bound.dim() != 2 or h_bound.size(0) not in (1, E) or not 1 <= h_bound.size(1) <= 64:
        raise RuntimeError("h_bound must be (edges, parts) or (1, parts) with 1..64 parts")
    for t, nm, shape in ((res_a, "res_a", (n_nodes, n)), (res_v, "res_v", (n_nodes, n, 3))):
        if t is not None:
            _check_input(t, nm)
            if tuple(t.shape) != shape:
                raise RuntimeError(f"{nm} has wrong shape")
    dev = x_v.device
    nbytes = ctypes.c_size_t(0)
    L.check(_lib.mg_painn_filter_message_workspace_bytes(E, n, ctypes.byref(nbytes)))
    with _on(dev):
        out_a = torch.empty(n_nodes, n, dtype=torch.float32, device=dev)
        out_v = torch.empty(n_nodes, n, 3, dtype=torch.float32, device=dev)
        work = torch.empty(nbytes.value // 4, dtype=torch.float32, device=dev)
        stride = 0 if h_bound.size(0) == 1 else int(h_bound.size(1))
        L.check(_lib.mg_painn_filter_message(
            _p(packed_weight_f16x2(W3_perm)), _p(bias3_perm), _p(h), _p(h_bound), int(h_bound.size(1)), stride,
            hidden, _p(row_ptr), _p(src), _p(dst), _p(r_ij), _p(actv), _p(x_v), n_nodes, E, n, float(epsilon),
            _p(res_a), _p(res_v), _p(work), _p(out_a), _p(out_v), _stream()))
    return out_a, out_v


# ------------------------------------------------------- rank-0/1/2 messages
def bee_edge_geometry(r_ij, r0):
    """(E,3) -> enc (E,8) = radial_encode_8(r_ij, r0), rhat (E,3) = tens_sigmoid(1, r_ij*7/r0)."""
    _check_input(r_ij, "r_ij")
    if r_ij.dim() != 2 or r_ij.size(1) != 3:
        raise RuntimeError("r_ij must have shape (edges, 3)")
    E = int(r_ij.size(0))
    with _on(r_ij.device):
        enc = torch.empty(E, 8, dtype=torch.float32, device=r_ij.device)
        rhat = torch.empty(E, 3, dtype=torch.float32, device=r_ij.device)
        L.check(_lib.mg_bee_edge_geometry(_p(r_ij), E, float(r0), _p(enc), _p(rhat), _stream()))
    return enc, rhat


_rank2_cache = {}


def bee_rank2_supported(chan, dim_d):
    """Can the edge kernel apply the rank-2 output linear (dim_d, 5 chan) itself?"""
    return bool(_lib.mg_bee_message_rank2_supported(int(chan), int(dim_d)))


def _packed_rank2_weight(Y2, chan):
    """Y2 (dim_d, 5 chan) in the lane order of the fused edge kernel; cached per tensor object and version."""
    key = id(Y2)
    hit = _rank2_cache.get(key)
    version = tensor_version(Y2)
    if hit is not None and version >= 0 and hit[0]() is Y2 and hit[1] == version and hit[2] == Y2.data_ptr():
        return hit[3]
    nbytes = ctypes.c_size_t(0)
    L.check(_lib.mg_bee_rank2_weight_bytes(chan, ctypes.byref(nbytes)))
    with _on(Y2.device):
        packed = torch.empty(nbytes.value // 4, dtype=torch.float32, device=Y2.device)
        L.check(_lib.mg_bee_pack_rank2_weight(_p(Y2), int(Y2.stride(0)), chan, int(Y2.size(0)), _p(packed), _stream()))
    if len(_rank2_cache) > 256:
        _rank2_cache.clear()
    _rank2_cache[key] = (weakref.ref(Y2, lambda _, key=key: _rank2_cache.pop(key, None)), version, Y2.data_ptr(), packed)
    return packed


def bee_node_products_rank2(l0, l1, l2, r0, r1, r2, Y2, want_lower_ranks=False, x_d=None, L2t=None, R2t=None):
    """The rank-2 output of SelfTensProds from its six operands in one kernel: Y2 (dim_d, 5 chan) applied to the five
    rank-2 products of l0/r0 (N, chan), l1/r1 (N, 3, chan), l2/r2 (N, 9, chan) -> (N, dim_d, 9); the rank-2 products
    are never stored.  For bee_rank2_supported(chan, dim_d).
    want_lower_ranks: returns (out_d, P0 (N,3,chan), P1 (N,3,5,chan), node_max (N, chan/64)) with the scalar and
    vector products of bee_node_products and their partial maxima per node, written in the same pass.
    x_d (N, dim_in, 3, 3) with L2t, R2t (dim_in, chan), dim_in <= 16, in place of l2 and r2 (then None): the rank-2
    operands l2 = L2 x_d, r2 = R2 x_d (L2t = L2.W.t() contiguous) are formed inside the kernel."""
    inside = x_d is not None
    named = [(l0, "l0"), (l1, "l1"), (r0, "r0"), (r1, "r1")] + ([(x_d, "x_d"), (L2t, "L2t"), (R2t, "R2t")] if inside
                                                                 else [(l2, "l2"), (r2, "r2")])
    for t, nm in named:
        _check_input(t, nm)
    N, chan = int(l0.size(0)), int(l0.size(1))
    shaped = [(l0, None), (r0, None), (l1, 3), (r1, 3)] + ([] if inside else [(l2, 9), (r2, 9)])
    for t, comps in shaped:
        if tuple(t.shape) != ((N, chan) if comps is None else (N, comps, chan)):
            raise RuntimeError("operands must be (nodes, chan), (nodes, 3, chan), (nodes, 9, chan)")
    dim_in2 = 0
    if inside:
        dim_in2 = int(L2t.size(0))
        if (tuple(L2t.shape) != (dim_in2, chan) or tuple(R2t.shape) != (dim_in2, chan) or dim_in2 > 16
                or x_d.numel() != N * dim_in2 * 9):
            raise RuntimeError("x_d must hold nodes x dim_in x 9 floats and L2t, R2t be (dim_in, chan), dim_in <= 16")
    if not Y2.is_cuda or Y2.dtype != torch.float32 or Y2.dim() != 2 or int(Y2.size(1)) != 5 * chan or Y2.stride(1) != 1:
        raise RuntimeError("Y2 must be a float32 CUDA tensor (dim_d, 5 chan) with unit stride along a row")
    if not bee_rank2_supported(chan, Y2.size(0)):
        raise RuntimeError("the fused rank-2 linear needs chan = 64, 128 or 256 and dim_d <= 16")
    dim_d = int(Y2.size(0))
    with _on(l0.device):
        out = torch.empty(N, dim_d, 9, dtype=torch.float32, device=l0.device)
        P0 = P1 = nmax = None
        if want_lower_ranks:
            P0 = torch.empty(N, 3, chan, dtype=torch.float32, device=l0.device)
            P1 = torch.empty(N, 3, 5, chan, dtype=torch.float32, device=l0.device)
            nmax = torch.empty(N, chan // 64, dtype=torch.float32, device=l0.device)
        L.check(_lib.mg_bee_node_products_rank2(N, chan, _p(l0), _p(l1), _p(l2), _p(r0), _p(r1), _p(r2),
                                                _p(_packed_rank2_weight(Y2, chan)), dim_d, _p(out), _p(P0), _p(P1),
                                                _p(nmax), _p(x_d), _p(L2t), _p(R2t), dim_in2, _stream()))
    return (out, P0, P1, nmax) if want_lower_ranks else out


def bee_message(row_ptr, dst, rhat, enc, La, Lv, Ld, enc_W, enc_b, node_order=None, want_node_max=False, Y2=None,
                out_d=None):
    """Fused products + edge sums of the rank-0/1/2 message (see mg_bee_message).
    La (N,chan), Lv (N,3,chan), Ld (N,9,chan) -> P0 (E,3,chan), S1 (N,3,5,chan), S2 (N,9,5,chan)
    (+ node_max (N, ceil(chan/64)) and edge_max (E, ceil(chan/64)): partial maxima of |S1|, |S2| per node
    and of |P0| per edge, with want_node_max).
    Y2 (dim_d, 5 chan), bee_rank2_supported(chan, dim_d): the rank-2 output linear is applied inside the kernel and
    the third result is Y2 S2 as (N, dim_d, 9) instead of S2 (mg_bee_message_rank2); with out_d (N dim_d 9 floats,
    contiguous) Y2 S2 is added to out_d in place, which is then the third result."""
    _check_input(row_ptr, "row_ptr", torch.int32)
    _check_input(dst, "dst", torch.int32)
    for t, nm in ((rhat, "rhat"), (enc, "enc"), (La, "La"), (Lv, "Lv"), (Ld, "Ld"), (enc_W, "enc_W"),
                  (enc_b, "enc_b")):
        _check_input(t, nm)
    N, chan = int(La.size(0)), int(La.size(1))
    E = int(dst.numel())
    if tuple(Lv.shape) != (N, 3, chan) or tuple(Ld.shape) != (N, 9, chan):
        raise RuntimeError("Lv / Ld must be component-major (nodes, 3, chan) / (nodes, 9, chan)")
    if tuple(enc.shape) != (E, 8) or tuple(rhat.shape) != (E, 3):
        raise RuntimeError("enc must be (edges, 8) and rhat (edges, 3)")
    if tuple(enc_W.shape) != (chan, 8) or enc_b.numel() != chan:
        raise RuntimeError("enc_W must be (chan, 8) and enc_b (chan)")
    if row_ptr.numel() != N + 1:
        raise RuntimeError("row_ptr must have nodes+1 entries")
    if node_order is not None:
        _check_input(node_order, "node_order", torch.int32)
        if node_order.numel() != N:
            raise RuntimeError("node_order must have one entry per node")
    dev = La.device
    if Y2 is not None:
        if not Y2.is_cuda or Y2.dtype != torch.float32:
            raise RuntimeError("Y2 must be a float32 CUDA tensor")
        if Y2.dim() != 2 or int(Y2.size(1)) != 5 * chan or Y2.stride(1) != 1:
            raise RuntimeError("Y2 must be (dim_d, 5 chan) with unit stride along a row")
        if not bee_rank2_supported(chan, Y2.size(0)):
            raise RuntimeError("the fused rank-2 linear needs chan = 64, 128 or 256 and dim_d <= 16")
    with _on(dev):
        P0 = torch.empty(E, 3, chan, dtype=torch.float32, device=dev)
        S1 = torch.empty(N, 3, 5, chan, dtype=torch.float32, device=dev)
        node_max = torch.empty(N, (chan + 63) // 64, dtype=torch.float32, device=dev) if want_node_max else None
        edge_max = torch.empty(E, (chan + 63) // 64, dtype=torch.float32, device=dev) if want_node_max else None
        if Y2 is not None:
            dim_d = int(Y2.size(0))
            if out_d is not None:
                _check_input(out_d, "out_d")
                if out_d.numel() != N * dim_d * 9:
                    raise RuntimeError("out_d must hold nodes x dim_d x 9 floats")
            S2 = out_d if out_d is not None else torch.empty(N, dim_d, 9, dtype=torch.float32, device=dev)
            L.check(_lib.mg_bee_message_rank2(_p(row_ptr), _p(dst), _p(node_order), N, E, _p(rhat), _p(enc), _p(La),
                                              _p(Lv), _p(Ld), chan, _p(enc_W), _p(enc_b),
                                              _p(_packed_rank2_weight(Y2, chan)), dim_d, _p(P0), _p(S1), _p(S2),
                                              int(out_d is not None), _p(node_max), _p(edge_max), _stream()))
        else:
            S2 = torch.empty(N, 9, 5, chan, dtype=torch.float32, device=dev)
            L.check(_lib.mg_bee_message(_p(row_ptr), _p(dst), _p(node_order), N, E, _p(rhat), _p(enc), _p(La), _p(Lv),
                                        _p(Ld), chan, _p(enc_W), _p(enc_b), _p(P0), _p(S1), _p(S2), _p(node_max),
                                        _p(edge_max), _stream()))
    return (P0, S1, S2, node_max, edge_max) if want_node_max else (P0, S1, S2)


# ------------------------------------------------- norms, squash, update glue
def _chan_view(t, name, lead_dims, chan, comps):
    """t: (*lead, chan, comps...) possibly a channel slice of a wider contiguous buffer.
    Returns the row stride in channels."""
    if not t.is_cuda or t.dtype != torch.float32:
        raise RuntimeError(f"{name} must be a float32 CUDA tensor")
    t3 = t.reshape(-1, chan, comps) if t.is_contiguous() else t
    if t.is_contiguous():
        return chan
    # accept (rows..., chan, comps) views whose only irregularity is a wider row
    comp_dims = t.dim() - lead_dims - 1
    strides, sizes = t.stride(), t.shape
    inner = 1
    for d in range(t.dim() - 1, lead_dims, -1):
        if strides[d] != inner:
            raise RuntimeError(f"{name}: unsupported memory layout")
        inner *= sizes[d]
    if strides[lead_dims] != comps:
        raise RuntimeError(f"{name}: unsupported memory layout")
    row_stride = strides[lead_dims - 1]
    if row_stride % comps != 0:
        raise RuntimeError(f"{name}: unsupported memory layout")
    expect = row_stride
    for d in range(lead_dims - 2, -1, -1):
        expect *= sizes[d + 1]
        if strides[d] != expect:
            raise RuntimeError(f"{name}: unsupported memory layout")
    return row_stride // comps


GN_TENSOR, GN_SCALAR = 0, 1


def group_norm(mode, x, groups, gamma, beta=None, eps=1e-5, mul=None, add=None, res=None):
    """TensGroupNorm (mode 0) / ScalGroupNorm (mode 1) of v = x (* mul), plus optional add and res.
    x: (batch, nodes, chan, (3,)^inds); x, mul and add may be channel slices of wider buffers."""
    B, N, chan = int(x.shape[0]), int(x.shape[1]), int(x.shape[2])
    comps = 1
    for d in x.shape[3:]:
        comps *= int(d)
    xs = _chan_view(x, "x", 2, chan, comps)
    ms = _chan_view(mul, "mul", 2, chan, comps) if mul is not None else 0
    as_ = _chan_view(add, "add", 2, chan, comps) if add is not None else 0
    _check_input(gamma, "gamma")
    if beta is not None:
        _check_input(beta, "beta")
    if res is not None:
        _check_input(res, "res")
        if tuple(res.shape) != tuple(x.shape):
            raise RuntimeError("res has wrong shape")
    nbytes = ctypes.c_size_t(0)
    L.check(_lib.mg_group_norm_scratch_bytes(B, int(groups), ctypes.byref(nbytes)))
    with _on(x.device):
        scratch = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=x.device)
        out = torch.empty(tuple(x.shape), dtype=torch.float32, device=x.device)
        L.check(_lib.mg_group_norm(int(mode), _p(x), xs, _p(mul), ms, B, N, chan, int(groups), comps, float(eps),
                                   _p(gamma), _p(beta), _p(add), as_, _p(res), _p(scratch), _p(out), _stream()))
    return out


def tens_sigmoid(inds, x):
    _check_input(x, "x")
    T = 3 ** inds
    with _on(x.device):
        out = torch.empty_like(x)
        L.check(_lib.mg_tens_sigmoid(int(inds), _p(x), int(x.numel()) // T, _p(out), _stream()))
    return out


def _lrv_layout(lrv, rows, n):
    """1 for component-major (rows, 3, 3n), 0 for the reference's (rows, 3n, 3)."""
    if tuple(lrv.shape) == (rows, 3 * n, 3):
        return 0
    if tuple(lrv.shape) == (rows, 3, 3 * n):
        return 1
    raise RuntimeError("lrv must have shape (rows, 3n, 3) or, component-major, (rows, 3, 3n)")


def painn_update_pre(lrv, x_a, want_rowmax=False):
    """lrv (rows, 3n, 3) or component-major (rows, 3, 3n), x_a (rows, n) -> ip (rows, n), cat (rows, 2n);
    want_rowmax: (ip, cat, rowmax) with rowmax (rows, 1) = max |cat[r, :]| from the same pass (None for n > 256)."""
    _check_input(lrv, "lrv")
    _check_input(x_a, "x_a")
    rows, n = int(x_a.shape[0]), int(x_a.shape[1])
    layout = _lrv_layout(lrv, rows, n)
    with _on(x_a.device):
        ip = torch.empty(rows, n, dtype=torch.float32, device=x_a.device)
        cat = torch.empty(rows, 2 * n, dtype=torch.float32, device=x_a.device)
        rowmax = torch.empty(rows, 1, dtype=torch.float32, device=x_a.device) if want_rowmax and n <= 256 else None
        L.check(_lib.mg_painn_update_pre(_p(lrv), layout, _p(x_a), rows, n, _p(ip), _p(cat), _p(rowmax), _stream()))
    return (ip, cat, rowmax) if want_rowmax else (ip, cat)


def painn_update_vec(lrv, y, res_v=None):
    """v = lin_v(x_v) * y[:, :n]; returns res_v + v / sqrt(1 + |v|^2), shape (rows, n, 3)."""
    _check_input(lrv, "lrv")
    _check_input(y, "y")
    rows, n = int(y.shape[0]), int(y.shape[1]) // 3
    layout = _lrv_layout(lrv, rows, n)
    if res_v is not None:
        _check_input(res_v, "res_v")
    with _on(y.device):
        out = torch.empty(rows, n, 3, dtype=torch.float32, device=y.device)
        L.check(_lib.mg_painn_update_vec(_p(lrv), layout, _p(y), _p(res_v), rows, n, _p(out), _stream()))
    return out


RADIAL_SQ, RADIAL_EDGE = 1, 2


def radial_encode(kind, r_ij, n, rmax):
    """kind 1: sq_radial_encode(normed_sq_dist(r, rmax), n); kind 2: radial_encode_edge(r, n, rmax)."""
    _check_input(r_ij, "r_ij")
    lead = tuple(r_ij.shape[:-1])
    if r_ij.shape[-1] != 3:
        raise RuntimeError("r_ij must have a last dimension of 3")
    E = 1
    for d in lead:
        E *= int(d)
    with _on(r_ij.device):
        out = torch.empty(lead + (n,), dtype=torch.float32, device=r_ij.device)
        L.check(_lib.mg_radial_encode(int(kind), _p(r_ij), E, int(n), float(rmax), _p(out), _stream()))
    return out


def displacement_sums(row_ptr, r_ij, phi, scale):
    """(A_a (N, C), A_v (N, C, 3), A_d (N, C, 3, 3)): sums over the edges of each CSR row of phi, phi (x) u and
    phi (x) u (x) u with u = tens_sigmoid(1, scale * r_ij) (archs/diffuser_atoms15.py:218-224)."""
    _check_input(row_ptr, "row_ptr", torch.int32)
    _check_input(r_ij, "r_ij")
    _check_input(phi, "phi")
    E = int(r_ij.size(0))
    if tuple(r_ij.shape) != (E, 3) or phi.dim() != 2 or phi.size(0) != E:
        raise RuntimeError("r_ij (edges, 3) and phi (edges, chan) expected")
    n_nodes, C = int(row_ptr.numel()) - 1, int(phi.size(1))
    dev = phi.device
    with _on(dev):
        out_a = torch.empty(n_nodes, C, dtype=torch.float32, device=dev)
        out_v = torch.empty(n_nodes, C, 3, dtype=torch.float32, device=dev)
        out_d = torch.empty(n_nodes, C, 3, 3, dtype=torch.float32, device=dev)
        L.check(_lib.mg_displacement_sums(_p(row_ptr), n_nodes, E, _p(r_ij), _p(phi), C, float(scale), _p(out_a),
                                          _p(out_v), _p(out_d), _stream()))
    return out_a, out_v, out_d


# ------------------------------------------------------------------ data generator
def repel5_sim(x, v, drag, T, dt, nsteps, seed, first_kick=0):
    """Langevin dynamics of bead chains in place (polymer_sim(SimId.REPEL5, ...) of
    extensions/polymer_sims_cuda/polymer_sims.cpp:17-47): x, v (batch, n, 3), drag (n).  seed, first_kick: the
    noise of velocity update first_kick + s of bead b is a pure function of (seed, b, first_kick + s)."""
    for t, nm in ((x, "x"), (v, "v"), (drag, "drag")):
        _check_input(t, nm)
    if x.dim() != 3 or v.dim() != 3 or drag.dim() != 1:
        raise RuntimeError("Input tensors must have correct dimensions")
    if x.size(0) != v.size(0):
        raise RuntimeError("Batch sizes must match")
    if x.size(1) != v.size(1) or x.size(1) != drag.size(0):
        raise RuntimeError("Number of particles must match")
    if x.size(2) != 3 or v.size(2) != 3:
        raise RuntimeError("Position and velocity must be 3D")
    with _on(x.device):
        L.check(_lib.mg_repel5_sim(_p(x), _p(v), _p(drag), float(T), float(dt), int(nsteps), int(x.size(0)),
                                   int(x.size(1)), int(seed) & 0xFFFFFFFFFFFFFFFF, int(first_kick), _stream()))


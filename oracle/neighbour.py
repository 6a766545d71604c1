"""TEST INFRASTRUCTURE ONLY — Python front end of neighbour_oracle.c.

`get_edges` mirrors the call signature and error behaviour of the reference's
extensions/neighbour_grid/neighbour_grid.cpp:170-195 (get_edges) on numpy
arrays; `boxwrap` / `image_shift` restate managan/graph_layers.py:62-66 and the
derived periodic-image triple.
"""
import ctypes
import numpy as np

from . import build

MODE_CELLS = 0          # the reference's walk: cells, then 3x3x3 window
MODE_BRUTE_WINDOW = 1   # all pairs, with the reference's cell-adjacency predicate
MODE_BRUTE_MINIMAGE = 2  # all pairs, textbook minimum image

_lib = None


def lib():
    global _lib
    if _lib is None:
        L = ctypes.CDLL(build())
        fp = ctypes.POINTER(ctypes.c_float)
        ip = ctypes.POINTER(ctypes.c_int)
        lp = ctypes.POINTER(ctypes.c_long)
        L.nbr_oracle_edges.restype = ctypes.c_long
        L.nbr_oracle_edges.argtypes = [fp, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                       ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int,
                                       ip, ip, ctypes.c_long, ip, ip, lp]
        L.nbr_oracle_ndiv.restype = ctypes.c_int
        L.nbr_oracle_ndiv.argtypes = [ctypes.c_float] * 4 + [ip]
        L.nbr_oracle_wrap_cells.restype = None
        L.nbr_oracle_wrap_cells.argtypes = [fp, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                            ctypes.c_float, ctypes.c_float, ctypes.c_float, fp, ip]
        L.nbr_oracle_remainderf.restype = ctypes.c_float
        L.nbr_oracle_remainderf.argtypes = [ctypes.c_float, ctypes.c_float]
        _lib = L
    return _lib


def _fptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _iptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int))


def ndiv(cutoff, box):
    out = (ctypes.c_int * 3)()
    rc = lib().nbr_oracle_ndiv(cutoff, box[0], box[1], box[2], out)
    return tuple(out), rc == 0


def wrap_cells(x, cutoff, box):
    x = np.ascontiguousarray(x, dtype=np.float32)
    B, N, _ = x.shape
    w = np.empty_like(x)
    cell = np.empty((B, N), dtype=np.int32)
    lib().nbr_oracle_wrap_cells(_fptr(x), B, N, cutoff, box[0], box[1], box[2], _fptr(w), _iptr(cell))
    return w, cell


def edges(x, cutoff, box, mode=MODE_CELLS):
    """x: (B,N,3) float32.  Returns dict(src,dst,counts,edge_counts,max_cell,max_degree,borderline).
    Rows ordered by (b,i); dst ascending inside a row."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.ndim == 3 and x.shape[2] == 3, "x must have shape (batch, nodes, 3)"
    B, N, _ = x.shape
    counts = np.zeros((B, N), dtype=np.int32)
    edge_counts = np.zeros((B,), dtype=np.int32)
    stats = (ctypes.c_long * 3)()
    null = ctypes.POINTER(ctypes.c_int)()
    E = lib().nbr_oracle_edges(_fptr(x), B, N, cutoff, box[0], box[1], box[2], mode,
                               null, null, 0, _iptr(counts), _iptr(edge_counts), stats)
    if E == -1:
        raise RuntimeError("box dimension must be greater than 3*cutoff")
    if E < 0:
        raise MemoryError("oracle allocation failed")
    src = np.empty((E,), dtype=np.int32)
    dst = np.empty((E,), dtype=np.int32)
    if E > 0:
        lib().nbr_oracle_edges(_fptr(x), B, N, cutoff, box[0], box[1], box[2], mode,
                               _iptr(src), _iptr(dst), E, null, null, None)
    return dict(src=src, dst=dst, counts=counts, edge_counts=edge_counts,
                max_cell=int(stats[0]), max_degree=int(stats[1]), borderline=int(stats[2]))


def get_edges(listmax, neighboursmax, cutoff, box_x, box_y, box_z, x, mode=MODE_CELLS):
    """Same argument order, outputs and errors as the reference's get_edges."""
    r = edges(x, cutoff, (box_x, box_y, box_z), mode)
    if r["max_cell"] > listmax:
        raise RuntimeError("Cell list overflow occurred. Trying increasing listmax.")
    if listmax not in (32, 64, 128, 256):
        raise RuntimeError("expected listmax to be one of 32, 64, 128, 256. other values not supported!")
    if r["max_degree"] > neighboursmax:
        raise RuntimeError("Neighbour list overflow occurred. Try increasing neighboursmax.")
    return r["src"], r["dst"], r["edge_counts"]


def boxwrap(box, delta_pos):
    """(delta + box/2) floor-mod box - box/2 in float32 (managan/graph_layers.py:62-66)."""
    box = np.asarray(box, dtype=np.float32)
    d = np.asarray(delta_pos, dtype=np.float32)
    half = np.float32(0.5) * box
    return np.mod(d + half, box).astype(np.float32) - half


def edge_vectors(x, src, dst, box):
    """r_ij = boxwrap(pos[dst] - pos[src]) from the UNWRAPPED inputs, fp32."""
    flat = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 3)
    return boxwrap(box, flat[dst] - flat[src])


def image_shift(x, src, dst, box):
    """Periodic-image triple derived from the edge list: rint(((x_j - x_i) - r_ij)/box)."""
    flat = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 3)
    raw = flat[dst] - flat[src]
    r = boxwrap(box, raw)
    return np.rint((raw - r) / np.asarray(box, dtype=np.float32)).astype(np.int32)


def sorted_triples(src, dst, shift=None):
    """Canonical ordering for set comparison."""
    cols = [np.asarray(src, dtype=np.int64), np.asarray(dst, dtype=np.int64)]
    if shift is not None:
        s = np.asarray(shift, dtype=np.int64)
        cols += [s[:, 0], s[:, 1], s[:, 2]]
    arr = np.stack(cols, axis=1)
    order = np.lexsort(arr.T[::-1])
    return arr[order]

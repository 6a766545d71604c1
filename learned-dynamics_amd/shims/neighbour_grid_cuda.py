"""Drop-in for the reference's `neighbour_grid_cuda` extension
(extensions/neighbour_grid/neighbour_grid.cpp:198-203), backed by HIP kernels."""
import importlib

_ops = importlib.import_module("learned-dynamics_amd.ops")


def get_edges(listmax, neighboursmax, cutoff, box_x, box_y, box_z, x):
    """Like get_neighbours, except it returns lists of edge tensors."""
    return _ops.get_edges(listmax, neighboursmax, cutoff, box_x, box_y, box_z, x)


def get_neighbours(listmax, neighboursmax, cutoff, box_x, box_y, box_z, x):
    """Define neighbours based on cutoff radius using a grid method."""
    return _ops.get_neighbours(listmax, neighboursmax, cutoff, box_x, box_y, box_z, x)


def edges_read(neighbourCounts, neighbours, x):
    """Read data from nodes to edges."""
    return _ops.padded_edges_read(neighbourCounts, neighbours, x)


def edges_reduce(neighbourCounts, neighbours, x):
    """Reduce data from edges to nodes."""
    return _ops.padded_edges_reduce(neighbourCounts, neighbours, x)

"""Pins the C neighbour-search oracle: the reference's golden 5-point case, its
invariants (symmetry, no self edges, sorted src, counts), and brute force.
Also proves the branch-based minimum image the HIP kernel uses equal to libm's
remainderf on the operand range it is applied to."""
import ctypes

import numpy as np
import pytest

from conftest import load_golden
from oracle import neighbour as ON

FIVE = load_golden("graph_layers_five_points")      # managan/graph_layers.py:83-122


def test_golden_five_points():
    # managan/graph_layers.py:83-103: r0=2, box 100 connects (0,1) and (1,2,3)
    pos = np.array(FIVE["positions"], dtype=np.float32)
    box = tuple(FIVE["box"])
    for mode in (ON.MODE_CELLS, ON.MODE_BRUTE_WINDOW, ON.MODE_BRUTE_MINIMAGE):
        r = ON.edges(pos, FIVE["radius"], box, mode)
        assert r["counts"].tolist() == FIVE["degrees"]
        assert set(zip(r["src"].tolist(), r["dst"].tolist())) == {tuple(e) for e in FIVE["edges"]}
        assert r["edge_counts"].tolist() == [len(FIVE["edges"])]
    src, dst, ec = ON.get_edges(32, 64, FIVE["radius"], *box, pos)
    assert np.all(src[1:] >= src[:-1])
    # boxwrap bound of the same self test (graph_layers.py:120-122)
    d = ON.edge_vectors(pos, src, dst, box)
    assert np.all((d ** 2).sum(-1) < FIVE["wrapped_length_bound"] ** 2)


def test_golden_sumprod_through_oracle_scatter():
    """graph_layers.py:106-117: sum_j x_i x_j 'calculated on paper'."""
    import torch
    from oracle import layers as OL
    pos = np.array(FIVE["positions"], dtype=np.float32)
    src, dst, _ = ON.get_edges(32, 64, FIVE["radius"], *FIVE["box"], pos)
    src_t, dst_t = torch.from_numpy(src).long(), torch.from_numpy(dst).long()
    x = torch.arange(5).float().repeat(4).reshape(1, 5, 4)
    flat = x.reshape(5, 4)
    sumprod = OL.edges_reduce_src(src_t, flat[src_t] * OL.edges_read_dst(dst_t, x, 1, 5), 1, 5)
    assert torch.equal(sumprod, torch.tensor(FIVE["sum_of_products"]))
    deg = OL.edges_reduce_src(src_t, torch.ones(len(src)), 1, 5)
    assert deg.tolist() == FIVE["degrees"]


def test_reference_invariants_on_its_test_shape():
    # extensions/neighbour_grid/test.py:9-33: B=20, N=60, box (30.5,33.5,36.5), cutoff 7
    rng = np.random.default_rng(0x947)
    box = (30.5, 33.5, 36.5)
    x = (rng.random((20, 60, 3)) * np.array(box)).astype(np.float32)
    r = ON.edges(x, 7.0, box)
    E = set(zip(r["src"].tolist(), r["dst"].tolist()))
    assert all((b, a) in E for a, b in E), "adjacency must be symmetric"
    assert all(a != b for a, b in E)
    assert all(a // 60 == b // 60 for a, b in E), "edges stay inside their box"
    assert np.all(np.diff(r["src"]) >= 0)
    assert np.array_equal(np.bincount(r["src"], minlength=1200), r["counts"].reshape(-1))
    assert np.array_equal(np.cumsum(r["counts"].sum(1)), r["edge_counts"])


@pytest.mark.parametrize("box,cutoff", [((30., 30., 30.), 5.0), ((30.5, 33.5, 36.5), 7.0), ((70., 70., 70.), 6.0),
                                        ((9., 12., 15.), 3.0)])
def test_cell_walk_equals_brute_force_with_window_predicate(box, cutoff):
    rng = np.random.default_rng(1)
    x = ((rng.random((2, 1500, 3)) * 3 - 1) * np.array(box)).astype(np.float32)
    a = ON.edges(x, cutoff, box, ON.MODE_CELLS)
    b = ON.edges(x, cutoff, box, ON.MODE_BRUTE_WINDOW)
    assert np.array_equal(a["src"], b["src"]) and np.array_equal(a["dst"], b["dst"])


def test_integer_ratio_equals_textbook_minimum_image():
    """When box/cutoff is an integer in every dimension the window predicate is vacuous."""
    rng = np.random.default_rng(2)
    box = (20., 25., 30.)
    x = (rng.random((1, 2500, 3)) * np.array(box)).astype(np.float32)
    a = ON.edges(x, 5.0, box, ON.MODE_CELLS)
    c = ON.edges(x, 5.0, box, ON.MODE_BRUTE_MINIMAGE)
    assert np.array_equal(a["src"], c["src"]) and np.array_equal(a["dst"], c["dst"])
    # independent float64 check of the same graph, ignoring pairs within 1e-4 of the cutoff
    p = x[0].astype(np.float64)
    d = p[:, None, :] - p[None, :, :]
    d -= np.array(box) * np.round(d / np.array(box))
    dist = np.sqrt((d ** 2).sum(-1))
    np.fill_diagonal(dist, 1e9)
    sure_in = set(zip(*np.nonzero(dist < 5.0 - 1e-4)))
    maybe = set(zip(*np.nonzero(dist < 5.0 + 1e-4)))
    got = set(zip(a["src"].tolist(), a["dst"].tolist()))
    assert sure_in <= got <= maybe


def test_under_resolved_grid_drops_pairs_two_cells_apart():
    """box/cutoff = 70/6 -> 12 cells of 5.83 A < cutoff: the reference misses some pairs."""
    rng = np.random.default_rng(3)
    box = (70., 70., 70.)
    x = (rng.random((1, 30000, 3)) * 70).astype(np.float32)
    a = ON.edges(x, 6.0, box, ON.MODE_CELLS)
    assert a["max_degree"] > 0
    w, cell = ON.wrap_cells(x, 6.0, box)
    # every listed pair sits in adjacent cells (per axis, periodically)
    cs, cd = cell.reshape(-1)[a["src"]], cell.reshape(-1)[a["dst"]]
    for axis_div in (144, 12, 1):
        ds = ((cs // axis_div) % 12 - (cd // axis_div) % 12) % 12
        assert np.all((ds == 0) | (ds == 1) | (ds == 11))


def test_rint_fma_minimum_image_equals_remainderf_wherever_a_pair_can_be_listed():
    """The HIP kernels evaluate remainder(t, box) for t = a - b, a, b in [0, box], as fma(-rint(t * (1 / box)), box, t).
    The multiple is -1, 0 or 1 and the fma is exact, so the value equals libm's remainderf bit for bit, except that
    for t / box within rounding of +-1/2 the other representative (t + box instead of t, ...) may be chosen.  There the
    magnitude of either representative is about box / 2 > cutoff (at least 3 cells per axis), so no listed pair can
    be affected: the test demands exact equality everywhere else and |value| > 0.49 box where the two differ."""
    L = ON.lib()
    rng = np.random.default_rng(5)
    rem = np.vectorize(lambda a, b: L.nbr_oracle_remainderf(a, b), otypes=[np.float32])
    for box in (np.float32(55.0), np.float32(30.5), np.float32(86.861), np.float32(7.3), np.float32(70.0)):
        half = np.float32(0.5) * box
        a = (rng.random(200000).astype(np.float32) * box).astype(np.float32)
        b = (rng.random(200000).astype(np.float32) * box).astype(np.float32)
        a[:8] = [box, 0, half, box, half, 0, np.nextafter(half, box), np.nextafter(half, np.float32(0))]
        b[:8] = [0, box, 0, half, box, half, 0, 0]
        # and many operands right around the tie
        a[8:5000] = (half + (rng.random(4992) - 0.5) * 1e-5 * float(box)).astype(np.float32)
        b[8:5000] = 0
        t = (a - b).astype(np.float32)
        inv = (np.float32(1.0) / box).astype(np.float32)
        r = np.rint((t * inv).astype(np.float32)).astype(np.float32)
        assert set(np.unique(r)) <= {-1.0, 0.0, 1.0}
        got = (t.astype(np.float64) - r.astype(np.float64) * float(box)).astype(np.float32)       # the fma: exact, rounded once
        assert np.array_equal(got.astype(np.float64), t.astype(np.float64) - r.astype(np.float64) * float(box))   # nothing to round
        ref = rem(t, np.full_like(t, box))
        differ = (got * got).view(np.uint32) != (ref * ref).view(np.uint32)
        assert np.all(np.abs(got[differ]) > 0.49 * box) and np.all(np.abs(ref[differ]) > 0.49 * box)
        assert differ.sum() < 5000


def test_branch_wrap_equals_remainderf():
    """d = a - b with a, b in [0, box]; one conditional +-box must equal remainderf(d, box)."""
    L = ON.lib()
    rng = np.random.default_rng(4)
    rem = np.vectorize(lambda a, b: L.nbr_oracle_remainderf(a, b), otypes=[np.float32])
    for box in (np.float32(55.0), np.float32(30.5), np.float32(86.861), np.float32(7.3)):
        half = np.float32(0.5) * box
        a = (rng.random(20000).astype(np.float32) * box).astype(np.float32)
        b = (rng.random(20000).astype(np.float32) * box).astype(np.float32)
        # ties and end points
        a[:6] = [box, 0, half, box, half, 0]
        b[:6] = [0, box, 0, half, box, half]
        d = (a - b).astype(np.float32)
        branch = np.where(d > half, d - box, np.where(d < -half, d + box, d)).astype(np.float32)
        ref = rem(d, np.full_like(d, box))
        # identical values; only the sign of a zero result may differ (d = -box gives +0 here,
        # -0 in libm), which the squared distance cannot see
        assert np.array_equal(branch, ref)
        assert np.array_equal((branch * branch).view(np.uint32), (ref * ref).view(np.uint32))


def test_overflow_and_argument_errors():
    rng = np.random.default_rng(5)
    x = (rng.random((1, 400, 3)) * 9).astype(np.float32)
    with pytest.raises(RuntimeError, match="greater than 3\\*cutoff"):
        ON.get_edges(32, 64, 5.5, 10., 10., 10., x)   # ceil(10/5.5) = 2 cells
    with pytest.raises(RuntimeError, match="Cell list overflow"):
        ON.get_edges(4, 1000, 3.0, 9., 9., 9., x)
    with pytest.raises(RuntimeError, match="one of 32, 64, 128, 256"):
        ON.get_edges(100, 1000, 3.0, 9., 9., 9., x)
    with pytest.raises(RuntimeError, match="Neighbour list overflow"):
        ON.get_edges(32, 2, 3.0, 9., 9., 9., x)


def test_image_shift_reconstructs_displacement():
    rng = np.random.default_rng(6)
    box = (20., 25., 30.)
    x = ((rng.random((1, 800, 3)) * 5 - 2) * np.array(box)).astype(np.float32)
    r = ON.edges(x, 5.0, box)
    shift = ON.image_shift(x, r["src"], r["dst"], box)
    flat = x.reshape(-1, 3).astype(np.float64)
    recon = flat[r["dst"]] - flat[r["src"]] - shift * np.array(box)
    assert np.all(np.sqrt((recon ** 2).sum(-1)) <= 5.0 + 1e-3)


# ---- atoms exactly on the periodic faces (wrapped coordinate == box, filed in cell 0) ---------------------
def test_two_atoms_across_the_face_are_neighbours():
    """box 70, cutoff 6 (12 cells of 5.83): x = 70.0 wraps to exactly 70.0 and is filed in cell 0; its partner at
    x = 5.9 sits in cell 1, 5.9 away through the face.  The reference applies the minimum image to every pair
    (neighbour_grid_kern.cu:44-48,135), so both directions are listed."""
    import neighbour_cases as NC
    for axis in range(3):
        x = np.zeros((1, 2, 3), dtype=np.float32)
        x[0, 0, axis], x[0, 1, axis] = 5.9, 70.0
        w, cell = ON.wrap_cells(x, 6.0, (70., 70., 70.))
        assert w[0, 1, axis] == np.float32(70.0) and cell[0, 1] == 0 and cell[0, 0] != 0
        for mode in (ON.MODE_CELLS, ON.MODE_BRUTE_WINDOW, ON.MODE_BRUTE_MINIMAGE):
            r = ON.edges(x, 6.0, (70., 70., 70.), mode)
            assert set(zip(r["src"].tolist(), r["dst"].tolist())) == {(0, 1), (1, 0)}
    assert NC.face_values(70.)[0] == np.float32(70.)


@pytest.mark.parametrize("box,cutoff", __import__("neighbour_cases").FACE_BOXES)
def test_face_atoms_cell_walk_equals_brute_force(box, cutoff):
    import neighbour_cases as NC
    for axis in range(3):
        x = NC.hand_placed_line(box, cutoff, axis)
        w, cell = ON.wrap_cells(x, cutoff, box)
        nd, _ = ON.ndiv(cutoff, box)
        a = ON.edges(x, cutoff, box, ON.MODE_CELLS)
        b = ON.edges(x, cutoff, box, ON.MODE_BRUTE_WINDOW)
        np.testing.assert_array_equal(ON.sorted_triples(a["src"], a["dst"]), ON.sorted_triples(b["src"], b["dst"]))
        # the case the test exists for is present: an edge from an atom whose axis cell is 1 to an atom whose wrapped
        # coordinate is exactly `box`
        stride = [nd[1] * nd[2], nd[2], 1][axis]
        axis_cell = (cell[0] // stride) % nd[axis]
        on_face = w[0, :, axis] == np.float32(box[axis])
        assert np.any((axis_cell[a["src"]] == 1) & on_face[a["dst"]])
        E = set(zip(a["src"].tolist(), a["dst"].tolist()))
        assert all((j, i) in E for i, j in E)
    x = NC.snapped_random(box, 1500, 2, seed=3)
    a = ON.edges(x, cutoff, box, ON.MODE_CELLS)
    b = ON.edges(x, cutoff, box, ON.MODE_BRUTE_WINDOW)
    np.testing.assert_array_equal(ON.sorted_triples(a["src"], a["dst"]), ON.sorted_triples(b["src"], b["dst"]))

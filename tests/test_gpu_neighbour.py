"""HIP periodic neighbour search against the C oracle: sorted (src, dst, image
shift) edge sets must be bit-identical."""
import importlib

import numpy as np
import pytest
import torch

from conftest import load_golden
from oracle import neighbour as ON

pytestmark = pytest.mark.gpu


def _triples(src, dst, shift=None):
    return ON.sorted_triples(np.asarray(src), np.asarray(dst), None if shift is None else np.asarray(shift))


def _run(ops, x, cutoff, box, listmax=None, nmax=None):
    xt = torch.from_numpy(x).cuda()
    if listmax is not None:
        src, dst, ec, row_ptr = ops.get_edges(listmax, nmax, cutoff, *box, xt, return_row_ptr=True)
    else:   # exact-size search without the reference's caps
        search = ops.NeighbourSearch(xt, cutoff, box)
        src, dst = search.fill()
        ec, row_ptr = search.edge_counts, search.row_ptr
    return xt, src, dst, ec, row_ptr


def _compare(ops, x, cutoff, box, mode=ON.MODE_CELLS):
    xt, src, dst, ec, row_ptr = _run(ops, x, cutoff, box)
    ref = ON.edges(x, cutoff, box, mode)
    s, d = src.cpu().numpy(), dst.cpu().numpy()
    assert len(s) == len(ref["src"]), (len(s), len(ref["src"]))
    assert np.all(s[1:] >= s[:-1]), "src must be non-decreasing"
    np.testing.assert_array_equal(ec.cpu().numpy(), ref["edge_counts"])
    np.testing.assert_array_equal(np.diff(row_ptr.cpu().numpy()), ref["counts"].reshape(-1))
    np.testing.assert_array_equal(_triples(s, d), _triples(ref["src"], ref["dst"]))
    # derived quantities: r_ij and the periodic image shift
    r, shift = ops.edge_vectors(xt.reshape(-1, 3), src, dst, box, want_shift=True)
    np.testing.assert_array_equal(r.cpu().numpy(), ON.edge_vectors(x, s, d, box))
    ref_shift = ON.image_shift(x, ref["src"], ref["dst"], box)
    np.testing.assert_array_equal(_triples(s, d, shift.cpu().numpy()),
                                  _triples(ref["src"], ref["dst"], ref_shift))
    return ref


def test_golden_five_points(ops):
    """Hand-placed points of the reference's self test (managan/graph_layers.py:83-103)."""
    five = load_golden("graph_layers_five_points")
    pos = np.array(five["positions"], dtype=np.float32)
    xt, src, dst, ec, row_ptr = _run(ops, pos, five["radius"], tuple(five["box"]), listmax=32, nmax=64)
    assert np.array_equal(np.diff(row_ptr.cpu().numpy()), five["degrees"][0])
    got = set(zip(src.tolist(), dst.tolist()))
    assert got == {tuple(e) for e in five["edges"]}
    assert ec.tolist() == [len(five["edges"])]


def test_wrap_cells_bit_exact(ops):
    rng = np.random.default_rng(5)
    box = (30.5, 33.5, 36.5)
    x = ((rng.random((4, 5000, 3)) * 5 - 2) * np.array(box)).astype(np.float32)
    x[0, :10] = np.array(box, dtype=np.float32) * np.array([0.5, 1.0, 0.0], dtype=np.float32)  # ties / edges
    w, cell = ops.wrap_cells(7.0, box, torch.from_numpy(x).cuda())
    w_ref, cell_ref = ON.wrap_cells(x, 7.0, box)
    np.testing.assert_array_equal(w.cpu().numpy(), w_ref)
    np.testing.assert_array_equal(cell.cpu().numpy(), cell_ref)


@pytest.mark.parametrize("box,cutoff", __import__("neighbour_cases").FACE_BOXES)
def test_atoms_on_the_box_faces(ops, box, cutoff):
    """Wrapped coordinate exactly `box` (x = box, -box, 3 box, nextafter(box, 0)): the atom is filed in cell 0 and its
    partners in cell 1 are reached only through the minimum image (neighbour_grid_kern.cu:39-48,75-80,124-139).  Cells
    narrower than the cutoff (70/6, 86.861/6) and exact cells (55/5), all three axes, then a random box with 5 % of
    the coordinates snapped to such values."""
    import neighbour_cases as NC
    for axis in range(3):
        ref = _compare(ops, NC.hand_placed_line(box, cutoff, axis), cutoff, box)
        E = set(zip(ref["src"].tolist(), ref["dst"].tolist()))
        assert all((j, i) in E for i, j in E)
    _compare(ops, NC.snapped_random(box, 6000, 3, seed=29), cutoff, box)
    _compare(ops, NC.snapped_random(box, 300, 2, seed=31), cutoff, box)      # sparse: one-wave workgroups


def test_fill_capacity_is_never_exceeded(ops):
    """src / dst shorter than the edge count: nothing is written past them and the leading rows are intact."""
    rng = np.random.default_rng(37)
    x = torch.from_numpy((rng.random((2, 3000, 3)) * 30).astype(np.float32)).cuda()
    search = ops.NeighbourSearch(x, 5.0, (30., 30., 30.))
    E = search.host_stats()[0]
    full_src, full_dst = search.fill()
    cap = E // 2
    guard = 4096
    src = torch.full((cap + guard,), -7, dtype=torch.int32, device="cuda")
    dst = torch.full((cap + guard,), -7, dtype=torch.int32, device="cuda")
    search.fill_into(src[:cap], dst[:cap])
    assert torch.equal(src[:cap], full_src[:cap]) and torch.equal(dst[:cap], full_dst[:cap])
    assert torch.all(src[cap:] == -7) and torch.all(dst[cap:] == -7)


def test_one_call_search_into_caller_sized_arrays(ops):
    """mg_neighbour_edges: count + fill in one enqueue; with enough capacity the result is the two-phase result, with
    less the leading edges; buffers can be reused for another set of positions."""
    rng = np.random.default_rng(41)
    box = (30., 30., 30.)
    x = torch.from_numpy((rng.random((2, 3000, 3)) * 30).astype(np.float32)).cuda()
    search = ops.NeighbourSearch(x, 5.0, box)
    E = search.host_stats()[0]
    src, dst = search.fill()
    out = ops.neighbour_edges(x, 5.0, box, E + 100)
    assert out["stats"].tolist() == list(search.host_stats())
    assert torch.equal(out["src"][:E], src) and torch.equal(out["dst"][:E], dst)
    assert torch.equal(out["row_ptr"], search.row_ptr) and torch.equal(out["edge_counts"], search.edge_counts)
    x2 = torch.from_numpy((rng.random((2, 3000, 3)) * 30).astype(np.float32)).cuda()
    ops.neighbour_edges(x2, 5.0, box, None, out=out)
    s2 = ops.NeighbourSearch(x2, 5.0, box)
    E2 = s2.host_stats()[0]
    src2, dst2 = s2.fill()
    n = min(E2, E + 100)
    assert int(out["stats"][0]) == E2 and torch.equal(out["src"][:n], src2[:n]) and torch.equal(out["dst"][:n], dst2[:n])
    small = ops.neighbour_edges(x, 5.0, box, E // 3)
    assert int(small["stats"][0]) == E and torch.equal(small["src"], src[:E // 3]) and torch.equal(small["dst"], dst[:E // 3])


def test_reference_test_shape(ops):
    """B=20, N=60, box (30.5,33.5,36.5), cutoff 7 (extensions/neighbour_grid/test.py:9-16)."""
    g = torch.Generator().manual_seed(0x947)
    box = (30.5, 33.5, 36.5)
    x = (torch.rand(20, 60, 3, generator=g) * torch.tensor(box)).numpy()
    ref = _compare(ops, x, 7.0, box)
    # adjacency symmetric (test.py:22-32)
    E = set(zip(ref["src"].tolist(), ref["dst"].tolist()))
    assert all((b, a) in E for a, b in E)


def test_unwrapped_and_clustered(ops):
    """Positions far outside the box, all atoms of one box in one cell, and an empty-ish box."""
    rng = np.random.default_rng(7)
    box = (24., 27., 31.)
    x = (rng.standard_normal((3, 700, 3)) * 40).astype(np.float32)
    x[1] = (rng.random((700, 3)) * 2.0 + 500.0).astype(np.float32)      # dense cluster: degree 699
    _compare(ops, x, 8.0, box)


def test_under_resolved_grid(ops):
    """box/cutoff not an integer: the 3x3x3 window misses pairs two cells apart; the HIP path
    must reproduce the reference's set, which differs from the plain minimum-image graph."""
    rng = np.random.default_rng(11)
    box = (70., 70., 70.)
    x = (rng.random((2, 20000, 3)) * 70).astype(np.float32)
    ref = _compare(ops, x, 6.0, box)
    assert ref["max_degree"] > 0


def test_sparse_box_uses_single_wave_blocks(ops):
    rng = np.random.default_rng(13)
    box = (70., 70., 70.)
    x = (rng.random((32, 2048, 3)) * 70).astype(np.float32)
    _compare(ops, x, 6.0, box)


@pytest.mark.parametrize("nodes,clump,box_len", [(2000, 600, 60.), (5000, 300, 30.)])
def test_rows_longer_than_a_hit_row_next_to_short_ones(ops, nodes, clump, box_len):
    """The count pass leaves each atom's neighbours in a row of 256 entries and the fill pass copies the rows; atoms of
    a clump have more neighbours than that and are swept again by the fill pass.  Both kinds of rows sit in one
    workgroup's range here, in the one-wave variant of the count pass (1.2 atoms per cell on average, and a clump whose
    window is larger than that variant's tile of 512) and in the four-wave variant; the clump straddles a box face."""
    rng = np.random.default_rng(nodes)
    box = (box_len,) * 3
    x = (rng.random((2, nodes, 3)) * box_len).astype(np.float32)
    x[0, ::nodes // clump][:clump] = (rng.standard_normal((clump, 3)) * 0.8 + np.array([box_len - 0.5, 14., 0.2])).astype(np.float32)
    ref = _compare(ops, x, 5.0, box)
    degrees = ref["counts"].reshape(-1)
    assert degrees.max() >= clump - 1 and degrees.min() < 150


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_and_densities(ops, seed):
    """Boxes, atom counts and densities drawn at random (1 to 4 boxes of 1 to 6000 atoms, 3 to 14 cells per axis,
    anisotropic, a third of them with a clump and a tenth of the coordinates outside the box): every variant of the
    sort (1 to 5 slabs per box), of the count pass (one and four waves per cell) and of the fill pass (copied and
    re-swept rows) against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    batch = int(rng.integers(1, 5))
    nodes = int(rng.choice([1, 2, 63, 64, 65, 300, 1023, 1025, 2500, 6000]))
    cutoff = float(rng.uniform(2.0, 7.0))
    box = tuple(float(cutoff * rng.uniform(3.05, 14.0)) for _ in range(3))
    x = (rng.random((batch, nodes, 3)) * np.array(box)).astype(np.float32)
    if seed % 3 == 0 and nodes >= 64:
        k = nodes // 4
        x[0, :k] = (rng.standard_normal((k, 3)) * 0.5 * cutoff + np.array(box) * rng.random(3)).astype(np.float32)
    far = rng.random((batch, nodes)) < 0.1
    x[far] += (rng.integers(-3, 4, size=(int(far.sum()), 3)) * np.array(box)).astype(np.float32)
    _compare(ops, np.ascontiguousarray(x), cutoff, box)


def test_many_candidates_exceed_lds_tile(ops):
    """More candidates in a 27-cell window than the LDS tile holds (1024): the tail is read from global
    memory, and every row is longer than a hit row, so the fill pass sweeps every window again."""
    rng = np.random.default_rng(17)
    box = (12., 12., 12.)
    x = (rng.random((1, 3000, 3)) * 12).astype(np.float32)     # 27 cells of 4 A: ~111 atoms per cell
    _compare(ops, x, 4.0, box)


def test_config2_one_box(ops):
    g = torch.Generator().manual_seed(0x947 + 2)
    x = (torch.rand(8, 16384, 3, generator=g) * 55).numpy()[:2]
    ref = _compare(ops, np.ascontiguousarray(x), 5.0, (55., 55., 55.))
    assert 1_600_000 < len(ref["src"]) < 1_800_000


def test_errors(ops):
    x = torch.rand(1, 100, 3).cuda() * 10
    with pytest.raises(RuntimeError, match="greater than 3\\*cutoff"):
        ops.get_edges(32, 64, 5.5, 10., 10., 10., x)   # ceil(10/5.5) = 2 cells
    dense = torch.rand(1, 400, 3).cuda() * 9
    with pytest.raises(RuntimeError, match="Cell list overflow"):
        ops.get_edges(4, 1000, 3.0, 9., 9., 9., dense)
    with pytest.raises(RuntimeError, match="one of 32, 64, 128, 256"):
        ops.get_edges(100, 1000, 3.0, 9., 9., 9., dense)
    with pytest.raises(RuntimeError, match="Neighbour list overflow"):
        ops.get_edges(32, 2, 3.0, 9., 9., 9., dense)
    with pytest.raises(RuntimeError, match="shape"):
        ops.get_edges(32, 64, 3.0, 9., 9., 9., torch.rand(100, 3).cuda())
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.get_edges(32, 64, 3.0, 9., 9., 9., torch.rand(1, 3, 100).cuda().transpose(1, 2))
    with pytest.raises(RuntimeError, match="CUDA"):
        ops.get_edges(32, 64, 3.0, 9., 9., 9., torch.rand(1, 100, 3))


def test_empty(ops):
    src, dst, ec = ops.get_edges(32, 64, 3.0, 9., 9., 9., torch.empty(0, 10, 3).cuda())
    assert src.numel() == 0 and ec.numel() == 0
    src, dst, ec = ops.get_edges(32, 64, 3.0, 9., 9., 9., torch.empty(2, 0, 3).cuda())
    assert src.numel() == 0 and ec.tolist() == [0, 0]
    src, dst, ec = ops.get_edges(32, 64, 1.0, 90., 90., 90., torch.rand(2, 5, 3).cuda() * 90)
    assert ec.numel() == 2


def test_deterministic_order(ops):
    rng = np.random.default_rng(19)
    x = torch.from_numpy((rng.random((2, 4000, 3)) * 30).astype(np.float32)).cuda()
    a = ops.get_edges(64, 512, 5.0, 30., 30., 30., x)
    b = ops.get_edges(64, 512, 5.0, 30., 30., 30., x)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_padded_api(ops):
    """get_neighbours / edges_read / edges_reduce invariants (extensions/neighbour_grid/test.py:35-46)."""
    g = torch.Generator().manual_seed(3)
    box = (30.5, 33.5, 36.5)
    x = (torch.rand(20, 60, 3, generator=g) * torch.tensor(box)).cuda()
    neighbours, counts = ops.get_neighbours(32, 32, 7.0, *box, x)
    idx = torch.arange(60, device="cuda")[None, :, None].expand(20, -1, -1).contiguous().float()
    read = ops.padded_edges_read(counts, neighbours, idx)
    mask = torch.arange(32, device="cuda")[None, None, :] < counts[:, :, None]
    assert torch.equal(read[..., 0][mask], neighbours[mask].float())
    assert torch.all(read[..., 0][~mask] == 0)
    ones = torch.ones(20, 60, 7, device="cuda")
    red = ops.padded_edges_reduce(counts, neighbours, ops.padded_edges_read(counts, neighbours, ones))
    assert torch.equal(red[:, :, 0], counts.float())


def test_cell_order_is_a_permutation_sorted_by_cell(ops):
    rng = np.random.default_rng(23)
    box = (30., 30., 30.)
    x = (rng.random((3, 2000, 3)) * 30).astype(np.float32)
    search = ops.NeighbourSearch(torch.from_numpy(x).cuda(), 5.0, box)
    order = search.cell_order().cpu().numpy()
    assert np.array_equal(np.sort(order), np.arange(6000))
    _, cell = ON.wrap_cells(x, 5.0, box)
    flat_cell = cell.reshape(-1) + (np.arange(6000) // 2000) * 216          # 6^3 cells per box
    keys = flat_cell[order]
    assert np.all(np.diff(keys) >= 0)
    same = np.diff(keys) == 0
    assert np.all(np.diff(order)[same] > 0)                                   # atom id ascending inside a cell


@pytest.mark.parametrize("nodes,box_len,cutoff", [(3000, 40.0, 5.0), (70000, 80.0, 4.0)])
def test_workspace_smaller_than_the_preferred_size(nodes, box_len, cutoff):
    """The count / fill / cell-order calls take any workspace down to neighbour rows of 32 entries: the edge list is
    the same bit for bit, whether the rows are 256 entries long or so short that most atoms overflow theirs and are
    swept again by the fill pass; one byte less than the minimum is refused.  Boxes of at most 65536 atoms keep
    16-bit neighbour ids between the passes, larger ones 32-bit ids."""
    import ctypes
    L = importlib.import_module("learned-dynamics_amd._lib")
    lib = L.load()
    rng = np.random.default_rng(nodes)
    B = 2 if nodes < 65536 else 1
    x = torch.from_numpy((rng.random((B, nodes, 3)) * box_len).astype(np.float32)).cuda()
    box = (box_len,) * 3
    ndiv = int(np.ceil(box_len / cutoff))
    A, C = B * nodes, B * ndiv ** 3
    entry = 2 if nodes <= 65536 else 4
    pref = ctypes.c_size_t(0)
    L.check(lib.mg_neighbour_workspace_bytes(B, nodes, cutoff, *box, ctypes.byref(pref)))
    assert A * 256 * entry < pref.value < A * (256 * entry + 60) + 8 * C + 8192
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def search(ws_bytes):
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        row_ptr = torch.empty(A + 1, dtype=torch.int32, device="cuda")
        ec = torch.empty(B, dtype=torch.int32, device="cuda")
        stats = torch.empty(4, dtype=torch.int32, device="cuda")
        status = lib.mg_neighbour_count(p(x), B, nodes, cutoff, *box, p(ws), ws_bytes, p(row_ptr), p(ec), p(stats), st)
        if status != 0:
            return status, None
        E = int(stats[0])
        src = torch.empty(E, dtype=torch.int32, device="cuda")
        dst = torch.empty(E, dtype=torch.int32, device="cuda")
        L.check(lib.mg_neighbour_fill(p(ws), ws_bytes, B, nodes, cutoff, *box, p(row_ptr), E, p(src), p(dst), st))
        order = torch.empty(A, dtype=torch.int32, device="cuda")
        L.check(lib.mg_neighbour_cell_order(p(ws), ws_bytes, B, nodes, cutoff, *box, p(order), st))
        return 0, (row_ptr, ec, stats, src, dst, order)

    status, want = search(pref.value)
    assert status == 0
    assert int(want[2][2]) > 40                                   # degrees above the shortest rows
    fixed = pref.value - A * 256 * entry
    for ws_bytes in (fixed + A * 100 * entry, fixed + A * 32 * entry + 4096):
        status, got = search(ws_bytes)
        assert status == 0, ws_bytes
        for a, b in zip(got, want):
            assert torch.equal(a, b)
    status, _ = search(fixed + A * 31 * entry)
    assert status == L.MG_ERR_WORKSPACE and b"at least" in lib.mg_last_error()

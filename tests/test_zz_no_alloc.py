"""mg_neighbour_edges_static (the radius graph with the library's built-in workspace: nothing is allocated by the
call) against mg_neighbour_edges with a caller-allocated workspace, through the C ABI, bit for bit, on two calls in
a row of which the second has the smaller input, so that what the first call left in the shared buffer is seen not
to matter."""
import ctypes
import importlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _buffers(B, N, capacity):
    i32 = dict(dtype=torch.int32, device="cuda")
    return dict(row_ptr=torch.full((B * N + 1,), -1, **i32), edge_counts=torch.full((B,), -1, **i32),
                stats=torch.full((4,), -1, **i32), src=torch.full((capacity,), -1, **i32),
                dst=torch.full((capacity,), -1, **i32))


def _call(lib, L, static, x, cutoff, box, capacity, out=None):
    B, N = x.shape[:2]
    out = _buffers(B, N, capacity) if out is None else out
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tail = (_ptr(out["row_ptr"]), _ptr(out["edge_counts"]), _ptr(out["stats"]), capacity, _ptr(out["src"]),
            _ptr(out["dst"]), stream)
    if static:
        L.check(lib.mg_neighbour_edges_static(_ptr(x), B, N, cutoff, *box, *tail))
    else:
        nbytes = ctypes.c_size_t(0)
        L.check(lib.mg_neighbour_workspace_bytes(B, N, cutoff, *box, ctypes.byref(nbytes)))
        ws = torch.empty(nbytes.value, dtype=torch.uint8, device="cuda")
        L.check(lib.mg_neighbour_edges(_ptr(x), B, N, cutoff, *box, _ptr(ws), nbytes.value, *tail))
    torch.cuda.synchronize()
    return out


def test_built_in_workspace_gives_the_same_graph_twice_in_a_row():
    L = importlib.import_module("learned-dynamics_amd._lib")
    lib = L.load()
    rng = np.random.default_rng(0x947)
    cases = [((4, 9000, 3), 5.0, (40., 40., 40.), 3_000_000),        # dense cells, ~120 neighbours per atom
             ((2, 700, 3), 6.0, (70., 70., 70.), 40_000),            # smaller, sparse cells (one-wave workgroups)
             ((1, 3000, 3), 4.0, (12., 12., 12.), 100_000),           # windows larger than the LDS tile; capacity < E
             # more atoms in one box than the per-box sort in LDS takes: the histogram / scan / place path, on a
             # workspace that the calls before left dirty
             ((1, 20000, 3), 5.0, (60., 60., 60.), 1_500_000),
             # 8 boxes x 16384 atoms at 0.098 atoms / A^3: the built-in workspace takes it with neighbour rows of 224
             # entries where the caller's workspace of the preferred size has 256; the graph is the same
             ((8, 16384, 3), 5.0, (55., 55., 55.), 7_200_000)]
    for shape, cutoff, box, capacity in cases:
        x = torch.from_numpy((rng.random(shape) * 3 - 1).astype(np.float32) * box[0]).cuda()
        print("case", shape, cutoff, box, capacity, flush=True)
        want = _call(lib, L, False, x, cutoff, box, capacity)
        # outputs allocated before the window; the driver's own count of free device memory (hipMemGetInfo) must
        # not move across the call: it sees any allocation, through torch or not
        got = _buffers(shape[0], shape[1], capacity)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        torch_before = torch.cuda.memory_allocated()
        _call(lib, L, True, x, cutoff, box, capacity, out=got)
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_allocated() == torch_before
        E = int(want["stats"][0])
        assert E > 0 and int(got["stats"][0]) == E
        for key in ("row_ptr", "edge_counts", "stats", "src", "dst"):
            assert torch.equal(got[key], want[key]), key
        if capacity < E:
            assert shape == (1, 3000, 3) and bool((got["src"] >= 0).all())
            assert int(got["row_ptr"].max()) == capacity and int(got["stats"][3]) & 2
        else:
            assert bool((got["src"][E:] == -1).all()) and bool((got["dst"][E:] == -1).all())


def test_search_larger_than_the_built_in_workspace_is_refused():
    L = importlib.import_module("learned-dynamics_amd._lib")
    lib = L.load()
    B, N = 16, 65536                                                  # 1048576 atoms: 122 MB even with the shortest rows
    x = torch.rand(B, N, 3, device="cuda") * 100
    out = _buffers(B, N, 16)
    status = lib.mg_neighbour_edges_static(_ptr(x), B, N, 5.0, 100., 100., 100., _ptr(out["row_ptr"]),
                                           _ptr(out["edge_counts"]), _ptr(out["stats"]), 16, _ptr(out["src"]),
                                           _ptr(out["dst"]), ctypes.c_void_p(0))
    assert status == L.MG_ERR_WORKSPACE
    assert b"built-in" in lib.mg_last_error()
    torch.cuda.synchronize()
    assert bool((out["row_ptr"] == -1).all())                         # nothing ran

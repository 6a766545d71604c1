"""The hot path at the FULL sizes of the BASELINE configurations, checked through properties that do
not need an oracle of that size: invariants of the neighbour graph (the ones
extensions/neighbour_grid/test.py:22-46 checks on 20 x 60 points), exact agreement with a brute-force
minimum-image search for a sample of atoms, SO(3) equivariance of the layers under a rotation that is
exact in fp32 (a quarter turn maps the cubic periodic box onto itself and only permutes / negates
coordinates), and the stated tolerance between the bf16-storage and the fp32-storage stacks."""
import importlib

import numpy as np
import pytest
import torch

from oracle import layers as OL
from oracle import neighbour as ON
from parity import assert_parity

pytestmark = pytest.mark.gpu

SEED = 0x947


def _quarter_turn(t_vec):
    """(x, y, z) -> (-y, x, z) on a trailing axis of size 3: exact in floating point."""
    return torch.stack([-t_vec[..., 1], t_vec[..., 0], t_vec[..., 2]], dim=-1)


def _quarter_turn_rank2(d):
    """R d R^T for the same rotation, on trailing axes (3, 3)."""
    return _quarter_turn(_quarter_turn(d).transpose(-1, -2)).transpose(-1, -2)


def _polymer(chains, beads, box, seed):
    g = torch.Generator().manual_seed(seed)
    steps = torch.randn(chains, beads, 3, generator=g)
    steps = 3.8 * steps / steps.norm(dim=-1, keepdim=True)
    origin = torch.rand(chains, 1, 3, generator=g) * box
    return (steps.cumsum(1) + origin).reshape(1, chains * beads, 3).contiguous()


def test_configs1_neighbour_search_invariants(ops):
    """8 boxes x 16384 atoms, box 55, cutoff 5 (ndiv = 11 exactly: the result is the plain minimum-image graph)."""
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    B, N, L, r0 = 8, 16384, 55.0, 5.0
    pos = (torch.rand(B, N, 3, generator=torch.Generator().manual_seed(SEED + 2)) * L).cuda()
    src, dst, counts = ops.get_edges(32, 128, r0, L, L, L, pos)
    E = int(src.numel())
    src, dst = src.long(), dst.long()
    assert 6_000_000 < E < 7_500_000
    assert bool((src[1:] >= src[:-1]).all()), "src must be sorted"
    assert bool((src != dst).all()), "no self edges"
    assert bool((src // N == dst // N).all()), "edges stay inside their box"
    assert int(counts[-1]) == E and bool((counts[1:] >= counts[:-1]).all())
    per_box = torch.bincount(src // N, minlength=B)
    assert torch.equal(per_box.cumsum(0).int(), counts)
    # symmetric adjacency: the multiset of (i, j) equals the multiset of (j, i)
    fwd = torch.sort(src * (B * N) + dst).values
    bwd = torch.sort(dst * (B * N) + src).values
    assert torch.equal(fwd, bwd)
    assert bool((fwd[1:] != fwd[:-1]).all()), "no duplicate edges"
    # reduce-of-ones = degrees, gather identity (extensions/neighbour_grid/test.py:36-46)
    graph = gl.Graph(src, dst, counts, B, N)
    deg = gl.edges_reduce_src(graph, torch.ones(E, 1, device="cuda")).reshape(-1)
    assert torch.equal(deg.long(), torch.bincount(src, minlength=B * N))
    x_src, _ = gl.edges_read(graph, pos)
    assert torch.equal(x_src, pos.reshape(-1, 3)[src])
    # every edge is within the cutoff, and for a sample of atoms the neighbour SET equals brute force
    r_ij = gl.edge_vectors(graph, pos, (L, L, L))
    assert float(r_ij.norm(dim=1).max()) <= r0 * (1 + 1e-6)
    g = torch.Generator().manual_seed(1)
    for b in range(0, B, 3):
        sample = torch.randint(0, N, (48,), generator=g).cuda()
        d = pos[b, sample][:, None, :] - pos[b][None, :, :]
        d = d - L * torch.round(d / L)
        d2 = (d.double() ** 2).sum(-1)
        near = d2 <= r0 * r0 * (1 + 1e-6)
        clear = (d2 <= r0 * r0 * (1 - 1e-6)) | ~near          # pairs not within rounding of the cutoff
        got = torch.zeros(48, N, dtype=torch.bool, device="cuda")
        for k, i in enumerate(sample.tolist()):
            row = b * N + i
            lo, hi = int(graph.row_ptr[row]), int(graph.row_ptr[row + 1])
            got[k, dst[lo:hi] - b * N] = True
            near[k, i] = False                                # self
        assert bool(((got == near) | ~clear).all())


def test_configs2_painn_layer_is_equivariant_at_full_size(pkg):
    """16 chains x 1024 beads, box 80, cutoff 8, n = 128, 16 radial functions."""
    painn = importlib.import_module("learned-dynamics_amd.painn")
    n, r0, L = 128, 8.0, 80.0
    box = (L, L, L)
    torch.manual_seed(SEED + 3)
    block = painn.Block(r0, n, n_rbf=16).cuda().eval()
    pos = _polymer(16, 1024, L, SEED + 3).cuda()
    g = torch.Generator().manual_seed(SEED + 4)
    x_a = torch.randn(1, 16384, n, generator=g).cuda()
    x_v = (torch.randn(1, 16384, n, 3, generator=g) / 3 ** 0.5).cuda()
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")

    def run(p, xv):
        graph, r_ij = gl.graph_setup(r0, box, p.contiguous(), neighbours_max=512, celllist_max=128)
        return block((p, graph, r_ij, None, None, x_a, xv, box))

    with torch.no_grad():
        out = run(pos, x_v)
        out_r = run(_quarter_turn(pos), _quarter_turn(x_v))
    a, v, a_r, v_r = out[5], out[6], out_r[5], out_r[6]
    assert torch.isfinite(a).all() and torch.isfinite(v).all()
    torch.testing.assert_close(a_r, a, rtol=1e-5, atol=2e-5 * float(a.abs().max()))
    torch.testing.assert_close(v_r, _quarter_turn(v), rtol=1e-5, atol=2e-5 * float(v.abs().max()))
    # and invariant under a translation by a multiple of the cell size in a periodic box
    with torch.no_grad():
        out_t = run(pos + torch.tensor([8.0, -16.0, 24.0], device="cuda"), x_v)
    torch.testing.assert_close(out_t[5], a, rtol=1e-5, atol=2e-5 * float(a.abs().max()))


def test_configs2_message_filter_grid_against_per_edge_mlp_and_oracle_at_full_size(pkg):
    """The PaiNN Message of configs[2] (16 chains x 1024 beads, box 80, cutoff 8, n = 128, 16 radial functions) at
    full size: the path that interpolates the filter from its grid against the path that evaluates the filter MLP
    on every edge (both HIP), and 64 sampled nodes of both against the oracle's Message
    (archs/meanflow_painn8.py:85-100) evaluated in float32 and float64 on exactly those nodes' edges."""
    painn = importlib.import_module("learned-dynamics_amd.painn")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    n, r0, L, N = 128, 8.0, 80.0, 16384
    box = (L, L, L)
    torch.manual_seed(SEED + 3)
    msg = painn.Message(r0, n, 16).cuda().eval()
    pos = _polymer(16, 1024, L, SEED + 3)
    g = torch.Generator().manual_seed(SEED + 4)
    x_a = torch.randn(1, N, n, generator=g)
    x_v = torch.randn(1, N, n, 3, generator=g) / 3 ** 0.5
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, box, pos.cuda(), neighbours_max=512, celllist_max=128)
        assert msg.table_rows() == 512
        ta, tv = msg(graph, x_a.cuda(), x_v.cuda(), r_ij)              # filter from the grid held in LDS
        msg.use_table = False
        ea, ev = msg(graph, x_a.cuda(), x_v.cuda(), r_ij)              # filter MLP on every edge
    E = int(graph.src.numel())
    assert 1_300_000 < E < 1_800_000
    # oracle on the rows of 64 sampled nodes
    sample = torch.randint(0, N, (64,), generator=g).sort().values.unique()
    row_ptr = graph.row_ptr.cpu().long()
    pick = torch.cat([torch.arange(int(row_ptr[i]), int(row_ptr[i + 1])) for i in sample.tolist()])
    src, dst = graph.src.cpu()[pick], graph.dst.cpu()[pick]
    r_ref = torch.from_numpy(ON.edge_vectors(pos.numpy(), src.numpy(), dst.numpy(), box))
    assert torch.equal(r_ij.cpu()[pick], r_ref)
    mlp_w = lambda m, dt: {k: getattr(m.layers[i], a).detach().cpu().to(dt) for k, i, a in
                           (("W1", 0, "weight"), ("b1", 0, "bias"), ("W2", 2, "weight"), ("b2", 2, "bias"),
                            ("W3", 4, "weight"), ("b3", 4, "bias"))}
    refs = {}
    for dt in (torch.float32, torch.float64):
        ra, rv = OL.painn_message(src, dst, 1, N, x_a.to(dt), x_v.to(dt), r_ref.to(dt), mlp_w(msg.mlp_dist, dt),
                                  mlp_w(msg.mlp_actv, dt), r0, n, 16)
        refs[dt] = (ra[0, sample], rv[0, sample])
    e_ref_a = e_ref_v = 0.0
    for name, (a, v) in (("filter grid", (ta, tv)), ("filter MLP per edge", (ea, ev))):
        e_ref_a = assert_parity(a[0, sample.cuda()], refs[torch.float32][0], refs[torch.float64][0],
                                f"configs[2] Message, {name}, dx_a")[0]
        e_ref_v = assert_parity(v[0, sample.cuda()], refs[torch.float32][1], refs[torch.float64][1],
                                f"configs[2] Message, {name}, dx_v")[0]
    # the two HIP paths against each other on every node: each is within 1e-6 + 1e-5 |exact| + 2 e_ref of exact
    # arithmetic (e_ref as measured on the sampled nodes), so they differ by at most twice that; nothing is added
    # for the grid
    torch.testing.assert_close(ta, ea, rtol=2e-5, atol=2 * (1e-6 + 2 * e_ref_a))
    torch.testing.assert_close(tv, ev, rtol=2e-5, atol=2 * (1e-6 + 2 * e_ref_v))


def test_configs3_one_system_of_the_full_batch_against_the_oracle(pkg):
    """configs[3] at full size (32 systems x 2048 atoms, 8 blocks, 256 / 64 / 16 channels, chan 256): the forward of
    the whole batch on the GPU, and the first system of it against the oracle's composition in float32 and float64
    (systems are independent graphs and the group norms take their statistics per system)."""
    den = importlib.import_module("learned-dynamics_amd.denoiser")
    from test_gpu_bee_layers import denoiser_oracle
    B, N, L, r0 = 32, 2048, 70.0, 6.0
    box = (L, L, L)
    torch.manual_seed(SEED + 4)
    model = den.Denoiser(r0, dim_a=256, dim_v=64, dim_d=16, chan=256, blocks=8).cuda().eval()
    g = torch.Generator().manual_seed(SEED + 4)
    steps = torch.randn(B, N, 3, generator=g)
    steps = 3.8 * steps / steps.norm(dim=-1, keepdim=True)
    x1 = steps.cumsum(1) + torch.rand(B, 1, 3, generator=g) * L + torch.randn(B, N, 3, generator=g)
    x0 = x1 + torch.randn(B, N, 3, generator=g)
    one_hot = torch.nn.functional.one_hot(torch.randint(0, 20, (B, N), generator=g), 20).float()
    s, t = torch.zeros(B), torch.rand(B, generator=g)
    with torch.no_grad():
        v = model((s.cuda(), t.cuda()), x0.cuda(), x1.cuda(), one_hot.cuda(), box)
    first = lambda x: x[:1].contiguous()
    args = (first(s), first(t), first(x0), first(x1), first(one_hot), box, r0)
    v32 = denoiser_oracle(model, *args, torch.float32)
    v64 = denoiser_oracle(model, *args, torch.float64)
    assert_parity(v[:1], v32, v64, "configs[3] denoiser, system 0 of 32")


def test_configs3_denoiser_is_equivariant_at_full_size(pkg):
    """32 systems x 2048 atoms, box 70, cutoff 6, 8 blocks, 256 / 64 / 16 channels, chan 256."""
    den = importlib.import_module("learned-dynamics_amd.denoiser")
    B, N, L, r0 = 32, 2048, 70.0, 6.0
    box = (L, L, L)
    torch.manual_seed(SEED + 4)
    model = den.Denoiser(r0, dim_a=256, dim_v=64, dim_d=16, chan=256, blocks=8).cuda().eval()
    g = torch.Generator().manual_seed(SEED + 4)
    steps = torch.randn(B, N, 3, generator=g)
    steps = 3.8 * steps / steps.norm(dim=-1, keepdim=True)
    x1 = (steps.cumsum(1) + torch.rand(B, 1, 3, generator=g) * L + torch.randn(B, N, 3, generator=g)).cuda()
    x0 = x1 + torch.randn(B, N, 3, generator=g).cuda()
    one_hot = torch.nn.functional.one_hot(torch.randint(0, 20, (B, N), generator=g), 20).float().cuda()
    s, t = torch.zeros(B).cuda(), torch.rand(B, generator=g).cuda()
    with torch.no_grad():
        v = model((s, t), x0, x1, one_hot, box)
        v_r = model((s, t), _quarter_turn(x0), _quarter_turn(x1), one_hot, box)
    assert v.shape == (B, N, 3) and torch.isfinite(v).all()
    # 8 blocks deep: fp32 rounding compounds through the group norms (rel 1e-4 of the output scale)
    torch.testing.assert_close(v_r, _quarter_turn(v), rtol=1e-4, atol=1e-4 * float(v.abs().max()))


def _configs4(seed_offset=5):
    N, r0, C = 65536, 6.0, 128
    L = (N / 0.1) ** (1.0 / 3.0)
    g = torch.Generator().manual_seed(SEED + seed_offset)
    pos = torch.rand(1, N, 3, generator=g) * L
    x_a = torch.randn(1, N, C, generator=g)
    x_v = torch.randn(1, N, C, 3, generator=g) / 3 ** 0.5
    x_d = torch.randn(1, N, C, 3, 3, generator=g) / 3.0
    return N, r0, C, L, pos, x_a, x_v, x_d


def test_configs4_bf16_storage_within_one_percent_at_full_size(pkg):
    """65536 atoms at 0.1 / A^3, cutoff 6, 128 channels per rank, all four layers of the stack: bf16 storage against
    fp32 storage after every layer (each layer ends in group norms, so the deviation does not grow with depth), and
    the rank-2 equivariance of the fp32 layer at this size."""
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    b16 = importlib.import_module("learned-dynamics_amd.bee_layers_bf16")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    N, r0, C, L, pos, x_a, x_v, x_d = _configs4()
    pos, x_a, x_v, x_d = pos.cuda(), x_a.cuda(), x_v.cuda(), x_d.cuda()
    torch.manual_seed(SEED + 5)
    msgs = [bee.Messages(r0, C, C, C, C).cuda().eval() for _ in range(4)]
    prods = [bee.SelfTensProds(C, C, C, C).cuda().eval() for _ in range(4)]
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, (L, L, L), pos, neighbours_max=256, celllist_max=64)
        assert 5_500_000 < int(graph.src.numel()) < 6_400_000
        ref = (x_a, x_v, x_d)
        for depth, (msg, prod) in enumerate(zip(msgs, prods), 1):
            da, dv, dd = msg(graph, r_ij, *ref)
            mid = (ref[0] + da, ref[1] + dv, ref[2] + dd)
            ref = prod(*mid, residual=True)
            out = b16.stack_forward(msgs[:depth], prods[:depth], graph, r_ij, x_a, x_v, x_d)
            dev = [float((o - r).abs().max() / r.abs().max()) for o, r in zip(out, ref)]
            print(f"[configs4] bf16 against fp32 storage after {depth} layers: {dev}")
            assert max(dev) < 1e-2
            if depth == 1:
                # rank-2 equivariance of the fp32 layer at this size
                ref_r = prod(*[f(t) for f, t in zip((lambda t: t, _quarter_turn, _quarter_turn_rank2), mid)], residual=True)
                torch.testing.assert_close(ref_r[2], _quarter_turn_rank2(ref[2]), rtol=1e-5,
                                           atol=1e-5 * float(ref[2].abs().max()))
            del da, dv, dd, mid, out


def test_configs4_messages_on_sampled_atoms_against_the_oracle(pkg):
    """The rank-0/1/2 Messages layer of configs[4] at full size (65536 atoms, about 90 neighbours each, 128 channels per
    rank): 48 sampled atoms of the fp32-storage path against the oracle's Messages (archs/diffuser_atoms15.py:238-253)
    evaluated in float32 and float64 on exactly those atoms' edges at the layer tolerance, and the same atoms of the
    bf16-storage path against the float64 oracle within 1e-2 of the output scale."""
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    b16 = importlib.import_module("learned-dynamics_amd.bee_layers_bf16")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    from oracle import products as OP
    from test_gpu_bee_layers import _mlp_leaky_weights
    N, r0, C, L, pos, x_a, x_v, x_d = _configs4(seed_offset=6)
    box = (L, L, L)
    torch.manual_seed(SEED + 6)
    msg = bee.Messages(r0, C, C, C, C).cuda().eval()
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, box, pos.cuda(), neighbours_max=256, celllist_max=64)
        got = msg(graph, r_ij, x_a.cuda(), x_v.cuda(), x_d.cuda())
        s = b16.to_storage(x_a.cuda(), x_v.cuda(), x_d.cuda())
        got16 = b16.from_storage(*b16.messages_forward(msg, graph, r_ij, *s), 1)
    g = torch.Generator().manual_seed(SEED + 7)
    sample = torch.randint(0, N, (48,), generator=g).sort().values.unique()
    row_ptr = graph.row_ptr.cpu().long()
    pick = torch.cat([torch.arange(int(row_ptr[i]), int(row_ptr[i + 1])) for i in sample.tolist()])
    assert pick.numel() > 3000
    src, dst = graph.src.cpu()[pick], graph.dst.cpu()[pick]
    r_ref = torch.from_numpy(ON.edge_vectors(pos.numpy(), src.numpy(), dst.numpy(), box))
    assert torch.equal(r_ij.cpu()[pick], r_ref)
    dd = lambda t, dt: t.detach().cpu().to(dt)
    refs = {}
    for dt in (torch.float32, torch.float64):
        w = {"L0": dd(msg.L0.W, dt), "L1": dd(msg.L1.W, dt), "L2": dd(msg.L2.W, dt),
             "Y": {lab: dd(getattr(msg, f"Y_{lab}").W, dt) for lab in OP.BEE_ORDER},
             "enc_W": dd(msg.lin_enc.weight, dt), "enc_b": dd(msg.lin_enc.bias, dt),
             "mlp_a": {k: v.to(dt) for k, v in _mlp_leaky_weights(msg.mlp_a).items()}}
        out = OL.bee_messages(src, dst, 1, N, r_ref.to(dt), x_a.to(dt), x_v.to(dt), x_d.to(dt), w, r0,
                              radial_dtype=torch.float64)
        refs[dt] = [t[0, sample] for t in out]
        del out, w
    for k, name in enumerate("avd"):
        assert_parity(got[k][0, sample.cuda()], refs[torch.float32][k], refs[torch.float64][k],
                      f"configs[4] Messages, fp32 storage, B_{name}")
        r64 = refs[torch.float64][k]
        dev = float((got16[k][0, sample.cuda()].cpu().double() - r64).abs().max() / r64.abs().max())
        print(f"[configs4] Messages, bf16 storage against the float64 oracle, B_{name}: {dev:.3g} of the output scale")
        assert dev < 1e-2


def test_configs2_training_step_through_the_filter_grid(pkg):
    """One PaiNN block at configs[2] (16384 atoms, n = 128, 16 radial functions, ~1.6 M edges), forward + backward
    through the differentiable path: the filter through its grid (MLP differentiated on 512 rows, edges interpolate)
    against the filter MLP on every edge, both on the HIP kernels.  The loss and every gradient (23 parameters, x_a,
    x_v) agree to 1e-5 of the gradient's largest entry; the gradients of a second run are the same bits."""
    painn = importlib.import_module("learned-dynamics_amd.painn")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    n, n_rbf, r0, box_len = 128, 16, 8.0, 80.0
    box = (box_len,) * 3
    torch.manual_seed(SEED + 3)
    pos = _polymer(16, 1024, box_len, SEED + 3).cuda()
    block = painn.Block(r0, n, n_rbf=n_rbf).cuda().train()
    g = torch.Generator().manual_seed(SEED + 4)
    x_a = torch.randn(1, 16384, n, generator=g).cuda().requires_grad_(True)
    x_v = (torch.randn(1, 16384, n, 3, generator=g) / 3 ** 0.5).cuda().requires_grad_(True)
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, box, pos, neighbours_max=512, celllist_max=128)
    assert graph.src.numel() > 1_000_000
    params = [p for p in block.parameters() if p.requires_grad]
    names = ["x_a", "x_v"] + [k for k, _ in block.named_parameters()]

    def step():
        out = block((pos, graph, r_ij, None, None, x_a, x_v, box))
        loss = out[5].square().mean() + out[6].square().mean()
        return loss, torch.autograd.grad(loss, [x_a, x_v] + params, allow_unused=True)

    assert block.message.table_rows() == 512
    loss_grid, g_grid = step()
    _, g_again = step()
    block.message.use_table = False
    loss_edge, g_edge = step()
    assert abs(float(loss_grid) - float(loss_edge)) <= 1e-6 * abs(float(loss_edge))
    checked = 0
    for name, a, b, c in zip(names, g_grid, g_again, g_edge):
        if c is None:
            assert a is None
            continue
        scale = float(c.abs().max())
        err = float((a - c).abs().max())
        assert err <= 1e-5 * scale, (name, err, scale)
        assert torch.equal(a, b), name
        checked += 1
    assert checked >= 20

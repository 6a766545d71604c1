"""Rank-0/1/2 message kernel and the Messages / SelfTensProds modules against
the oracle's restatement of archs/diffuser_atoms15.py (float64 oracle for the
ill-conditioned radial encoding, see oracle test for its conditioning)."""
import importlib

import numpy as np
import pytest
import torch

from oracle import layers as OL
from oracle import neighbour as ON
from oracle import products as OP
from parity import assert_parity, assert_parity_of

pytestmark = pytest.mark.gpu


def _to(tree, dtype):
    if isinstance(tree, dict):
        return {k: _to(v, dtype) for k, v in tree.items()}
    return tree.to(dtype)


def test_edge_geometry(ops):
    g = torch.Generator().manual_seed(1)
    r = torch.randn(4000, 3, generator=g) * 3
    enc, rhat = ops.bee_edge_geometry(r.cuda(), 6.0)
    # radial_encode_8: the kernel evaluates the polynomial in float64 and rounds once (the reference's float32
    # monomial form is ill-conditioned, tests/test_oracle_layers.py), so the bar is the float64 oracle with no e_ref.
    # z = |r| / rmax itself is formed in float32, as in the reference: half an ulp of z (at most 3e-8) passes through
    # the polynomial's slope (up to about 30 where z is large enough to have such an ulp), which is the second 1e-6
    ref = OL.radial_encode_8(r.double(), 6.0)
    torch.testing.assert_close(enc.cpu().double(), ref, rtol=1e-5, atol=2e-6)
    assert_parity_of(rhat, lambda dt: OL.tens_sigmoid(1, r.to(dt) * (7.0 / 6.0)), "edge direction")


@pytest.mark.parametrize("lin_layout", [(0, 64, 40), (1, 64, 40), (2, 32, 72), (1, 20, 7), (2, 8, 130)])
def test_linear_layouts(ops, lin_layout):
    inds, dim_in, dim_out = lin_layout
    T = 3 ** inds
    g = torch.Generator().manual_seed(2)
    W = torch.randn(dim_out, dim_in, generator=g)
    x = torch.randn(50, dim_in, *([3] * inds), generator=g)
    def ref(dt):                                                         # (50, O, 3..)
        return OP.tensor_linear(inds, W.to(dt), x.to(dt))

    ref_cm = lambda dt: ref(dt).reshape(50, dim_out, T).transpose(1, 2).contiguous()     # (50, T, O)
    x_cm = x.reshape(50, dim_in, T).transpose(1, 2).contiguous()         # (50, T, I)
    C = ops.LAYOUT_COMP_CHAN
    y = ops.tensor_linear_fwd(inds, W.cuda(), x.cuda(), y_layout=C)
    assert_parity_of(y, ref_cm, f"tensor_linear rank {inds}, component-major output")
    y = ops.tensor_linear_fwd(inds, W.cuda(), x_cm.cuda(), x_layout=C)
    assert_parity_of(y, ref, f"tensor_linear rank {inds}, component-major input")
    y = ops.tensor_linear_fwd(inds, W.cuda(), x_cm.cuda(), x_layout=C, y_layout=C)
    assert_parity_of(y, ref_cm, f"tensor_linear rank {inds}, component-major both")


@pytest.mark.parametrize("chan,E", [(64, 3000), (8, 3000), (100, 3000), (64, 9000), (40, 7000)])
def test_bee_message_kernel(ops, chan, E):
    """E / N below and above 32: the kernel pipelines its gathers only on long rows."""
    torch.manual_seed(chan)
    N = 200
    src = torch.sort(torch.randint(0, N, (E,))).values
    src[src == 5] = 6
    dst = torch.randint(0, N, (E,))
    r = torch.randn(E, 3) * 2.5
    La, Lv, Ld = torch.randn(N, chan), torch.randn(N, chan, 3), torch.randn(N, chan, 3, 3)
    encW, encb = torch.randn(chan, 8) * 0.3, torch.randn(chan)
    enc, rhat = ops.bee_edge_geometry(r.cuda(), 6.0)
    row_ptr = ops.segment_row_ptr(src.int().cuda(), N)
    Lv_cm = Lv.transpose(1, 2).contiguous()
    Ld_cm = Ld.reshape(N, chan, 9).transpose(1, 2).contiguous()
    order = torch.randperm(N).int().cuda()
    for node_order in (None, order):
        P0, S1, S2, nmax, emax = ops.bee_message(row_ptr, dst.int().cuda(), rhat, enc, La.cuda(), Lv_cm.cuda(), Ld_cm.cuda(),
                                           encW.cuda(), encb.cuda(), node_order=node_order, want_node_max=True)
        # the emitted per-node maxima are exactly the maxima of what was written
        assert nmax.shape == (N, (chan + 63) // 64)
        assert torch.equal(nmax.amax(1), torch.maximum(S1.abs().amax(dim=(1, 2, 3)), S2.abs().amax(dim=(1, 2, 3))))
        assert emax.shape == (E, (chan + 63) // 64) and torch.equal(emax.amax(1), P0.abs().amax(dim=(1, 2)))
        # oracle on the device's own enc / rhat (they are checked separately)
        def products(dt):
            phi_a = torch.nn.functional.linear(enc.cpu().to(dt), encW.to(dt), encb.to(dt))
            rh = rhat.cpu().to(dt)
            phi_v = phi_a[..., None] * rh[:, None, :]
            phi_d = phi_a[..., None, None] * rh[:, None, None, :] * rh[:, None, :, None]
            return dict(zip(OP.BEE_ORDER, OP.bee(La.to(dt)[dst], Lv.to(dt)[dst], Ld.to(dt)[dst], phi_a, phi_v, phi_d)))

        for k, lab in enumerate(("000", "110", "220")):
            assert_parity_of(P0[:, k], lambda dt: products(dt)[lab], f"bee_message P0 {lab} chan={chan}")
        for k, lab in enumerate(("011", "101", "121", "211", "111")):
            assert_parity_of(S1[:, :, k], lambda dt: torch.zeros(N, chan, 3, dtype=dt).index_add_(
                0, src, products(dt)[lab]).transpose(1, 2), f"bee_message S1 {lab} chan={chan}")
        for k, lab in enumerate(("022", "202", "112", "222", "212")):
            assert_parity_of(S2[:, :, k], lambda dt: torch.zeros(N, chan, 3, 3, dtype=dt).index_add_(
                0, src, products(dt)[lab]).reshape(N, chan, 9).transpose(1, 2), f"bee_message S2 {lab} chan={chan}")


@pytest.mark.parametrize("chan,dim_d,N,E", [(256, 16, 203, 3000), (128, 7, 101, 2500), (64, 16, 37, 900), (256, 1, 50, 30)])
def test_bee_message_with_the_rank2_linear_inside(ops, chan, dim_d, N, E):
    """mg_bee_message_rank2: Y2 S2 from the edge kernel against Y2 applied to the S2 of mg_bee_message by the oracle's
    matmul; everything else the two entry points write is bit-equal.  Node counts that leave the last workgroup partly
    filled (chan 128: two nodes per workgroup, odd node count), nodes without edges, and an uneven row stride of Y2."""
    torch.manual_seed(chan + dim_d)
    src = torch.sort(torch.randint(0, N, (E,))).values
    src[src == 5] = 6
    dst = torch.randint(0, N, (E,))
    r = torch.randn(E, 3) * 2.5
    La, Lv, Ld = torch.randn(N, chan).cuda(), torch.randn(N, 3, chan).cuda(), torch.randn(N, 9, chan).cuda()
    encW, encb = (torch.randn(chan, 8) * 0.3).cuda(), torch.randn(chan).cuda()
    wide = (torch.randn(dim_d, 5 * chan + 4) / (5 * chan) ** 0.5).cuda()
    Y2 = wide[:, :5 * chan]
    enc, rhat = ops.bee_edge_geometry(r.cuda(), 6.0)
    row_ptr = ops.segment_row_ptr(src.int().cuda(), N)
    assert ops.bee_rank2_supported(chan, dim_d) and not ops.bee_rank2_supported(chan, 17) and not ops.bee_rank2_supported(100, 8)
    for node_order in (None, torch.randperm(N).int().cuda()):
        args = (row_ptr, dst.int().cuda(), rhat, enc, La, Lv, Ld, encW, encb)
        P0, S1, S2, nmax, emax = ops.bee_message(*args, node_order=node_order, want_node_max=True)
        Q0, T1, out, nmax2, emax2 = ops.bee_message(*args, node_order=node_order, want_node_max=True, Y2=Y2)
        assert torch.equal(Q0, P0) and torch.equal(T1, S1) and torch.equal(nmax2, nmax) and torch.equal(emax2, emax)
        assert out.shape == (N, dim_d, 9)
        s2 = S2.cpu().reshape(N, 9, 5 * chan)
        assert_parity_of(out, lambda dt: (s2.to(dt) @ Y2.cpu().to(dt).t()).transpose(1, 2),
                         f"rank-2 linear inside the edge kernel, chan={chan}, dim_d={dim_d}")
    with pytest.raises(RuntimeError, match="dim_d <= 16"):
        ops.bee_message(*args, Y2=torch.zeros(17, 5 * chan, device="cuda"))
    with pytest.raises(RuntimeError, match="5 chan"):
        ops.bee_message(*args, Y2=torch.zeros(8, 4 * chan, device="cuda"))
    # the packed weight follows an in-place update of Y2's storage
    with torch.no_grad():
        wide.mul_(2.0)
    out2 = ops.bee_message(*args, Y2=Y2)[2]
    assert_parity_of(out2, lambda dt: (s2.to(dt) @ Y2.cpu().to(dt).t()).transpose(1, 2), "after the weight changed")


def test_node_products_emit_node_maxima(ops):
    g = torch.Generator().manual_seed(3)
    N, chan = 50, 128
    t = [torch.randn(N, *([c] if c > 1 else []), chan, generator=g).cuda() for c in (1, 3, 9, 1, 3, 9)]
    P0, P1, P2, nmax = ops.bee_node_products(*t, want_node_max=True)
    assert nmax.shape == (N, 2)
    want = torch.stack([P0.abs().amax(dim=(1, 2)), P1.abs().amax(dim=(1, 2, 3)), P2.abs().amax(dim=(1, 2, 3))]).amax(0)
    assert torch.equal(nmax.amax(1), want)
    # channel counts that a wave straddles: no maxima (the caller falls back to a pass over the rows)
    t = [torch.randn(N, *([c] if c > 1 else []), 40, generator=g).cuda() for c in (1, 3, 9, 1, 3, 9)]
    assert ops.bee_node_products(*t, want_node_max=True)[3] is None


def _mlp_leaky_weights(m):
    L = m.layers
    return {"W_direct": m.lin_direct.weight.detach().cpu().double(),
            "W1": L[0].weight.detach().cpu().double(), "b1": L[0].bias.detach().cpu().double(),
            "W2": L[2].weight.detach().cpu().double(), "b2": L[2].bias.detach().cpu().double(),
            "W3": L[4].weight.detach().cpu().double(), "b3": L[4].bias.detach().cpu().double()}


@pytest.mark.parametrize("dims", [(32, 16, 8, 32), (64, 32, 16, 64)])
def test_messages_module(pkg, dims):
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    dim_a, dim_v, dim_d, chan = dims
    torch.manual_seed(0x947 + 4)
    box, r0 = (30., 30., 30.), 6.0
    pos = torch.rand(2, 500, 3) * 30
    msg = bee.Messages(r0, dim_a, dim_v, dim_d, chan).cuda()
    x_a, x_v, x_d = torch.randn(2, 500, dim_a), torch.randn(2, 500, dim_v, 3), torch.randn(2, 500, dim_d, 3, 3)
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, box, pos.cuda(), neighbours_max=256, celllist_max=64)
        B_a, B_v, B_d = msg(graph, r_ij, x_a.cuda(), x_v.cuda(), x_d.cuda())
    src, dst = graph.src.cpu(), graph.dst.cpu()
    r_ref = torch.from_numpy(ON.edge_vectors(pos.numpy(), src.numpy(), dst.numpy(), box))
    assert torch.equal(r_ij.cpu(), r_ref)
    dd = lambda t: t.detach().cpu().double()
    w = {"L0": dd(msg.L0.W), "L1": dd(msg.L1.W), "L2": dd(msg.L2.W),
         "Y": {lab: dd(getattr(msg, f"Y_{lab}").W) for lab in OP.BEE_ORDER},
         "enc_W": dd(msg.lin_enc.weight), "enc_b": dd(msg.lin_enc.bias), "mlp_a": _mlp_leaky_weights(msg.mlp_a)}
    r64 = OL.bee_messages(src, dst, 2, 500, r_ref.double(), x_a.double(), x_v.double(), x_d.double(), w, r0)
    # the fp32 evaluation of the same math (radial polynomial rounded once from float64, as the kernel does: the
    # reference's fp32 monomial form is ill-conditioned, see tests/test_oracle_layers.py)
    r32 = OL.bee_messages(src, dst, 2, 500, r_ref, x_a, x_v, x_d, _to(w, torch.float32), r0, radial_dtype=torch.float64)
    for k, (got, name) in enumerate(zip((B_a, B_v, B_d), "avd")):
        assert_parity(got, r32[k], r64[k], f"Messages {dims} B_{name}")
    # the residual step formed in the inputs' memory: x + messages against the same oracle, the inputs overwritten,
    # and a non-contiguous input taking the out-of-place route
    own = [x_a.cuda(), x_v.cuda(), x_d.cuda()]
    with torch.no_grad():
        y = msg(graph, r_ij, *own, add_to_inputs=True)
    for k, (got, x, name) in enumerate(zip(y, (x_a, x_v, x_d), "avd")):
        assert got.data_ptr() == own[k].data_ptr() and got.shape == x.shape
        assert_parity(got, x + r32[k], x.double() + r64[k], f"Messages {dims} x_{name} + B_{name} in place")
    wide = torch.randn(2, 500, dim_a + 3).cuda()
    wide[..., :dim_a] = x_a.cuda()
    with torch.no_grad():
        y2 = msg(graph, r_ij, wide[..., :dim_a], x_v.cuda(), x_d.cuda(), add_to_inputs=True)
    assert torch.equal(wide[..., :dim_a], x_a.cuda())
    for k, (got, x, name) in enumerate(zip(y2, (x_a, x_v, x_d), "avd")):
        assert_parity(got, x + r32[k], x.double() + r64[k], f"Messages {dims} x_{name} + B_{name} out of place")


def test_self_tens_prods_module(pkg):
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    torch.manual_seed(7)
    dim_a, dim_v, dim_d, chan = 32, 16, 8, 24
    mod = bee.SelfTensProds(dim_a, dim_v, dim_d, chan).cuda()
    with torch.no_grad():
        for gn in (mod.gn_a, mod.gn_v, mod.gn_d):
            gn.gamma.copy_(torch.randn_like(gn.gamma))
    x_a, x_v, x_d = torch.randn(2, 90, dim_a), torch.randn(2, 90, dim_v, 3), torch.randn(2, 90, dim_d, 3, 3)
    with torch.no_grad():
        y_a, y_v, y_d = mod(x_a.cuda(), x_v.cuda(), x_d.cuda())
    dd = lambda t: t.detach().cpu()
    w = {k: dd(getattr(mod, k).W) for k in ("L0", "R0", "L1", "R1", "L2", "R2")}
    w["Y"] = {lab: dd(getattr(mod, f"Y_{lab}").W) for lab in OP.BEE_ORDER}
    w.update(gn_a=dd(mod.gn_a.gamma), gn_v=dd(mod.gn_v.gamma), gn_d=dd(mod.gn_d.gamma))
    r32 = OL.self_tens_prods(x_a, x_v, x_d, w)
    r64 = OL.self_tens_prods(x_a.double(), x_v.double(), x_d.double(), _to(w, torch.float64))
    for k, (got, name) in enumerate(zip((y_a, y_v, y_d), "avd")):
        assert_parity(got, r32[k], r64[k], f"SelfTensProds y_{name}")


def test_state_dict_names_match_reference():
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    names = set(bee.Messages(5.0, 8, 8, 8, 8).state_dict().keys())
    for expect in ("L0.W", "L1.W", "L2.W", "Y_000.W", "Y_212.W", "lin_enc.weight", "lin_enc.bias",
                   "mlp_a.lin_direct.weight", "mlp_a.layers.0.weight", "mlp_a.layers.4.bias"):
        assert expect in names, expect
    names = set(bee.SelfTensProds(8, 8, 8, 8).state_dict().keys())
    for expect in ("L0.W", "R0.W", "L2.W", "R2.W", "Y_111.W", "gn_a.gamma", "gn_v.gamma", "gn_d.gamma"):
        assert expect in names, expect


def denoiser_oracle(model, s, t, x0, x1, one_hot, box, r0, dtype):
    """The Denoiser assembly (embed + time embed + read-in, blocks of Messages + SelfTensProds with residuals,
    read-out with the meanflow factor) composed from the oracle's functions in `dtype`; the graph is the oracle's."""
    B, N = x1.shape[:2]
    dim_d = model.prods[0].L2.W.shape[1]
    dd = lambda p: p.detach().cpu().to(dtype)
    ref = ON.edges(x1.numpy(), r0, box)
    src, dst = torch.from_numpy(ref["src"]).long(), torch.from_numpy(ref["dst"]).long()
    r_ij = torch.from_numpy(ON.edge_vectors(x1.numpy(), ref["src"], ref["dst"], box)).to(dtype)
    x_a = torch.nn.functional.linear(one_hot.to(dtype), dd(model.embed.weight), dd(model.embed.bias))
    freqs = torch.exp(-torch.arange(32) / 31.0).to(dtype)
    ph = torch.cat([t.to(dtype)[:, None] * freqs, (t - s).to(dtype)[:, None] * freqs], 1)
    temb = torch.nn.functional.linear(torch.cat([torch.sin(ph), torch.cos(ph)], 1), dd(model.t_embed.lin1.weight),
                                      dd(model.t_embed.lin1.bias))
    x_a = x_a + temb[:, None]
    x_v = OP.tensor_linear(1, dd(model.v_readin.W), (x1 - x0).to(dtype)[..., None, :])
    x_d = torch.zeros(B, N, dim_d, 3, 3, dtype=dtype)
    for msg, prod in zip(model.messages, model.prods):
        w = {"L0": dd(msg.L0.W), "L1": dd(msg.L1.W), "L2": dd(msg.L2.W),
             "Y": {lab: dd(getattr(msg, f"Y_{lab}").W) for lab in OP.BEE_ORDER},
             "enc_W": dd(msg.lin_enc.weight), "enc_b": dd(msg.lin_enc.bias),
             "mlp_a": _to(_mlp_leaky_weights(msg.mlp_a), dtype)}
        d = OL.bee_messages(src, dst, B, N, r_ij, x_a, x_v, x_d, w, r0, radial_dtype=torch.float64)
        x_a, x_v, x_d = x_a + d[0], x_v + d[1], x_d + d[2]
        ws = {k: dd(getattr(prod, k).W) for k in ("L0", "R0", "L1", "R1", "L2", "R2")}
        ws["Y"] = {lab: dd(getattr(prod, f"Y_{lab}").W) for lab in OP.BEE_ORDER}
        ws.update(gn_a=dd(prod.gn_a.gamma), gn_v=dd(prod.gn_v.gamma), gn_d=dd(prod.gn_d.gamma))
        d = OL.self_tens_prods(x_a, x_v, x_d, ws)
        x_a, x_v, x_d = x_a + d[0], x_v + d[1], x_d + d[2]
    return (1. - (t - s).to(dtype)[:, None, None]) * OP.tensor_linear(1, dd(model.readout.W), x_v).squeeze(-2)


def test_denoiser_forward_matches_oracle_composition(pkg):
    """Small instance of the configs[3] assembly, end to end against the float64 oracle."""
    den = importlib.import_module("learned-dynamics_amd.denoiser")
    torch.manual_seed(0x947 + 4)
    dim_a, dim_v, dim_d, chan, blocks = 32, 16, 8, 32, 2
    box, r0, B, N = (24., 24., 24.), 6.0, 2, 300
    model = den.Denoiser(r0, dim_a, dim_v, dim_d, chan, blocks).cuda()
    x1 = torch.rand(B, N, 3) * 24
    x0 = x1 + torch.randn(B, N, 3)
    one_hot = torch.nn.functional.one_hot(torch.randint(0, 20, (B, N)), 20).float()
    s, t = torch.zeros(B), torch.rand(B)
    with torch.no_grad():
        v = model((s.cuda(), t.cuda()), x0.cuda(), x1.cuda(), one_hot.cuda(), box)
    v32 = denoiser_oracle(model, s, t, x0, x1, one_hot, box, r0, torch.float32)
    v64 = denoiser_oracle(model, s, t, x0, x1, one_hot, box, r0, torch.float64)
    assert_parity(v, v32, v64, "2-block denoiser v")


@pytest.mark.parametrize("plus_identity", [False, True])
def test_mlp_summed_over_rows_equals_sum_of_rows(pkg, plus_identity):
    """MLP.summed_over_rows applies the direct linear and the last layer after the segment sum: the result
    must equal the segment sum of the per-row MLP (archs/diffuser_atoms15.py:98-110, 244-246) up to the
    order of fp32 additions, also for empty segments and with the bias of the last layer counted once per
    row of the segment."""
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    ops = importlib.import_module("learned-dynamics_amd.ops")
    torch.manual_seed(5)
    d, N = 64, 300
    mlp = bee.MLP(d).cuda()
    with torch.no_grad():
        mlp.layers[4].bias.normal_()                      # make the bias term visible
    deg = torch.randint(0, 40, (N,))
    deg[::7] = 0
    src = torch.repeat_interleave(torch.arange(N), deg)
    E = int(src.numel())
    x = torch.randn(E, d).cuda()
    row_ptr = ops.segment_row_ptr(src.int().cuda(), N)
    with torch.no_grad():
        got = mlp.summed_over_rows(x, row_ptr, N, plus_identity=plus_identity, scale=0.1)
        per_row = mlp(x, plus_identity=plus_identity)
    f = torch.nn.functional
    L = mlp.layers

    def rows(dt):
        """The per-row MLP from plain torch modules in dt."""
        w = lambda t: t.detach().cpu().to(dt)
        xd = x.cpu().to(dt)
        h = f.leaky_relu(f.linear(xd, w(L[0].weight), w(L[0].bias)), 0.1)
        h = f.leaky_relu(f.linear(h, w(L[2].weight), w(L[2].bias)), 0.1)
        y = f.linear(h, w(L[4].weight), w(L[4].bias)) + f.linear(xd, w(mlp.lin_direct.weight))
        return y + xd if plus_identity else y

    assert_parity_of(per_row, rows, "MLP per row")
    assert_parity_of(got, lambda dt: 0.1 * torch.zeros(N, d, dtype=dt).index_add_(0, src, rows(dt)), "MLP summed over rows")
    assert not bool(got[deg.cuda() == 0].any())


@pytest.mark.parametrize("chan,dims,N", [(64, (48, 40, 16), 1500), (32, (256, 64, 16), 1100), (96, (32, 100, 8), 1300)])
def test_products_and_output_linears_in_one_kernel(pkg, chan, dims, N):
    """mg_bee_products_linear (13 products built in registers + the concatenated Y linears) against the
    stored-products path (node_products_kernel + one GEMM per rank) and against float64 einsums of the
    oracle's products; operands with rows of very different size."""
    ops = importlib.import_module("learned-dynamics_amd.ops")
    g = torch.Generator().manual_seed(chan + N)
    size = torch.rand(N, 1, generator=g) * 3 + 0.01
    l = [torch.randn(N, chan, generator=g) * size, torch.randn(N, 3, chan, generator=g) * size[:, None],
         torch.randn(N, 9, chan, generator=g) * size[:, None]]
    r = [torch.randn(N, chan, generator=g), torch.randn(N, 3, chan, generator=g), torch.randn(N, 9, chan, generator=g)]
    dev = [t.cuda() for t in l + r]
    lmax = torch.cat([t.reshape(N, -1) for t in l], 1).abs().amax(1)
    rmax = torch.cat([t.reshape(N, -1) for t in r], 1).abs().amax(1)
    bound = (9.0 * lmax * rmax).cuda()
    P0, P1, P2, nmax = ops.bee_node_products(*dev, want_node_max=True)
    # the oracle's products in the reference layout (rows, chan, 3..)
    to_ref = lambda t, k: t if k == 0 else t.reshape(N, 3 ** k, chan).transpose(1, 2).reshape(N, chan, *([3] * k))
    groups = (("000", "110", "220"), ("011", "101", "121", "211", "111"), ("022", "202", "112", "222", "212"))
    for rank, (labs, P, dim_out) in enumerate(zip(groups, (P0, P1, P2), dims)):
        W = (torch.randn(dim_out, len(labs) * chan, generator=g) / (len(labs) * chan) ** 0.5).cuda()
        y = ops.bee_products_linear(rank, W, *dev, bound)
        T = 3 ** rank
        assert y.shape == (N, dim_out) + (3,) * rank
        if rank == 0:
            stored = ops.tensor_linear_fwd(0, W, P.reshape(N, 3 * chan))
        else:
            stored = ops.tensor_linear_fwd(rank, W, P.reshape(N, T, len(labs) * chan), x_layout=ops.LAYOUT_COMP_CHAN)
        def ref(dt):
            pr = dict(zip(OP.BEE_ORDER, OP.bee(*[to_ref(t.to(dt), k) for k, t in enumerate(l)],
                                               *[to_ref(t.to(dt), k) for k, t in enumerate(r)])))
            return sum(torch.einsum("oc,nc...->no...", W[:, k * chan:(k + 1) * chan].cpu().to(dt), pr[lab])
                       for k, lab in enumerate(labs))

        assert_parity_of(y, ref, f"bee_products_linear rank {rank} chan={chan}")
        assert_parity_of(stored, ref, f"stored products + GEMM rank {rank} chan={chan}")
        # rows of small nodes keep their relative accuracy (per-node scales): the same bar on those rows alone,
        # where e_ref is the float32 formula's error on rows of that size
        small = (size[:, 0] < 0.1)
        if bool(small.any()):
            assert_parity_of(y[small.cuda()], lambda dt: ref(dt)[small], f"bee_products_linear rank {rank}, small rows")


@pytest.mark.parametrize("chan,dim_d,N", [(256, 16, 1001), (128, 5, 333), (64, 16, 70), (256, 1, 2)])
def test_rank2_products_and_their_output_linear_in_one_kernel(pkg, chan, dim_d, N):
    """mg_bee_node_products_rank2 against float64 einsums of the oracle's rank-2 products; node counts that leave the
    last workgroup partly filled, nodes of very different size, a weight with an uneven row stride."""
    ops = importlib.import_module("learned-dynamics_amd.ops")
    g = torch.Generator().manual_seed(chan + N)
    size = torch.rand(N, 1, generator=g) * 3 + 0.01
    l = [torch.randn(N, chan, generator=g) * size, torch.randn(N, 3, chan, generator=g) * size[:, None],
         torch.randn(N, 9, chan, generator=g) * size[:, None]]
    r = [torch.randn(N, chan, generator=g), torch.randn(N, 3, chan, generator=g), torch.randn(N, 9, chan, generator=g)]
    dev = [t.cuda() for t in l + r]
    wide = (torch.randn(dim_d, 5 * chan + 8, generator=g) / (5 * chan) ** 0.5).cuda()
    W = wide[:, :5 * chan]
    y = ops.bee_node_products_rank2(*dev, W)
    assert y.shape == (N, dim_d, 9)
    to_ref = lambda t, k: t if k == 0 else t.reshape(N, 3 ** k, chan).transpose(1, 2).reshape(N, chan, *([3] * k))
    labs = ("022", "202", "112", "222", "212")

    def ref(dt):
        pr = dict(zip(OP.BEE_ORDER, OP.bee(*[to_ref(t.to(dt), k) for k, t in enumerate(l)],
                                           *[to_ref(t.to(dt), k) for k, t in enumerate(r)])))
        return sum(torch.einsum("oc,ncxy->noxy", W[:, k * chan:(k + 1) * chan].cpu().to(dt), pr[lab])
                   for k, lab in enumerate(labs)).reshape(N, dim_d, 9)

    assert_parity_of(y, ref, f"rank-2 products + linear, chan={chan}, dim_d={dim_d}")
    small = (size[:, 0] < 0.1)
    if bool(small.any()):
        assert_parity_of(y[small.cuda()], lambda dt: ref(dt)[small], "rank-2 products + linear, small nodes")
    # the scalar and vector products written in the same pass, against the oracle's, and the emitted maxima are
    # exactly the maxima of what was written
    y3, Q0, Q1, nmax = ops.bee_node_products_rank2(*dev, W, want_lower_ranks=True)
    assert torch.equal(y3, y)

    def products(dt):
        return dict(zip(OP.BEE_ORDER, OP.bee(*[to_ref(t.to(dt), k) for k, t in enumerate(l)],
                                             *[to_ref(t.to(dt), k) for k, t in enumerate(r)])))
    for k, lab in enumerate(("000", "110", "220")):
        assert_parity_of(Q0[:, k], lambda dt: products(dt)[lab], f"scalar product {lab} from the node pass")
    for k, lab in enumerate(("011", "101", "121", "211", "111")):
        assert_parity_of(Q1[:, :, k], lambda dt: products(dt)[lab].transpose(1, 2), f"vector product {lab} from the node pass")
    assert nmax.shape == (N, chan // 64)
    assert torch.equal(nmax.amax(1), torch.maximum(Q0.abs().amax(dim=(1, 2)), Q1.abs().amax(dim=(1, 2, 3))))
    P2 = ops.bee_node_products(*dev)[2]
    # the rank-2 operands formed inside the kernel from x_d and the two weights: against the oracle fed with the
    # float64 (float32) operands L2 x_d, R2 x_d
    dim_in = 16 if chan == 256 else 5
    x_d = torch.randn(N, dim_in, 3, 3, generator=g) * size[:, None, None]
    W_L2, W_R2 = torch.randn(chan, dim_in, generator=g) / dim_in ** 0.5, torch.randn(chan, dim_in, generator=g) / dim_in ** 0.5
    y4, R0, R1, nmax4 = ops.bee_node_products_rank2(dev[0], dev[1], None, dev[3], dev[4], None, W, want_lower_ranks=True,
                                                     x_d=x_d.cuda(), L2t=W_L2.t().contiguous().cuda(),
                                                     R2t=W_R2.t().contiguous().cuda())

    def products_inside(dt):
        l2 = torch.einsum("ci,nixy->ncxy", W_L2.to(dt), x_d.to(dt))
        r2 = torch.einsum("ci,nixy->ncxy", W_R2.to(dt), x_d.to(dt))
        return dict(zip(OP.BEE_ORDER, OP.bee(to_ref(l[0].to(dt), 0), to_ref(l[1].to(dt), 1), l2,
                                             to_ref(r[0].to(dt), 0), to_ref(r[1].to(dt), 1), r2)))
    assert_parity_of(y4, lambda dt: sum(torch.einsum("oc,ncxy->noxy", W[:, k * chan:(k + 1) * chan].cpu().to(dt),
                                                      products_inside(dt)[lab])
                                        for k, lab in enumerate(labs)).reshape(N, dim_d, 9),
                     "rank-2 output with the rank-2 operands formed inside")
    assert_parity_of(R0[:, 2], lambda dt: products_inside(dt)["220"], "220 with the rank-2 operands formed inside")
    for k, lab in ((2, "121"), (3, "211")):
        assert_parity_of(R1[:, :, k], lambda dt: products_inside(dt)[lab].transpose(1, 2), f"{lab} with operands formed inside")
    assert torch.equal(nmax4.amax(1), torch.maximum(R0.abs().amax(dim=(1, 2)), R1.abs().amax(dim=(1, 2, 3))))
    # the stored-products route gives the same within the same bar
    stored = ops.tensor_linear_fwd(2, W, P2.reshape(N, 9, 5 * chan), x_layout=ops.LAYOUT_COMP_CHAN)
    assert_parity_of(stored.reshape(N, dim_d, 9), ref, "stored products + GEMM")
    with pytest.raises(RuntimeError, match="dim_d <= 16"):
        ops.bee_node_products_rank2(*dev, torch.zeros(32, 5 * chan, device="cuda"))
    assert ops.bee_node_products_rank2(*[t[:0] for t in dev], W).shape == (0, dim_d, 9)
    assert ops.bee_node_products_rank2(*[t[:0] for t in dev], W, want_lower_ranks=True)[2].shape == (0, 3, 5, chan)


def test_self_tens_prods_module_fused_path(pkg):
    """SelfTensProds at a size that takes the products + linears kernel (chan % 32 == 0, >= 8192 nodes)."""
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    torch.manual_seed(8)
    dim_a, dim_v, dim_d, chan = 64, 32, 16, 64
    mod = bee.SelfTensProds(dim_a, dim_v, dim_d, chan).cuda()
    with torch.no_grad():
        for gn in (mod.gn_a, mod.gn_v, mod.gn_d):
            gn.gamma.copy_(torch.randn_like(gn.gamma))
    x_a, x_v, x_d = torch.randn(2, 4200, dim_a), torch.randn(2, 4200, dim_v, 3), torch.randn(2, 4200, dim_d, 3, 3)
    with torch.no_grad():
        y_a, y_v, y_d = mod(x_a.cuda(), x_v.cuda(), x_d.cuda(), residual=True)
    dd = lambda t: t.detach().cpu()
    w = {k: dd(getattr(mod, k).W) for k in ("L0", "R0", "L1", "R1", "L2", "R2")}
    w["Y"] = {lab: dd(getattr(mod, f"Y_{lab}").W) for lab in OP.BEE_ORDER}
    w.update(gn_a=dd(mod.gn_a.gamma), gn_v=dd(mod.gn_v.gamma), gn_d=dd(mod.gn_d.gamma))
    r32 = OL.self_tens_prods(x_a, x_v, x_d, w)
    r64 = OL.self_tens_prods(x_a.double(), x_v.double(), x_d.double(), _to(w, torch.float64))
    for k, (got, x, name) in enumerate(zip((y_a, y_v, y_d), (x_a, x_v, x_d), "avd")):
        assert_parity(got, x + r32[k], x.double() + r64[k], f"SelfTensProds (products + linears kernel) y_{name}")


@pytest.mark.parametrize("chan,kind", [(64, "mixed"), (100, "short"), (7, "mixed"), (256, "long")])
def test_displacement_sums_kernel(ops, chan, kind):
    """mg_displacement_sums against float64 index_add of the per-edge tensors the reference materialises
    (archs/diffuser_atoms15.py:218-224), with empty rows, channel counts that are not a multiple of 64 and
    rows much longer than a wave."""
    g = torch.Generator().manual_seed(chan)
    N = 200
    deg = {"mixed": torch.randint(0, 40, (N,), generator=g), "short": torch.randint(0, 3, (N,), generator=g),
           "long": torch.randint(100, 300, (N,), generator=g)}[kind]
    src = torch.repeat_interleave(torch.arange(N), deg)
    E = int(src.numel())
    r = torch.randn(E, 3, generator=g) * 3
    phi = torch.randn(E, chan, generator=g)
    row_ptr = ops.segment_row_ptr(src.int().cuda(), N)
    s = 7.0 / 6.0
    A_a, A_v, A_d = ops.displacement_sums(row_ptr, r.cuda(), phi.cuda(), s)
    def sums(dt):
        u = OL.tens_sigmoid(1, r.to(dt) * s)
        p = phi.to(dt)
        return (torch.zeros(N, chan, dtype=dt).index_add_(0, src, p),
                torch.zeros(N, chan, 3, dtype=dt).index_add_(0, src, p[..., None] * u[:, None, :]),
                torch.zeros(N, chan, 3, 3, dtype=dt).index_add_(0, src, p[..., None, None] * u[:, None, :, None] * u[:, None, None, :]))

    assert_parity_of((A_a, A_v, A_d), sums, f"displacement_sums chan={chan} {kind}")
    assert not bool(A_a[(deg == 0).cuda()].any()) and not bool(A_d[(deg == 0).cuda()].any())


@pytest.mark.parametrize("dims", [(64, 32, 16), (128, 64, 16), (20, 12, 5)])
def test_displacement_tensors_module(pkg, dims):
    """DisplacementTensors.forward against the oracle's restatement of archs/diffuser_atoms15.py:206-225."""
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    dim_a, dim_v, dim_d = dims
    torch.manual_seed(0x947 + 14)
    box, r0 = (30., 30., 30.), 6.0
    pos = torch.rand(2, 500, 3) * 30
    mod = bee.DisplacementTensors(r0, dim_a, dim_v, dim_d).cuda()
    assert sorted(mod.state_dict()) == sorted(
        ["mlp_radial.0.weight", "mlp_radial.0.bias", "mlp_radial.1.lin_direct.weight"]
        + [f"mlp_radial.1.layers.{i}.{p}" for i in (0, 2, 4) for p in ("weight", "bias")] + ["readout_v.W", "readout_d.W"])
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, box, pos.cuda(), neighbours_max=256, celllist_max=64)
        A_a, A_v, A_d = mod(graph, r_ij)
    assert A_a.shape == (2, 500, dim_a) and A_v.shape == (2, 500, dim_v, 3) and A_d.shape == (2, 500, dim_d, 3, 3)
    src, dst = graph.src.cpu(), graph.dst.cpu()
    r_ref = torch.from_numpy(ON.edge_vectors(pos.numpy(), src.numpy(), dst.numpy(), box))
    dd = lambda t: t.detach().cpu().double()
    w = {"lin_W": dd(mod.mlp_radial[0].weight), "lin_b": dd(mod.mlp_radial[0].bias),
         "mlp": _mlp_leaky_weights(mod.mlp_radial[1]), "readout_v": dd(mod.readout_v.W), "readout_d": dd(mod.readout_d.W)}
    r64 = OL.displacement_tensors(src, 2, 500, r_ref.double(), w, r0)
    r32 = OL.displacement_tensors(src, 2, 500, r_ref, _to(w, torch.float32), r0, radial_dtype=torch.float64)
    for k, (got, name) in enumerate(zip((A_a, A_v, A_d), "avd")):
        assert_parity(got, r32[k], r64[k], f"DisplacementTensors {dims} A_{name}")

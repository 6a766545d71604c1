"""bf16-storage configuration (BASELINE configs[4]): features stored as bfloat16, fp32 accumulation.

Kernel tests feed the kernels bf16-representable inputs, so the float64 oracle sees exactly the same
numbers and the only differences are fp32 accumulation order and the final rounding of the stored
result to bf16 (relative 2^-9 of the value).  The stack test compares against the float64 oracle of
the float32 model at the tolerance the configuration states: rel 1e-2 of the output scale."""
import importlib

import pytest
import torch

from oracle import layers as OL
from oracle import neighbour as ON
from oracle import products as OP

pytestmark = pytest.mark.gpu

BF16_EPS = 2.0 ** -8          # one ulp of bfloat16 relative to the value


def _bf(t):
    return t.to(torch.bfloat16)


def _close_bf16(out, ref, extra_abs=0.0):
    """out: bf16 or fp32 device tensor; ref: float64.  |out - ref| <= ulp_bf16(ref)/2 (+ accumulate slack)."""
    out = out.cpu().double()
    tol = BF16_EPS * ref.abs() * 1.01 + 1e-5 * ref.abs().max() + extra_abs
    bad = (out - ref).abs() > tol
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} out of tolerance, max err {(out - ref).abs().max():.3e}"


@pytest.mark.parametrize("shape", [(5000, 128, 256, 1, 1), (777, 384, 128, 2, 1), (3000, 640, 96, 0, 3),
                                   (1800, 32, 128, 0, 9), (130, 96, 8, 1, 1)])
@pytest.mark.parametrize("y_bf16", [True, False])
def test_linear_bf16(ops, shape, y_bf16):
    rows, dim_in, dim_out, act, comps = shape
    g = torch.Generator().manual_seed(rows + dim_in)
    x = _bf(torch.randn(rows, dim_in, generator=g))
    W = torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5
    b = torch.randn(dim_out, generator=g)
    # the kernel uses the hi + mid bf16 pieces of W: 16 significand bits
    hi = _bf(W).float()
    W16 = (hi + _bf(W - hi).float()).double()
    pre = x.double() @ W16.t() + b.double()
    ref = {0: pre, 1: torch.nn.functional.silu(pre), 2: torch.where(pre > 0, pre, 0.1 * pre)}[act]
    y = ops.tensor_linear_bf16(W.cuda(), x.cuda(), bias=b.cuda(), act=act, out_comps=comps,
                               out_dtype=torch.bfloat16 if y_bf16 else torch.float32)
    if comps > 1:
        assert y.shape == (rows // comps, dim_out, comps)
        ref = ref.reshape(rows // comps, comps, dim_out).transpose(1, 2)
    if y_bf16:
        _close_bf16(y, ref)
    else:
        torch.testing.assert_close(y.cpu().double(), ref, rtol=1e-5, atol=2e-6 * dim_in ** 0.5)
    # accumulate into an existing fp32 result
    if not y_bf16 and comps == 1:
        y2 = ops.tensor_linear_bf16(W.cuda(), x.cuda(), out=y.clone(), accumulate=True)
        torch.testing.assert_close(y2.cpu().double(), ref + x.double() @ W16.t(), rtol=1e-5, atol=4e-6 * dim_in ** 0.5)


def test_linear_bf16_errors(ops):
    W = torch.randn(64, 48, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of 32"):
        ops.tensor_linear_bf16(W, torch.zeros(10, 48, device="cuda", dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="must be bfloat16"):
        ops.tensor_linear_bf16(torch.randn(64, 64, device="cuda"), torch.zeros(10, 64, device="cuda"))
    assert ops.tensor_linear_bf16(torch.randn(64, 64, device="cuda"),
                                  torch.zeros(0, 64, device="cuda", dtype=torch.bfloat16)).shape == (0, 64)


@pytest.mark.parametrize("chan", [128, 64, 40])
def test_bee_message_bf16(ops, chan):
    torch.manual_seed(chan)
    N, E = 200, 3000
    src = torch.sort(torch.randint(0, N, (E,))).values
    src[src == 5] = 6
    dst = torch.randint(0, N, (E,))
    r = torch.randn(E, 3) * 2.5
    La, Lv, Ld = _bf(torch.randn(N, chan)), _bf(torch.randn(N, chan, 3)), _bf(torch.randn(N, chan, 3, 3))
    encW, encb = torch.randn(chan, 8) * 0.3, torch.randn(chan)
    enc, rhat = ops.bee_edge_geometry(r.cuda(), 6.0)
    row_ptr = ops.segment_row_ptr(src.int().cuda(), N)
    Lv_cm = Lv.transpose(1, 2).contiguous()
    Ld_cm = Ld.reshape(N, chan, 9).transpose(1, 2).contiguous()
    P0, S1, S2 = ops.bee_message_bf16(row_ptr, dst.int().cuda(), rhat, enc, La.cuda(), Lv_cm.cuda(), Ld_cm.cuda(),
                                      encW.cuda(), encb.cuda(), node_order=torch.randperm(N).int().cuda())
    assert P0.dtype == S1.dtype == S2.dtype == torch.bfloat16
    phi_a = torch.nn.functional.linear(enc.cpu().double(), encW.double(), encb.double())
    rh = rhat.cpu().double()
    phi_v = phi_a[..., None] * rh[:, None, :]
    phi_d = phi_a[..., None, None] * rh[:, None, None, :] * rh[:, None, :, None]
    prods = dict(zip(OP.BEE_ORDER, OP.bee(La.double()[dst], Lv.double()[dst], Ld.double()[dst], phi_a, phi_v, phi_d)))
    for k, lab in enumerate(("000", "110", "220")):
        _close_bf16(P0[:, k], prods[lab])
    for k, lab in enumerate(("011", "101", "121", "211", "111")):
        ref = torch.zeros(N, chan, 3, dtype=torch.float64).index_add_(0, src, prods[lab])
        _close_bf16(S1[:, :, k], ref.transpose(1, 2))
    for k, lab in enumerate(("022", "202", "112", "222", "212")):
        ref = torch.zeros(N, chan, 3, 3, dtype=torch.float64).index_add_(0, src, prods[lab]).reshape(N, chan, 9)
        _close_bf16(S2[:, :, k], ref.transpose(1, 2))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_node_products(ops, dtype):
    torch.manual_seed(5)
    N, chan = 333, 48
    mk = lambda *s: torch.randn(*s).to(dtype)
    l0, l1, l2, r0, r1, r2 = mk(N, chan), mk(N, chan, 3), mk(N, chan, 3, 3), mk(N, chan), mk(N, chan, 3), mk(N, chan, 3, 3)
    cm1 = lambda t: t.transpose(1, 2).contiguous().cuda()
    cm2 = lambda t: t.reshape(N, chan, 9).transpose(1, 2).contiguous().cuda()
    P0, P1, P2 = ops.bee_node_products(l0.cuda(), cm1(l1), cm2(l2), r0.cuda(), cm1(r1), cm2(r2))
    d = lambda t: t.double()
    prods = dict(zip(OP.BEE_ORDER, OP.bee(d(l0), d(l1), d(l2), d(r0), d(r1), d(r2))))
    check = _close_bf16 if dtype == torch.bfloat16 else \
        (lambda out, ref: torch.testing.assert_close(out.cpu().double(), ref, rtol=1e-5, atol=1e-5))
    for k, lab in enumerate(("000", "110", "220")):
        check(P0[:, k], prods[lab])
    for k, lab in enumerate(("011", "101", "121", "211", "111")):
        check(P1[:, :, k], prods[lab].transpose(1, 2))
    for k, lab in enumerate(("022", "202", "112", "222", "212")):
        check(P2[:, :, k], prods[lab].reshape(N, chan, 9).transpose(1, 2))


@pytest.mark.parametrize("feat", [128, 8, 300, 1024])
def test_segment_sum_bf16(ops, feat):
    torch.manual_seed(feat)
    N, E = 150, 4000
    src = torch.sort(torch.randint(0, N, (E,))).values
    src[src == 9] = 10
    x = _bf(torch.randn(E, feat))
    row_ptr = ops.segment_row_ptr(src.int().cuda(), N)
    out = ops.segment_sum_csr_bf16(x.cuda(), row_ptr, N, 0.1)
    ref = 0.1 * torch.zeros(N, feat, dtype=torch.float64).index_add_(0, src, x.double())
    _close_bf16(out, ref)
    assert torch.all(out[9] == 0)


def _mlp_leaky_weights(m):
    L = m.layers
    dd = lambda t: t.detach().cpu().double()
    return {"W_direct": dd(m.lin_direct.weight), "W1": dd(L[0].weight), "b1": dd(L[0].bias), "W2": dd(L[2].weight),
            "b2": dd(L[2].bias), "W3": dd(L[4].weight), "b3": dd(L[4].bias)}


def test_stack_bf16_against_fp32_oracle(pkg):
    """2 x [Messages -> SelfTensProds] with bf16 storage against the float64 oracle of the same
    float32 model: rel 1e-2 of the output scale (the tolerance the bf16 configuration states)."""
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    b16 = importlib.import_module("learned-dynamics_amd.bee_layers_bf16")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    torch.manual_seed(0x947 + 5)
    dim, chan, blocks = 64, 64, 2
    B, N, r0 = 1, 700, 6.0
    box = (24., 24., 24.)
    pos = torch.rand(B, N, 3) * 24
    msgs = [bee.Messages(r0, dim, dim, dim, chan).cuda() for _ in range(blocks)]
    prods = [bee.SelfTensProds(dim, dim, dim, chan).cuda() for _ in range(blocks)]
    x_a, x_v, x_d = torch.randn(B, N, dim), torch.randn(B, N, dim, 3) / 3 ** 0.5, torch.randn(B, N, dim, 3, 3) / 3
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, box, pos.cuda(), neighbours_max=256, celllist_max=64)
        y_a, y_v, y_d = b16.stack_forward(msgs, prods, graph, r_ij, x_a.cuda(), x_v.cuda(), x_d.cuda())
    dd = lambda p: p.detach().cpu().double()
    src, dst = graph.src.cpu(), graph.dst.cpu()
    r_ref = torch.from_numpy(ON.edge_vectors(pos.numpy(), src.numpy(), dst.numpy(), box)).double()
    ra, rv, rd = x_a.double(), x_v.double(), x_d.double()
    for msg, prod in zip(msgs, prods):
        w = {"L0": dd(msg.L0.W), "L1": dd(msg.L1.W), "L2": dd(msg.L2.W),
             "Y": {lab: dd(getattr(msg, f"Y_{lab}").W) for lab in OP.BEE_ORDER},
             "enc_W": dd(msg.lin_enc.weight), "enc_b": dd(msg.lin_enc.bias), "mlp_a": _mlp_leaky_weights(msg.mlp_a)}
        d = OL.bee_messages(src, dst, B, N, r_ref, ra, rv, rd, w, r0)
        ra, rv, rd = ra + d[0], rv + d[1], rd + d[2]
        ws = {k: dd(getattr(prod, k).W) for k in ("L0", "R0", "L1", "R1", "L2", "R2")}
        ws["Y"] = {lab: dd(getattr(prod, f"Y_{lab}").W) for lab in OP.BEE_ORDER}
        ws.update(gn_a=dd(prod.gn_a.gamma), gn_v=dd(prod.gn_v.gamma), gn_d=dd(prod.gn_d.gamma))
        d = OL.self_tens_prods(ra, rv, rd, ws)
        ra, rv, rd = ra + d[0], rv + d[1], rd + d[2]
    for out, ref in ((y_a, ra), (y_v, rv), (y_d, rd)):
        scale = float(ref.abs().max())
        err = (out.cpu().double() - ref).abs()
        assert float(err.max()) <= 1e-2 * scale, (float(err.max()), scale)
        assert float(err.pow(2).mean().sqrt()) <= 1e-2 * float(ref.pow(2).mean().sqrt())


@pytest.mark.parametrize("dim_in,dim_out,act,kind,want_rows", [(256, 256, 2, "long", False), (384, 128, 0, "short", True),
                                                               (64, 384, 1, "aligned", True), (128, 512, 2, "mixed", False)])
def test_linear_bf16_with_row_sums_in_the_epilogue(ops, dim_in, dim_out, act, kind, want_rows):
    """out[s] = scale * sum over the rows of segment s of the bf16-rounded act(x W^T + b): exactly the fp32 sum
    of what mg_tensor_linear_bf16 writes (order of additions aside), for segments placed in every way relative
    to the kernel's 32-row blocks."""
    g = torch.Generator().manual_seed(dim_in + dim_out)
    n_seg = 300
    if kind == "long":
        lengths = torch.randint(40, 140, (n_seg,), generator=g)
    elif kind == "short":
        lengths = torch.randint(0, 9, (n_seg,), generator=g)
    elif kind == "aligned":
        lengths = torch.tensor([32, 64, 1, 31, 32, 0, 0, 96, 33, 31] * (n_seg // 10))
    else:
        lengths = torch.cat([torch.randint(0, 5, (n_seg // 2,), generator=g),
                             torch.randint(20, 300, (n_seg - n_seg // 2,), generator=g)])[torch.randperm(n_seg, generator=g)]
    seg = torch.repeat_interleave(torch.arange(n_seg), lengths)
    rows = int(seg.numel())
    x = torch.randn(rows, dim_in, generator=g).cuda().to(torch.bfloat16)
    W = (torch.randn(dim_out, dim_in, generator=g) / dim_in ** 0.5).cuda()
    b = torch.randn(dim_out, generator=g).cuda()
    row_ptr = ops.segment_row_ptr(seg.int().cuda(), n_seg)
    out, y = ops.tensor_linear_bf16_rowsum(W, x, row_ptr, seg.int().cuda(), n_seg, bias=b, act=act, scale=0.5,
                                           want_rows=want_rows)
    y_ref = ops.tensor_linear_bf16(W, x, bias=b, act=act)
    if want_rows:
        assert torch.equal(y, y_ref)
    else:
        assert y is None
    ref = 0.5 * torch.zeros(n_seg, dim_out, dtype=torch.float64).index_add_(0, seg, y_ref.double().cpu())
    torch.testing.assert_close(out.cpu().double(), ref, rtol=1e-5, atol=2e-6 * float(ref.abs().max()))
    assert not bool(out[(lengths == 0).cuda()].any())


@pytest.mark.parametrize("kind,dim_in", [("mixed", 384), ("short", 384), ("tiny", 96), ("aligned", 32)])
def test_scalar_message_chain_in_one_kernel(ops, kind, dim_in):
    """mg_mlp_chain_bf16 against the three separate kernels it replaces: the sums over segments of the bf16-rounded
    psi = Y x and h2 = leaky(W2 leaky(W1 psi + b1) + b2).  psi is computed in the same order as by the plain
    kernel, so its sums agree to fp32 summation order.  The two later layers multiply in a permuted order of the
    input channels, so a few bf16 roundings of h1 and h2 fall the other way (one unit in the last place, 2^-8
    relative): the sums of h2 are compared with an allowance of two such units of the largest element, and no
    more than 5 % of them may differ beyond fp32 summation order at all."""
    g = torch.Generator().manual_seed(11 + dim_in)
    n_seg = 300
    if kind == "mixed":
        lengths = torch.cat([torch.randint(0, 5, (n_seg // 2,), generator=g),
                             torch.randint(20, 300, (n_seg - n_seg // 2,), generator=g)])[torch.randperm(n_seg, generator=g)]
    elif kind == "short":
        lengths = torch.randint(0, 9, (n_seg,), generator=g)
    elif kind == "tiny":
        n_seg = 4
        lengths = torch.tensor([30, 0, 6, 1])
    else:
        lengths = torch.tensor([32, 64, 1, 31, 32, 0, 0, 96, 33, 31] * (n_seg // 10))
    seg = torch.repeat_interleave(torch.arange(n_seg), lengths)
    rows = int(seg.numel())
    x = torch.randn(rows, dim_in, generator=g).cuda().to(torch.bfloat16)
    Y = (torch.randn(128, dim_in, generator=g) / dim_in ** 0.5).cuda()
    W1 = (torch.randn(256, 128, generator=g) / 128 ** 0.5).cuda()
    W2 = (torch.randn(256, 256, generator=g) / 256 ** 0.5).cuda()
    b1, b2 = torch.randn(256, generator=g).cuda(), torch.randn(256, generator=g).cuda()
    segc = seg.int().cuda()
    row_ptr = ops.segment_row_ptr(segc, n_seg)
    s_psi, s_h = ops.mlp_chain_bf16(Y, x, W1, b1, W2, b2, row_ptr, segc, n_seg)
    psi = ops.tensor_linear_bf16(Y, x)
    h2 = ops.tensor_linear_bf16(W2, ops.tensor_linear_bf16(W1, psi, bias=b1, act=ops.ACT_LEAKY), bias=b2,
                                act=ops.ACT_LEAKY)
    ref_psi = torch.zeros(n_seg, 128, dtype=torch.float64).index_add_(0, seg, psi.double().cpu())
    ref_h = torch.zeros(n_seg, 256, dtype=torch.float64).index_add_(0, seg, h2.double().cpu())
    torch.testing.assert_close(s_psi.cpu().double(), ref_psi, rtol=1e-5, atol=2e-6 * float(ref_psi.abs().max()))
    err = (s_h.cpu().double() - ref_h).abs()
    ulp = 2.0 ** -8 * float(h2.float().abs().max())
    assert float(err.max()) <= 2 * ulp + 1e-5 * float(ref_h.abs().max())
    assert float((err > 1e-5 * ref_h.abs().clamp_min(1.0)).double().mean()) < 0.05
    empty = (lengths == 0).cuda()
    assert not bool(s_psi[empty].any()) and not bool(s_h[empty].any())


def test_messages_bf16_chain_equals_separate_kernels(pkg, ops):
    """messages_forward with the one-kernel scalar chain against the same call with the separate kernels."""
    bl = importlib.import_module("learned-dynamics_amd.bee_layers")
    b16 = importlib.import_module("learned-dynamics_amd.bee_layers_bf16")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    torch.manual_seed(3)
    N, chan, r0 = 4096, 128, 5.0
    side = (N / 0.1) ** (1 / 3)
    pos = (torch.rand(1, N, 3) * side).cuda()
    mod = bl.Messages(r0, chan, chan, chan, chan).cuda()
    x_a, x_v, x_d = torch.randn(1, N, chan).cuda(), torch.randn(1, N, chan, 3).cuda(), torch.randn(1, N, chan, 3, 3).cuda()
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, (side, side, side), pos, neighbours_max=256, celllist_max=64)
        s = b16.to_storage(x_a, x_v, x_d)
        out_chain = b16.messages_forward(mod, graph, r_ij, *s, chain=True)
        out_sep = b16.messages_forward(mod, graph, r_ij, *s, chain=False)
    assert graph.src.numel() >= 4096                          # the chain kernel is the one that ran
    assert torch.equal(out_chain[1], out_sep[1]) and torch.equal(out_chain[2], out_sep[2])
    a, b = out_chain[0].float(), out_sep[0].float()
    assert float((a - b).abs().max()) <= 2.0 ** -6 * float(b.abs().max())


@pytest.mark.parametrize("comps,chan,groups,with_res", [(1, 128, 8, True), (3, 128, 8, True), (9, 128, 8, False),
                                                        (9, 64, 4, True), (3, 24, 8, True), (9, 512, 8, True)])
def test_tens_group_norm_bf16(ops, comps, chan, groups, with_res):
    """mg_tens_group_norm_bf16 against TensGroupNorm's formula (managan/tensor_products.py:215-232) in float64 on the
    same bf16 inputs: the result is the exact value rounded to bf16, up to one unit in the last place where the fp32
    scale falls on the other side of a rounding boundary."""
    g = torch.Generator().manual_seed(comps * chan + groups)
    batch, nodes, eps = 2, 777, 1e-5
    shape = (batch * nodes, chan) if comps == 1 else (batch * nodes, comps, chan)
    y = (torch.randn(shape, generator=g) * torch.rand(1, generator=g) * 3).to(torch.bfloat16)
    y[nodes:] *= 0.25                                        # the two boxes have different statistics
    res = torch.randn(shape, generator=g).to(torch.bfloat16) if with_res else None
    gamma = torch.randn(chan, generator=g)
    out = ops.tens_group_norm_bf16(y.cuda(), batch, groups, gamma.cuda(), eps, res.cuda() if with_res else None)
    x = y.double().reshape(batch, nodes, comps, groups, chan // groups)
    m2 = (x * x).sum(2, keepdim=True).mean(dim=(1, 4), keepdim=True)
    ref = (x / torch.sqrt(eps + m2)).reshape(y.shape) * gamma.double()
    fp32_noise = 3e-7 * ref.abs()                            # of the fp32 value that is rounded to bfloat16
    if with_res:
        fp32_noise = 3e-7 * (ref.abs() + res.double().abs())  # the sum may cancel
        ref = ref + res.double()
    assert out.dtype == torch.bfloat16 and out.shape == y.shape
    err = (out.cpu().double() - ref).abs()
    half_ulp = 2.0 ** (torch.floor(torch.log2(ref.abs().clamp_min(1e-30))) - 8)      # of bfloat16 at the exact value
    assert bool((err <= 2.02 * half_ulp + fp32_noise).all())
    assert float((err > 1.001 * half_ulp + fp32_noise).double().mean()) < 0.01       # almost always correctly rounded
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ops.tens_group_norm_bf16(torch.zeros(4, 12, dtype=torch.bfloat16, device="cuda"), 1, 4, torch.ones(12, device="cuda"), eps)

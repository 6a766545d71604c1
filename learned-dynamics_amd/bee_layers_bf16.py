"""bf16-storage forward of the rank-0/1/2 blocks (archs/diffuser_atoms15.py:59-110,227-253):
the same modules and parameters as bee_layers.py (float32 weights, state dicts unchanged), with every
feature tensor that lives in HBM stored as bfloat16 and every product and sum done in fp32.

Storage layout: component-major, x_a (rows, dim_a), x_v (rows, 3, dim_v), x_d (rows, 9, dim_d) with
rows = batch * nodes, so every linear map is one plain GEMM over (row, component) rows and the edge
kernel's gathers are unit stride.  to_storage / from_storage convert from and to the reference's
(batch, nodes, chan, 3, 3) float32 tensors at the ends of a stack.

What is rounded to bf16: the node features between modules, L_k x_k, the per-edge scalar products
and the hidden activations of the per-edge MLP, the per-node product sums.  Weights keep 16
significand bits.  Group-norm statistics are taken in fp32.
"""
import torch

from . import ops
from .bee_layers import LABELS_0, LABELS_1, LABELS_2, Messages, SelfTensProds, _derived
from .graph_layers import Graph


def to_storage(x_a, x_v, x_d):
    """(B,N,da), (B,N,dv,3), (B,N,dd,3,3) float32 -> (rows,da), (rows,3,dv), (rows,9,dd) bfloat16."""
    B, N = x_a.shape[:2]
    rows = B * N
    return (x_a.reshape(rows, -1).to(torch.bfloat16).contiguous(),
            x_v.reshape(rows, -1, 3).transpose(1, 2).to(torch.bfloat16).contiguous(),
            x_d.reshape(rows, x_d.shape[2], 9).transpose(1, 2).to(torch.bfloat16).contiguous())


def from_storage(s_a, s_v, s_d, batch):
    """Inverse of to_storage (float32 result)."""
    rows = s_a.shape[0]
    N = rows // batch
    return (s_a.float().reshape(batch, N, -1),
            s_v.float().transpose(1, 2).reshape(batch, N, -1, 3).contiguous(),
            s_d.float().transpose(1, 2).reshape(batch, N, -1, 3, 3).contiguous())


def _lin(W, x, comps):
    """x (rows, comps, dim_in) or (rows, dim_in) bf16 -> same leading shape with dim_out."""
    rows = x.shape[0]
    y = ops.tensor_linear_bf16(W, x.reshape(rows * comps, x.shape[-1]))
    return y if comps == 1 else y.reshape(rows, comps, -1)


def _cat_Y(mod, labels, scale=None):
    """[Y_lab.W for lab in labels] concatenated along K (optionally scaled), kept while the weights are unchanged so
    that its packed planes stay valid from one forward to the next."""
    params = tuple(getattr(mod, f"Y_{lab}").W for lab in labels)

    def make():
        W = torch.cat(params, dim=1)
        return W if scale is None else W * scale
    return _derived(mod, ("cat_Y_bf16", labels, scale), params, make)


def mlp_forward(mlp, x, plus_identity=False):
    """bee_layers.MLP on bf16 rows: lin_direct(x) [+ x] + layers(x)."""
    Wd = mlp.lin_direct.weight
    if plus_identity:
        W0 = Wd
        Wd = _derived(mlp, "direct_plus_identity", (W0,),
                      lambda: W0 + torch.eye(W0.shape[0], device=W0.device, dtype=W0.dtype))
    Ls = mlp.layers
    h = ops.tensor_linear_bf16(Ls[0].weight, x, bias=Ls[0].bias, act=ops.ACT_LEAKY)
    h = ops.tensor_linear_bf16(Ls[2].weight, h, bias=Ls[2].bias, act=ops.ACT_LEAKY)
    out = ops.tensor_linear_bf16(Wd, x, out_dtype=torch.float32)
    ops.tensor_linear_bf16(Ls[4].weight, h, bias=Ls[4].bias, out=out, accumulate=True)
    return out.to(torch.bfloat16)


def _mlp_after_sums(mlp, s_x, s_h, row_ptr, plus_identity, scale):
    """(W_direct [+ 1]) s_x + W_last s_h + count * b_last, scaled, as bf16: the linear tail of the MLP applied to
    the sums over rows of its input and of its last hidden layer."""
    Wd = mlp.lin_direct.weight
    if plus_identity:
        W0 = Wd
        Wd = _derived(mlp, "direct_plus_identity", (W0,),
                      lambda: W0 + torch.eye(W0.shape[0], device=W0.device, dtype=W0.dtype))
    last = mlp.layers[4]
    out = ops.tensor_linear_bf16(Wd, s_x, out_dtype=torch.float32)
    ops.tensor_linear_bf16(last.weight, s_h, out=out, accumulate=True)
    count = (row_ptr[1:] - row_ptr[:-1]).to(out.dtype)[:, None]
    return torch.addcmul(out, count, last.bias[None, :]).mul_(scale).to(torch.bfloat16)


def mlp_summed_over_rows(mlp, x, row_ptr, n_out, plus_identity=False, scale=1.0, seg=None, s_x=None):
    """scale * (sum over each CSR segment of mlp_forward(mlp, x, plus_identity)) as bf16 (n_out, d).  The
    direct linear and the last layer are linear in their inputs, so they are applied to the summed rows
    (bee_layers.MLP.summed_over_rows).  With seg (the segment of every row) the second layer sums its
    bf16-rounded output rows in its own epilogue and never stores them; s_x: the sums of x if the caller has
    them.  Sums are accumulated in fp32 and stored in bf16 like every other feature."""
    Ls = mlp.layers
    h = ops.tensor_linear_bf16(Ls[0].weight, x, bias=Ls[0].bias, act=ops.ACT_LEAKY)
    if seg is not None and ops.bf16_rowsum_supported(h.shape[0], Ls[2].in_features, Ls[2].out_features):
        s_h, _ = ops.tensor_linear_bf16_rowsum(Ls[2].weight, h, row_ptr, seg, n_out, bias=Ls[2].bias, act=ops.ACT_LEAKY)
        s_h = s_h.to(torch.bfloat16)
    else:
        h = ops.tensor_linear_bf16(Ls[2].weight, h, bias=Ls[2].bias, act=ops.ACT_LEAKY)
        s_h = ops.segment_sum_csr_bf16(h, row_ptr, n_out)
    del h
    if s_x is None:
        s_x = ops.segment_sum_csr_bf16(x, row_ptr, n_out)
    return _mlp_after_sums(mlp, s_x, s_h, row_ptr, plus_identity, scale)


def messages_forward(mod: Messages, graph: Graph, r_ij, s_a, s_v, s_d, node_order="cell", chain=True):
    """Messages.forward (archs/diffuser_atoms15.py:238-253) on storage tensors; returns the three
    0.1 * (sum over edges) increments in storage layout."""
    if isinstance(node_order, str):
        node_order = getattr(graph, "cell_order", None)
    rows = s_a.shape[0]
    La, Lv, Ld = _lin(mod.L0.W, s_a, 1), _lin(mod.L1.W, s_v, 3), _lin(mod.L2.W, s_d, 9)
    enc, rhat = ops.bee_edge_geometry(r_ij.contiguous(), mod.r0)
    P0, S1, S2 = ops.bee_message_bf16(graph.row_ptr, graph.dst32, rhat, enc, La, Lv, Ld, mod.lin_enc.weight,
                                      mod.lin_enc.bias, node_order=node_order)
    E, chan = P0.shape[0], P0.shape[2]
    Y0 = _cat_Y(mod, LABELS_0)
    Ls = mod.mlp_a.layers
    if chain and ops.mlp_chain_bf16_supported(E, 3 * chan, Y0.shape[0], Ls[0].out_features) \
            and Ls[2].out_features == Ls[0].out_features:
        # psi_a and both hidden layers stay in registers; only their sums over the edges of a node are written
        s_psi, s_h = ops.mlp_chain_bf16(Y0, P0.reshape(E, 3 * chan), Ls[0].weight, Ls[0].bias, Ls[2].weight,
                                        Ls[2].bias, graph.row_ptr, graph.src32, rows)
        B_a = _mlp_after_sums(mod.mlp_a, s_psi.to(torch.bfloat16), s_h.to(torch.bfloat16), graph.row_ptr, True, 0.1)
    else:
        if ops.bf16_rowsum_supported(E, 3 * chan, Y0.shape[0]):
            s_psi, psi_a = ops.tensor_linear_bf16_rowsum(Y0, P0.reshape(E, 3 * chan), graph.row_ptr, graph.src32,
                                                         rows, want_rows=True)
            s_psi = s_psi.to(torch.bfloat16)
        else:
            psi_a, s_psi = ops.tensor_linear_bf16(Y0, P0.reshape(E, 3 * chan)), None
        B_a = mlp_summed_over_rows(mod.mlp_a, psi_a, graph.row_ptr, rows, plus_identity=True, scale=0.1,
                                   seg=graph.src32, s_x=s_psi)
    B_v = _lin(_cat_Y(mod, LABELS_1, 0.1), S1.reshape(rows, 3, 5 * chan), 3)
    B_d = _lin(_cat_Y(mod, LABELS_2, 0.1), S2.reshape(rows, 9, 5 * chan), 9)
    return B_a, B_v, B_d


def _flat_gamma(gn):
    return _derived(gn, "flat_gamma", (gn.gamma,), lambda: gn.gamma.detach().reshape(-1).contiguous())


def _tens_group_norm(gn, y, res, batch):
    """TensGroupNorm (managan/tensor_products.py:215-232) on a component-major storage tensor
    y (rows, T, dim) or (rows, dim): statistics in fp32 over (nodes, components, group channels)."""
    rows = y.shape[0]
    comps = 1 if y.dim() == 2 else y.shape[1]
    if ops.tens_group_norm_bf16_supported(comps, gn.chan):
        return ops.tens_group_norm_bf16(y, batch, gn.groups, _flat_gamma(gn), gn.epsilon, res)
    x = y.float().reshape(batch, rows // batch, -1, gn.groups, gn.chan // gn.groups)
    m2 = (x * x).sum(2, keepdim=True).mean(dim=(1, 4), keepdim=True)
    out = (x * torch.rsqrt(gn.epsilon + m2)).reshape(y.shape) * gn.gamma.reshape(-1)
    if res is not None:
        out = out + res.float()
    return out.to(torch.bfloat16)


def self_tens_prods_forward(mod: SelfTensProds, s_a, s_v, s_d, batch, residual=True):
    """SelfTensProds.forward (archs/diffuser_atoms15.py:80-95) on storage tensors."""
    rows = s_a.shape[0]
    chan = mod.L0.W.shape[0]
    P0, P1, P2 = ops.bee_node_products(_lin(mod.L0.W, s_a, 1), _lin(mod.L1.W, s_v, 3), _lin(mod.L2.W, s_d, 9),
                                       _lin(mod.R0.W, s_a, 1), _lin(mod.R1.W, s_v, 3), _lin(mod.R2.W, s_d, 9))
    y_a = _lin(_cat_Y(mod, LABELS_0), P0.reshape(rows, 3 * chan), 1)
    y_v = _lin(_cat_Y(mod, LABELS_1), P1.reshape(rows, 3, 5 * chan), 3)
    y_d = _lin(_cat_Y(mod, LABELS_2), P2.reshape(rows, 9, 5 * chan), 9)
    return (_tens_group_norm(mod.gn_a, y_a, s_a if residual else None, batch),
            _tens_group_norm(mod.gn_v, y_v, s_v if residual else None, batch),
            _tens_group_norm(mod.gn_d, y_d, s_d if residual else None, batch))


def stack_forward(messages, prods, graph, r_ij, x_a, x_v, x_d, node_order="cell"):
    """blocks x [Messages (residual) -> SelfTensProds (residual)] with bf16 storage between and
    inside the modules; float32 reference-layout tensors in and out."""
    batch = x_a.shape[0]
    s_a, s_v, s_d = to_storage(x_a, x_v, x_d)
    for msg, prod in zip(messages, prods):
        d_a, d_v, d_d = messages_forward(msg, graph, r_ij, s_a, s_v, s_d, node_order=node_order)
        s_a, s_v, s_d = s_a + d_a, s_v + d_v, s_d + d_d
        s_a, s_v, s_d = self_tens_prods_forward(prod, s_a, s_v, s_d, batch, residual=True)
    return from_storage(s_a, s_v, s_d, batch)

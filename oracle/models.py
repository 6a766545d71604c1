"""TEST INFRASTRUCTURE ONLY — CPU restatement (PyTorch, any float dtype) of the reference's PaiNN meanflow denoiser
and of the samplers / rollout loop that call it, assembled from oracle/layers.py.

Follows (relative to the reference checkout):
  archs/meanflow_painn8.py:102-125   Block.forward (bond message, radius message, update, residuals)
  archs/meanflow_painn8.py:127-143   CPaiNN.forward
  archs/meanflow_painn8.py:145-165   TimeEmbedding
  archs/meanflow_painn8.py:174-183   PosEmbed
  archs/meanflow_painn8.py:185-217   SE3ITO.forward, get_v_pred
  archs/meanflow_painn8.py:302-310   Meanflow.generate (one network call per frame)
  archs/diffuser_atoms15.py:511-516,536-555   epsilon combination and the reverse-diffusion loop
  managan/predictor.py:164-176       ModelPredictor.predict (frame fed back L times)

Weights come as a flat dict name -> tensor with the reference's parameter names (a state dict); the per-atom
embedding of ResidueAtomEmbed is replaced by a linear map of one-hot atom types ("atom_embed.lin.*"), as in the
product's mirror.  Parity unpinned beyond its parts: this file only composes functions of oracle/layers.py and
oracle/neighbour.py, each pinned by its own tests; the composition itself (order of the residual adds, which graph
and which positions feed which block) is pinned by tests/test_oracle_models.py through properties (equivariance,
zero-weight reductions), not by reference outputs, because the reference ships none.
"""
import math

import numpy as np
import torch
import torch.nn.functional as F

from . import layers as OL
from . import neighbour as ON
from . import products as OP


def _mlp(sd, prefix, dtype):
    g = lambda k: sd[f"{prefix}.layers.{k}"].to(dtype)
    return {"W1": g("0.weight"), "b1": g("0.bias"), "W2": g("2.weight"), "b2": g("2.bias"), "W3": g("4.weight"),
            "b3": g("4.bias")}


def radius_graph(pos, r0, box):
    """(src, dst, r_ij) of the reference's graph_setup (archs/meanflow_painn8.py:167-172); pos (batch, atoms, 3).
    The graph and the fp32 edge vectors come from the C oracle, as the device computes them."""
    p32 = pos.detach().to(torch.float32).numpy()
    ref = ON.edges(p32, r0, box)
    src, dst = torch.from_numpy(ref["src"]).long(), torch.from_numpy(ref["dst"]).long()
    if pos.requires_grad:
        # a gradient for the positions is wanted: the same wrap as torch arithmetic (managan/graph_layers.py:62-66)
        flat = pos.reshape(-1, 3)
        tbox = torch.tensor(box, dtype=pos.dtype)
        return src, dst, OL.boxwrap(tbox, flat[dst] - flat[src])
    r = ON.edge_vectors(p32, ref["src"], ref["dst"], box)
    return src, dst, torch.from_numpy(r).to(pos.dtype)


def block(sd, prefix, tup, r0, n, dtype):
    pos, graph, graph_bond, x_a, x_v, box = tup
    B, N = x_a.shape[:2]
    if graph is None:
        graph = radius_graph(pos, r0, box)
    if graph_bond is not None:
        bs, bd, br = graph_bond
        da, dv = OL.painn_message(bs, bd, B, N, x_a, x_v, br, _mlp(sd, f"{prefix}.message_bond.mlp_dist", dtype),
                                  _mlp(sd, f"{prefix}.message_bond.mlp_actv", dtype), r0, n)
        x_a, x_v = x_a + da, x_v + dv
    s, d, r = graph
    da, dv = OL.painn_message(s, d, B, N, x_a, x_v, r, _mlp(sd, f"{prefix}.message.mlp_dist", dtype),
                              _mlp(sd, f"{prefix}.message.mlp_actv", dtype), r0, n)
    x_a, x_v = x_a + da, x_v + dv
    w = {"W_l": sd[f"{prefix}.update.lin_l.W"].to(dtype), "W_r": sd[f"{prefix}.update.lin_r.W"].to(dtype),
         "W_v": sd[f"{prefix}.update.lin_v.W"].to(dtype), "mlp": _mlp(sd, f"{prefix}.update.mlp", dtype),
         "gn_gamma": sd[f"{prefix}.update.gn.gamma"].to(dtype), "gn_beta": sd[f"{prefix}.update.gn.beta"].to(dtype)}
    ua, uv = OL.painn_update(x_a, x_v, w, n)
    x_a, x_v = x_a + ua, x_v + uv
    if f"{prefix}.lin_push_pos.W" in sd:          # Block(pos_mutable=True): move the atoms, drop the graph
        pos = pos + OP.tensor_linear(1, sd[f"{prefix}.lin_push_pos.W"].to(dtype), x_v).squeeze(-2)
        graph = None
    return pos, graph, graph_bond, x_a, x_v, box


def cpainn(sd, prefix, blks, pos, graph_bond, x_a, x_v, box, one_hot, r0, n, dtype):
    emb = F.linear(one_hot.to(dtype), sd[f"{prefix}.atom_embed.lin.weight"].to(dtype), sd[f"{prefix}.atom_embed.lin.bias"].to(dtype))
    x_a = x_a + emb[None]
    tup = (pos, None, graph_bond, x_a, x_v, box)
    for k in range(blks):
        tup = block(sd, f"{prefix}.blocks.{k}", tup, r0, n, dtype)
    return tup[0], tup[3], tup[4]


def time_embedding(sd, prefix, st, dtype, freqs=32):
    s, t = st[0].to(dtype), st[1].to(dtype)
    ang = torch.exp(-torch.arange(freqs).to(dtype) / (freqs - 1))
    ph = torch.cat([t[:, None] * ang[None], (t - s)[:, None] * ang[None]], dim=1)
    raw = torch.cat([torch.sin(ph), torch.cos(ph)], dim=1)
    return F.linear(raw, sd[f"{prefix}.lin1.weight"].to(dtype), sd[f"{prefix}.lin1.bias"].to(dtype))


def se3ito(sd, st, x0, x1, box, one_hot, bond_src, bond_dst, r0, n, blks_0, blks_1, dtype):
    """SE3ITO.forward.  bond_src / bond_dst: the directed bonds of one system."""
    x0, x1 = x0.to(dtype), x1.to(dtype)
    B, N = x0.shape[:2]
    order = torch.argsort(bond_src, stable=True)
    offs = N * torch.arange(B)[:, None]
    bs = (bond_src[order][None] + offs).reshape(-1)
    bd = (bond_dst[order][None] + offs).reshape(-1)
    rb0 = x0.reshape(-1, 3)[bd] - x0.reshape(-1, 3)[bs]
    rb1 = x1.reshape(-1, 3)[bd] - x1.reshape(-1, 3)[bs]
    x_a = sd["atom_embeddings"].to(dtype)[None].expand(B, -1, -1)
    x_v = OP.tensor_linear(1, sd["v_readin.W"].to(dtype), (x1 - x0)[..., None, :])
    x_a = OL.mlp_silu(x_a, _mlp(sd, "mlp_embed", dtype))
    # the first stack returns its (possibly moved) positions, and PosEmbed is fed with THOSE (:212-214)
    x0_s, x_a, x_v = cpainn(sd, "cpainn_0", blks_0, x0, (bs, bd, rb0), x_a, x_v, box, one_hot, r0, n, dtype)
    x_a = OL.mlp_silu(x_a + time_embedding(sd, "t_embed", st, dtype)[:, None], _mlp(sd, "mlp_denoise", dtype))
    x_v = x_v + OP.tensor_linear(1, sd["pos_emb.lin_v.W"].to(dtype), (0.1 * (x1 - x0_s))[:, :, None])
    x1_s, x_a, x_v = cpainn(sd, "cpainn_1", blks_1, x1, (bs, bd, rb1), x_a, x_v, box, one_hot, r0, n, dtype)
    v_pred = OP.tensor_linear(1, sd["readout.W"].to(dtype), x_v).squeeze(-2)
    s, t = st[0].to(dtype), st[1].to(dtype)
    return (1. - (t - s)[:, None, None]) * v_pred + x1 - x1_s


def nodecay_cosine_schedule(t, sigma_max):
    return torch.cos(0.5 * math.pi * t) / torch.sqrt(sigma_max ** -2 + torch.sin(0.5 * math.pi * t) ** 2)


def meanflow_generate(dn, x_0, sigma_0, noise):
    """Meanflow.generate with the normal draw passed in: z_1 = x_0 + sigma_0 noise; one call at (s, t) = (0, 1)."""
    B = x_0.shape[0]
    z_1 = x_0 + sigma_0 * noise
    st = (torch.zeros(B, dtype=x_0.dtype), torch.ones(B, dtype=x_0.dtype))
    return z_1 - dn(st, x_0, z_1)


def diffusion_generate(dn, x_0, sigma_max, zeta, steps, noises):
    """The reverse-diffusion loop with its `steps + 1` normal draws passed in (noises[0] starts the chain)."""
    sigma = lambda t: nodecay_cosine_schedule(t, sigma_max)[:, None, None]
    ans = x_0 + sigma(torch.zeros(1, dtype=x_0.dtype)) * noises[0]
    for i in range(steps):
        t = torch.full((1,), i / steps, dtype=x_0.dtype)
        t_next = torch.full((1,), (i + 1) / steps, dtype=x_0.dtype)
        s_t, s_next = sigma(t), sigma(t_next)
        d_sigma = torch.sqrt(s_t ** 2 - s_next ** 2)
        eps_pred, x1_pred = dn(t, x_0, ans)
        eps_comb = (zeta * eps_pred + (ans - x1_pred)) / (zeta + s_t)
        ans = ans - (d_sigma ** 2 / s_t) * eps_comb
        ans = ans + (d_sigma * s_next / s_t) * noises[i + 1]
    return ans


def rollout(step, length, x):
    """ModelPredictor.predict: `length` frames, each fed with the last; step(frame_index, x) -> next x."""
    traj = []
    for i in range(length):
        x = step(i, x)
        traj.append(x)
    return torch.stack(traj)

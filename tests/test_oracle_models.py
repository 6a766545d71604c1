"""Properties that pin the composition in oracle/models.py (the restated SE3ITO forward of
archs/meanflow_painn8.py:185-217 and the samplers around it); its parts are pinned in tests/test_oracle_layers*.py.

  * rotating and translating both frames rotates the predicted displacement (the rotation about the centre of a box
    whose atoms stay far from the faces; the reference's fixed rotation matrix, managan/symmetries.py:54-57);
  * with positions left in place by the blocks, x1 - x1_s_pred vanishes and the output is (1 - (t - s)) readout(x_v):
    it is exactly zero at (s, t) = (0, 1), for any weights, and linear in the readout weights otherwise;
  * with pos_mutable blocks and a zero readout the output is minus the total push of the second stack, which is the
    sum of lin_push_pos over its blocks: checked against a loop written here;
  * the samplers against closed forms (a network that knows the answer)."""
import math

import numpy as np
import pytest
import torch

from conftest import load_golden
from oracle import models as OM
from oracle import products as OP

F64 = torch.float64
ROT = torch.tensor(load_golden("symmetry_checks")["rotation"], dtype=F64)       # managan/symmetries.py:54-57
Q, _ = torch.linalg.qr(ROT)
ROT = Q * torch.sign(torch.linalg.det(Q))            # exact rotation next to the printed one


def _state_dict(n, natoms, blks_0, blks_1, seed, mutate_pos=False, types=5):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s, scale=1.0: torch.randn(*s, generator=g, dtype=F64) * scale
    sd = {"atom_embeddings": rn(natoms, n), "v_readin.W": rn(n, 1), "readout.W": rn(1, n, scale=n ** -0.5),
          "pos_emb.lin_v.W": rn(n, 1), "t_embed.lin1.weight": rn(n, 128, scale=0.1), "t_embed.lin1.bias": rn(n, scale=0.1)}

    def mlp(prefix, din, dout):
        for k, (o, i) in zip((0, 2, 4), ((dout, din), (dout, dout), (dout, dout))):
            sd[f"{prefix}.layers.{k}.weight"] = rn(o, i, scale=i ** -0.5)
            sd[f"{prefix}.layers.{k}.bias"] = rn(o, scale=0.1)
    mlp("mlp_embed", n, n)
    mlp("mlp_denoise", n, n)
    for stack, blks in (("cpainn_0", blks_0), ("cpainn_1", blks_1)):
        sd[f"{stack}.atom_embed.lin.weight"] = rn(n, types, scale=0.3)
        sd[f"{stack}.atom_embed.lin.bias"] = rn(n, scale=0.1)
        for k in range(blks):
            p = f"{stack}.blocks.{k}"
            for m in ("message", "message_bond"):
                mlp(f"{p}.{m}.mlp_dist", n, 4 * n)
                mlp(f"{p}.{m}.mlp_actv", n, 4 * n)
            for lin in ("lin_l", "lin_r", "lin_v"):
                sd[f"{p}.update.{lin}.W"] = rn(n, n, scale=n ** -0.5)
            mlp(f"{p}.update.mlp", 2 * n, 3 * n)
            sd[f"{p}.update.gn.gamma"], sd[f"{p}.update.gn.beta"] = rn(n), rn(n, scale=0.1)
            if mutate_pos:
                sd[f"{p}.lin_push_pos.W"] = rn(1, n, scale=0.05 * n ** -0.5)
    return sd


def _system(B, N, box, seed):
    g = torch.Generator().manual_seed(seed)
    steps = torch.randn(B, N, 3, generator=g, dtype=F64)
    x = (1.5 * steps / steps.norm(dim=-1, keepdim=True)).cumsum(1)
    x = x - x.mean(1, keepdim=True) + 0.5 * box                          # a blob around the centre of the box
    assert float((x - 0.5 * box).abs().max()) < 0.5 * box - 6.5, "the blob must stay clear of the faces"
    one_hot = torch.nn.functional.one_hot(torch.randint(0, 5, (N,), generator=g), 5).to(F64)
    i = torch.arange(N - 1)
    return x, one_hot, torch.cat([i, i + 1]), torch.cat([i + 1, i])


def _forward(sd, st, x0, x1, box, one_hot, bs, bd, n=8, blks=(1, 2)):
    return OM.se3ito(sd, st, x0, x1, (box,) * 3, one_hot, bs, bd, 3.0, n, blks[0], blks[1], F64)


def test_se3ito_rotates_with_its_inputs_and_ignores_translations():
    box, n = 60.0, 8
    sd = _state_dict(n, 20, 1, 2, seed=1)
    x0, one_hot, bs, bd = _system(2, 20, box, seed=2)
    x1 = x0 + 0.3 * torch.randn(x0.shape, generator=torch.Generator().manual_seed(3), dtype=F64)
    st = (torch.tensor([0.1, 0.4], dtype=F64), torch.tensor([0.7, 0.9], dtype=F64))
    v = _forward(sd, st, x0, x1, box, one_hot, bs, bd)
    assert v.shape == (2, 20, 3) and float(v.abs().max()) > 1e-3
    c = torch.full((3,), 0.5 * box, dtype=F64)
    rot = lambda x: (x - c) @ ROT + c
    v_r = _forward(sd, st, rot(x0), rot(x1), box, one_hot, bs, bd)
    # the edge vectors are the fp32 quantities the device computes (5e-6 from a rotation of themselves), not float64
    assert torch.allclose(v_r, v @ ROT, atol=1e-5) and float((v_r - v).abs().max()) > 1e-2
    shift = torch.tensor([3.7, -11.2, 29.0], dtype=F64)                  # through the periodic faces too
    v_t = _forward(sd, st, x0 + shift, x1 + shift, box, one_hot, bs, bd)
    assert torch.allclose(v_t, v, atol=1e-4)      # graph and edge vectors are fp32 quantities of the shifted positions


def test_output_vanishes_at_s0_t1_when_positions_stay_in_place_and_is_linear_in_the_readout():
    box, n = 60.0, 8
    sd = _state_dict(n, 20, 1, 2, seed=4)
    x0, one_hot, bs, bd = _system(2, 20, box, seed=5)
    x1 = x0 + 0.3 * torch.randn(x0.shape, generator=torch.Generator().manual_seed(6), dtype=F64)
    ones, zeros = torch.ones(2, dtype=F64), torch.zeros(2, dtype=F64)
    assert not _forward(sd, (zeros, ones), x0, x1, box, one_hot, bs, bd).any()
    st = (torch.tensor([0.2, 0.0], dtype=F64), torch.tensor([0.5, 0.25], dtype=F64))
    v = _forward(sd, st, x0, x1, box, one_hot, bs, bd)
    v2 = _forward(dict(sd, **{"readout.W": 2.0 * sd["readout.W"]}), st, x0, x1, box, one_hot, bs, bd)
    assert torch.allclose(v2, 2.0 * v, rtol=1e-12)
    # the factor (1 - (t - s)) per system: same t - s, same output up to the time embedding (switched off here)
    quiet = dict(sd, **{"t_embed.lin1.weight": torch.zeros_like(sd["t_embed.lin1.weight"])})
    va = _forward(quiet, (zeros, torch.tensor([0.5, 0.5], dtype=F64)), x0, x1, box, one_hot, bs, bd)
    vb = _forward(quiet, (zeros, torch.tensor([0.75, 0.75], dtype=F64)), x0, x1, box, one_hot, bs, bd)
    assert torch.allclose(va / 0.5, vb / 0.25, rtol=1e-12)


def test_mutable_positions_feed_the_head():
    """pos_mutable blocks: with a zero readout the output is x1 - x1_s_pred = -(sum of the pushes of the second
    stack); the push of its LAST block is lin_push_pos of the final x_v, which the test recomputes from the x_v the
    last block returns."""
    box, n = 60.0, 8
    sd = _state_dict(n, 20, 1, 2, seed=7, mutate_pos=True)
    sd["readout.W"] = torch.zeros_like(sd["readout.W"])
    x0, one_hot, bs, bd = _system(1, 20, box, seed=8)
    x1 = x0 + 0.3 * torch.randn(x0.shape, generator=torch.Generator().manual_seed(9), dtype=F64)
    st = (torch.zeros(1, dtype=F64), torch.ones(1, dtype=F64))
    v = _forward(sd, st, x0, x1, box, one_hot, bs, bd)
    assert float(v.abs().max()) > 1e-6                                   # no longer identically zero
    # switching the last block's push off changes the output by exactly that block's push
    sd_off = dict(sd, **{"cpainn_1.blocks.1.lin_push_pos.W": torch.zeros_like(sd["cpainn_1.blocks.1.lin_push_pos.W"])})
    v_off = _forward(sd_off, st, x0, x1, box, one_hot, bs, bd)
    # ... which is linear in its weight: doubling the weight doubles the difference
    sd_dbl = dict(sd, **{"cpainn_1.blocks.1.lin_push_pos.W": 2.0 * sd["cpainn_1.blocks.1.lin_push_pos.W"]})
    v_dbl = _forward(sd_dbl, st, x0, x1, box, one_hot, bs, bd)
    assert torch.allclose(v_dbl - v_off, 2.0 * (v - v_off), rtol=1e-9, atol=1e-12)
    assert float((v - v_off).abs().max()) > 1e-6


def test_pos_embed_sees_the_positions_the_first_stack_returns():
    """archs/meanflow_painn8.py:212-214: `x0, x_a, x_v = cpainn_0(x0, ...)` rebinds x0, so PosEmbed gets the moved
    atoms.  With no block in the second stack the head reads x_v right after PosEmbed was added, and the part of the
    output that is proportional to PosEmbed's weight is (1 - (t - s)) readout(W_pe 0.1 (x1 - x0_moved)), with
    x0_moved from the first stack's block evaluated on its own."""
    box, n = 60.0, 8
    sd = _state_dict(n, 20, 1, 0, seed=11, mutate_pos=True)
    x0, one_hot, bs, bd = _system(1, 20, box, seed=12)
    x1 = x0 + 0.3 * torch.randn(x0.shape, generator=torch.Generator().manual_seed(13), dtype=F64)
    st = (torch.tensor([0.2], dtype=F64), torch.tensor([0.5], dtype=F64))
    fwd = lambda d: OM.se3ito(d, st, x0, x1, (box,) * 3, one_hot, bs, bd, 3.0, n, 1, 0, F64)
    part = fwd(sd) - fwd(dict(sd, **{"pos_emb.lin_v.W": torch.zeros_like(sd["pos_emb.lin_v.W"])}))
    # the first stack's block on its own: same inputs as SE3ITO gives it
    order = torch.argsort(bs, stable=True)
    b_s, b_d = bs[order], bd[order]
    rb0 = x0.reshape(-1, 3)[b_d] - x0.reshape(-1, 3)[b_s]
    x_a = OM.OL.mlp_silu(sd["atom_embeddings"][None], OM._mlp(sd, "mlp_embed", F64))
    x_a = x_a + torch.nn.functional.linear(one_hot, sd["cpainn_0.atom_embed.lin.weight"], sd["cpainn_0.atom_embed.lin.bias"])[None]
    x_v = OP.tensor_linear(1, sd["v_readin.W"], (x1 - x0)[..., None, :])
    x0_moved = OM.block(sd, "cpainn_0.blocks.0", (x0, None, (b_s, b_d, rb0), x_a, x_v, (box,) * 3), 3.0, n, F64)[0]
    assert float((x0_moved - x0).abs().max()) > 1e-4
    emb = OP.tensor_linear(1, sd["pos_emb.lin_v.W"], (0.1 * (x1 - x0_moved))[:, :, None])
    want = (1.0 - 0.3) * OP.tensor_linear(1, sd["readout.W"], emb).squeeze(-2)
    assert torch.allclose(part, want, rtol=1e-9, atol=1e-12)
    wrong = (1.0 - 0.3) * OP.tensor_linear(1, sd["readout.W"], OP.tensor_linear(1, sd["pos_emb.lin_v.W"], (0.1 * (x1 - x0))[:, :, None])).squeeze(-2)
    assert not torch.allclose(part, wrong, rtol=1e-4, atol=1e-7)


def test_samplers_against_closed_forms():
    target = torch.randn(2, 5, 3, generator=torch.Generator().manual_seed(1), dtype=F64)
    x_0 = torch.zeros(2, 5, 3, dtype=F64)
    sigma_max, zeta, steps = 5.0, 0.3, 12
    noises = [torch.randn(2, 5, 3, generator=torch.Generator().manual_seed(10 + k), dtype=F64) for k in range(steps + 1)]

    def dn(t, x0, noised):
        s = OM.nodecay_cosine_schedule(t, sigma_max)[:, None, None]
        return (noised - target) / s, target
    out = OM.diffusion_generate(dn, x_0, sigma_max, zeta, steps, noises)
    assert torch.allclose(out, target, atol=1e-9)             # exact predictions remove every bit of noise by t = 1
    assert abs(float(OM.nodecay_cosine_schedule(torch.tensor([0.0], dtype=F64), 20.0)) - 20.0) < 1e-12
    assert abs(float(OM.nodecay_cosine_schedule(torch.tensor([0.5], dtype=F64), 20.0))
               - math.cos(math.pi / 4) / math.sqrt(1 / 400 + 0.5)) < 1e-12
    # meanflow: z_1 = x_0 + sigma_0 noise, answer z_1 - v(z_1)
    nxt = OM.meanflow_generate(lambda st, x0, z1: 0.25 * (z1 - x0), x_0 + 1.0, 2.0, noises[0])
    assert torch.allclose(nxt, x_0 + 1.0 + 2.0 * noises[0] - 0.25 * 2.0 * noises[0])
    traj = OM.rollout(lambda k, x: x + float(k + 1), 3, torch.zeros(2, dtype=F64))
    assert traj[:, 0].tolist() == [1.0, 3.0, 6.0]

"""The PaiNN meanflow denoiser of the reference, archs/meanflow_painn8.py:127-217 (CPaiNN, PosEmbed, SE3ITO), on the
HIP blocks of painn.py.  Module and parameter names follow the reference, so `states["dn"]` of a checkpoint loads by
name, with one exception: the reference's ResidueAtomEmbed (managan/flavour_layers.py) derives its per-atom embedding
from an OpenMM topology through a submodule this build does not mirror; here `atom_embed` is a linear map of per-atom
one-hot type vectors, and the topology an OpenMMMetadata carries is passed as a `Topology` (one-hots and bond list).
"""
import torch
import torch.nn as nn

from . import differentiable as diff
from . import ops
from .denoiser import TimeEmbedding
from .graph_layers import Graph
from .painn import MLP, Block
from .tensor_products import TensLinear


class Topology:
    """What the denoiser needs to know about a system besides positions: one_hot (atoms, types) float32 and the
    directed bond list (bond_src, bond_dst) of ONE system (both directions listed, as get_bond_src_dst gives them)."""

    def __init__(self, one_hot, bond_src, bond_dst):
        self.one_hot = one_hot
        self.bond_src = bond_src
        self.bond_dst = bond_dst


def get_bond_graph(batch: int, topology: Topology, device) -> Graph:
    """managan/flavour_layers.py:256-272: bonds sorted by src, copied for every system of the batch."""
    src, dst = topology.bond_src.to(device), topology.bond_dst.to(device)
    sort_idx = torch.argsort(src, stable=True)
    src, dst = src[sort_idx], dst[sort_idx]
    atoms = int(topology.one_hot.shape[0])
    offs = atoms * torch.arange(batch, device=device)[:, None]
    return Graph((src[None] + offs).reshape(-1), (dst[None] + offs).reshape(-1), None, batch, atoms)


class OneHotAtomEmbed(nn.Module):
    """Stands in for ResidueAtomEmbed(n): (atoms, types) one-hots -> (atoms, n)."""

    def __init__(self, n, atom_types=20):
        super().__init__()
        self.lin = nn.Linear(atom_types, n)

    def forward(self, topology: Topology):
        if diff.wants_grad(self):
            return diff.linear(self.lin, topology.one_hot)
        return ops.tensor_linear_fwd(0, self.lin.weight, topology.one_hot.contiguous(), bias=self.lin.bias)


class CPaiNN(nn.Module):
    """archs/meanflow_painn8.py:127-143"""

    def __init__(self, r0: float, n: int, blks: int, mutate_pos: bool = False, atom_types: int = 20):
        super().__init__()
        self.atom_embed = OneHotAtomEmbed(n, atom_types)
        self.blocks = nn.Sequential(*[Block(r0, n, pos_mutable=mutate_pos) for _ in range(blks)])

    def forward(self, pos, graph_bond, r_ij_bond, x_a, x_v, box, topology):
        x_a = diff.add(x_a, self.atom_embed(topology)[None])
        pos, _, _, _, _, x_a, x_v, _ = self.blocks((pos, None, None, graph_bond, r_ij_bond, x_a, x_v, box))
        return pos, x_a, x_v


class PosEmbed(nn.Module):
    """archs/meanflow_painn8.py:174-183"""

    def __init__(self, dim_v):
        super().__init__()
        self.lin_v = TensLinear(1, 1, dim_v)

    def forward(self, pos_0, pos_1):
        return self.lin_v(diff.mul(diff.sub(pos_1, pos_0), 0.1)[:, :, None].contiguous())


class SE3ITO(nn.Module):
    """archs/meanflow_painn8.py:185-217"""

    def __init__(self, r0: float, n: int, natoms: int, blks_0: int = 2, blks_1: int = 5, atom_types: int = 20,
                 mutate_pos: bool = False):
        """mutate_pos: build the blocks with pos_mutable=True (archs/meanflow_painn8.py:102-125; the reference's SE3ITO
        leaves it off, in which case x1 - x1_s_pred vanishes and the output at (s, t) = (0, 1) is identically zero)."""
        super().__init__()
        self.r0 = r0
        self.atom_embeddings = nn.Parameter(torch.randn(natoms, n))
        self.t_embed = TimeEmbedding(32, n)
        self.mlp_embed = MLP(n, n)
        self.mlp_denoise = MLP(n, n)
        self.pos_emb = PosEmbed(n)
        self.cpainn_0 = CPaiNN(r0, n, blks_0, mutate_pos=mutate_pos, atom_types=atom_types)
        self.cpainn_1 = CPaiNN(r0, n, blks_1, mutate_pos=mutate_pos, atom_types=atom_types)
        self.v_readin = TensLinear(1, 1, n)
        self.readout = TensLinear(1, n, 1)

    def get_v_pred(self, st, v_pred, x1_s_pred, x1_t):
        s, t = st
        span = diff.sub(1., diff.sub(t, s)[:, None, None])
        return diff.sub(diff.add(diff.mul(span, v_pred), x1_t), x1_s_pred)

    def forward(self, st, x0, x1, box, topology: Topology):
        """st: ((batch), (batch)); x0, x1: (batch, atoms, 3)."""
        x0, x1 = x0.contiguous(), x1.contiguous()
        x1_t = x1
        batch = x0.shape[0]
        graph_bond = get_bond_graph(batch, topology, x0.device)
        # bond vectors are plain differences: bonded atoms are never a box apart (archs/meanflow_painn8.py:208-209)
        r_ij_bond_0 = (x0.reshape(-1, 3)[graph_bond.dst] - x0.reshape(-1, 3)[graph_bond.src]).contiguous()
        r_ij_bond_1 = (x1.reshape(-1, 3)[graph_bond.dst] - x1.reshape(-1, 3)[graph_bond.src]).contiguous()
        x_a = self.atom_embeddings[None].expand(batch, -1, -1)
        x_v = self.v_readin(diff.sub(x1, x0)[..., None, :].contiguous())
        x_a = self.mlp_embed(x_a.contiguous())
        x0, x_a, x_v = self.cpainn_0(x0, graph_bond, r_ij_bond_0, x_a, x_v, box, topology)
        x_a = self.mlp_denoise(diff.add(x_a, self.t_embed(st)[:, None]))
        x_v = diff.add(x_v, self.pos_emb(x0, x1))
        x1, x_a, x_v = self.cpainn_1(x1, graph_bond, r_ij_bond_1, x_a, x_v, box, topology)
        return self.get_v_pred(st, self.readout(x_v).squeeze(-2), x1, x1_t)

"""The caller of the native chain simulation: `CUDASim` and its two registered configurations
(managan/sims.py:233-292), on top of `ops.repel5_sim`.  Same call pattern; a `seed` makes runs reproducible
(the reference reseeds from the wall clock on every integrator call)."""
import time

import torch

from . import ops


class ChainSim:
    """CUDASim (managan/sims.py:234-283) for the REPEL5 force field."""

    def __init__(self, drag, T, l, delta_t, t_res, metadata=None, seed=None, device="cuda"):
        self.drag = drag.to(device=device, dtype=torch.float32).contiguous()
        self.T, self.l, self.delta_t, self.t_res = T, l, delta_t, t_res
        self.dt = delta_t / t_res
        self.shape = (l, 3)
        self.device = device
        self.seed = time.time_ns() if seed is None else int(seed)
        self._kick = 0                      # velocity updates drawn so far: consecutive calls continue one stream
        if metadata is not None:
            for key in metadata:
                setattr(self, key, metadata[key])

    def _integrate(self, x, v, drag, T, steps):
        steps = int(steps)
        kicks = max(steps, 1) + 1
        if self._kick + kicks >= 1 << 32:   # the kick index is 32 bits wide: move on to the next key
            self.seed, self._kick = self.seed + 1, 0
        ops.repel5_sim(x, v, drag, T, self.dt, steps, self.seed, self._kick)
        self._kick += kicks

    def generate_trajectory(self, x, v, time, ret=True):
        """x, v (batch, l, 3) are overwritten; returns (batch, time, l, 3) when ret."""
        batch = x.shape[0]
        if tuple(x.shape) != (batch, self.l, 3) or tuple(v.shape) != (batch, self.l, 3):
            raise RuntimeError(f"x and v must have shape (batch, {self.l}, 3)")
        ans = torch.zeros((batch, time, *self.shape), device=x.device) if ret else None
        for i in range(time):
            self._integrate(x, v, self.drag, self.T, self.t_res)
            if ret:
                ans[:, i] = x
        return ans

    def sample_equilibrium(self, batch, iterations, t_noise=None, t_ballistic=None, drag_const=20.):
        """Alternate high-drag and drag-free stretches, then one regular interval (managan/sims.py:264-283)."""
        t_noise = self.delta_t if t_noise is None else t_noise
        t_ballistic = self.delta_t if t_ballistic is None else t_ballistic
        high_drag = self.drag + drag_const
        zero_drag = torch.zeros_like(self.drag)
        gen = torch.Generator(device="cpu").manual_seed(self.seed & 0x7FFFFFFFFFFFFFFF)
        x = torch.randn(batch, *self.shape, generator=gen).to(self.device)
        v = torch.zeros(batch, *self.shape, device=self.device)
        for _ in range(iterations):
            self._integrate(x, v, high_drag, self.T, int(t_noise / self.dt))
            self._integrate(x, v, zero_drag, self.T, int(t_ballistic / self.dt))
        self._integrate(x, v, self.drag, self.T, self.t_res)
        return x, v


def repel5(l, t, seed=None):
    """"repel5_l%d_t%d" (managan/sims.py:284-287)."""
    return ChainSim(torch.tensor([1.] * l), 1.0, l, float(t), 100 * t, {"poly_len": l, "space_dim": 3}, seed)


def repel5a(l, t, seed=None):
    """"repel5a_l%d_t%d" (managan/sims.py:288-291)."""
    return ChainSim(torch.tensor([1.] * l), 1.0, l, float(t), 200 * t, {"poly_len": l, "space_dim": 3}, seed)

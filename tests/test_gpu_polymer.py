"""The bead-chain Langevin generator (mg_repel5_sim behind `polymer_sims_cuda.polymer_sim`) against the CPU
restatement oracle/polymer.py on the same inputs and the same counter-based normals."""
import importlib

import numpy as np
import pytest
import torch

from oracle import polymer as OPY

pytestmark = pytest.mark.gpu


def _chains(batch, n, seed):
    rng = np.random.default_rng(seed)
    steps = rng.normal(size=(batch, n, 3))
    steps *= 0.8 / np.linalg.norm(steps, axis=-1, keepdims=True)
    x = np.cumsum(steps, axis=1) + rng.normal(size=(batch, n, 3)) * 0.02
    v = rng.normal(size=(batch, n, 3)) * 0.5
    drag = rng.uniform(0.2, 2.0, size=n)
    return x.astype(np.float32), v.astype(np.float32), drag.astype(np.float32)


@pytest.fixture(scope="module")
def sim(pkg):
    pkg.install_shims()
    return importlib.import_module("polymer_sims_cuda")


@pytest.mark.parametrize("n,nsteps,T", [(1, 5, 0.0), (2, 5, 1.0), (3, 7, 0.0), (5, 1, 1.0), (5, 0, 1.0), (64, 20, 0.0),
                                        (64, 20, 1.0), (200, 12, 1.0), (300, 6, 0.5), (1500, 3, 1.0), (2048, 2, 0.0)])
def test_trajectory_matches_the_oracle(sim, n, nsteps, T):
    """Tolerance rel 1e-4 / abs 2e-5 on positions and velocities after up to 20 steps: both sides run fp32 with the
    force sum in the same order; the oracle divides and takes the bond factor in double as the reference does, the
    kernel in float, and the kernel's logf / cosf differ from numpy's by a few units in the last place."""
    batch, dt, seed, first_kick = 3, 0.004, 0xfeedbeef12345, 11
    x0, v0, drag = _chains(batch, n, n + nsteps)
    x, v = torch.from_numpy(x0).cuda(), torch.from_numpy(v0).cuda()
    sim.polymer_sim(sim.SimId.REPEL5, x, v, torch.from_numpy(drag).cuda(), T, dt, nsteps, seed=seed, first_kick=first_kick)
    normals = OPY.philox_normals(seed, batch, n, first_kick, max(nsteps, 1) + 1)
    xr, vr = OPY.repel5_sim(x0, v0, drag, T, dt, nsteps, normals)
    np.testing.assert_allclose(x.cpu().numpy(), xr, rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(v.cpu().numpy(), vr, rtol=1e-4, atol=1e-4 * float(np.abs(vr).max()))
    if T > 0:                                                # and the noise did act
        xz, vz = OPY.repel5_sim(x0, v0, drag, 0.0, dt, nsteps, normals)
        assert float(np.abs(vz - vr).max()) > 1e-3


def test_stream_is_a_function_of_seed_and_kick_only(sim):
    x0, v0, drag = _chains(4, 33, 1)
    d = torch.from_numpy(drag).cuda()

    def run(seed, first_kick):
        x, v = torch.from_numpy(x0).cuda(), torch.from_numpy(v0).cuda()
        sim.polymer_sim(sim.SimId.REPEL5, x, v, d, 1.0, 0.01, 10, seed=seed, first_kick=first_kick)
        return x, v

    a, b, c, e = run(5, 0), run(5, 0), run(6, 0), run(5, 1)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert not torch.equal(a[1], c[1]) and not torch.equal(a[1], e[1])
    # without a seed every call draws a new one, as the reference does from the wall clock
    x1, v1 = torch.from_numpy(x0).cuda(), torch.from_numpy(v0).cuda()
    x2, v2 = torch.from_numpy(x0).cuda(), torch.from_numpy(v0).cuda()
    sim.polymer_sim(sim.SimId.REPEL5, x1, v1, d, 1.0, 0.01, 10)
    sim.polymer_sim(sim.SimId.REPEL5, x2, v2, d, 1.0, 0.01, 10)
    assert not torch.equal(v1, v2)


def test_free_beads_reach_the_temperature(sim):
    """n = 1 chains feel no force: the scheme is an Ornstein-Uhlenbeck recursion v <- v (1 - g dt) + sqrt(2 g T dt) xi
    whose stationary variance is T / (1 - g dt / 2).  16384 x 3 samples: standard error of the variance 0.64 %."""
    g, T, dt = 1.0, 1.5, 0.01
    batch = 16384
    x = torch.zeros(batch, 1, 3, device="cuda")
    v = torch.zeros(batch, 1, 3, device="cuda")
    sim.polymer_sim(sim.SimId.REPEL5, x, v, torch.full((1,), g, device="cuda"), T, dt, 1500, seed=99)
    var = float(v.double().pow(2).mean())
    assert abs(var / (T / (1 - 0.5 * g * dt)) - 1) < 0.03
    assert abs(float(v.double().mean())) < 0.03
    # positions diffuse: <x^2> = 2 (T / g) t for t >> 1 / g, here t = 15 (ballistic correction -2 T / g^2 (1 - e^-gt))
    msd = float(x.double().pow(2).mean())
    want = 2 * T / g * 15.0 - 2 * T / g ** 2 * (1 - np.exp(-g * 15.0))
    assert abs(msd / want - 1) < 0.05


def test_argument_checks(sim):
    x, v, d = torch.zeros(2, 4, 3, device="cuda"), torch.zeros(2, 4, 3, device="cuda"), torch.ones(4, device="cuda")
    with pytest.raises(RuntimeError, match="Batch sizes must match"):
        sim.polymer_sim(sim.SimId.REPEL5, x, torch.zeros(3, 4, 3, device="cuda"), d, 1.0, 0.01, 1)
    with pytest.raises(RuntimeError, match="Number of particles must match"):
        sim.polymer_sim(sim.SimId.REPEL5, x, v, torch.ones(5, device="cuda"), 1.0, 0.01, 1)
    with pytest.raises(RuntimeError, match="Position and velocity must be 3D"):
        sim.polymer_sim(sim.SimId.REPEL5, torch.zeros(2, 4, 2, device="cuda"), torch.zeros(2, 4, 2, device="cuda"), d, 1.0, 0.01, 1)
    with pytest.raises(RuntimeError, match="correct dimensions"):
        sim.polymer_sim(sim.SimId.REPEL5, x[0], v[0], d, 1.0, 0.01, 1)
    with pytest.raises(RuntimeError, match="contiguous"):
        sim.polymer_sim(sim.SimId.REPEL5, x.transpose(0, 1), v, d, 1.0, 0.01, 1)
    with pytest.raises(RuntimeError, match="CUDA"):
        sim.polymer_sim(sim.SimId.REPEL5, x.cpu(), v, d, 1.0, 0.01, 1)
    with pytest.raises(RuntimeError, match="at most 2048 beads"):
        sim.polymer_sim(sim.SimId.REPEL5, torch.zeros(1, 2049, 3, device="cuda"), torch.zeros(1, 2049, 3, device="cuda"),
                        torch.ones(2049, device="cuda"), 1.0, 0.01, 1)
    with pytest.raises(RuntimeError, match="unrecognized simulation id"):
        sim.polymer_sim(7, x, v, d, 1.0, 0.01, 1)
    e = torch.zeros(0, 4, 3, device="cuda")
    sim.polymer_sim(sim.SimId.REPEL5, e, e.clone(), d, 1.0, 0.01, 3)          # no chains: nothing to do


def test_chain_sim_caller(pkg):
    """generate_trajectory / sample_equilibrium as managan/sims.py:247-283 calls the integrator: consecutive calls
    continue one noise stream, so the whole trajectory is a function of the seed."""
    sims = importlib.import_module("learned-dynamics_amd.sims")
    a, b = sims.repel5(24, 1, seed=3), sims.repel5(24, 1, seed=3)
    assert a.t_res == 100 and abs(a.dt - 0.01) < 1e-12 and a.poly_len == 24 and a.shape == (24, 3)
    xa, va = a.sample_equilibrium(8, 2)
    xb, vb = b.sample_equilibrium(8, 2)
    assert torch.equal(xa, xb) and torch.equal(va, vb) and bool(torch.isfinite(xa).all())
    ta = a.generate_trajectory(xa, va, 3)
    tb = b.generate_trajectory(xb, vb, 3)
    assert ta.shape == (8, 3, 24, 3) and torch.equal(ta, tb) and torch.equal(ta[:, -1], xa)
    assert not torch.equal(ta[:, 0], ta[:, 1])
    bonds = (ta[:, -1, 1:] - ta[:, -1, :-1]).norm(dim=-1)
    assert 0.5 < float(bonds.mean()) < 1.1                   # bonded neighbours stay near r0 = 0.8

"""Pins the CPU restatement of the bead-chain Langevin generator (oracle/polymer.py) without the reference:
forces against a numerical energy gradient, the integrator against closed forms and energy conservation, the
noise generator against published known-answer vectors.  CPU only."""
import numpy as np
import pytest

from conftest import load_golden
from oracle import polymer as OPY


def test_forces_are_the_negative_gradient_of_the_pair_energy():
    """A wrong sign, a missing bond, a wrong exclusion (the reference excludes i-1, i, i+1 CYCLICALLY from the
    repulsion, so beads 0 and n-1 do not repel) or a wrong power each fail this."""
    rng = np.random.default_rng(0)
    for n in (1, 2, 3, 4, 7, 12):
        x = rng.normal(size=(2, n, 3)) * 1.2
        f = OPY.repel5_forces(x, dtype=np.float64)
        num = np.zeros_like(x)
        h = 1e-6
        for i in range(n):
            for c in range(3):
                xp, xm = x.copy(), x.copy()
                xp[:, i, c] += h
                xm[:, i, c] -= h
                num[:, i, c] = -(OPY.repel5_energy(xp) - OPY.repel5_energy(xm)) / (2 * h)
        np.testing.assert_allclose(f, num, rtol=2e-6, atol=2e-6)
    # float32 path agrees with the float64 one
    x = rng.normal(size=(3, 20, 3))
    np.testing.assert_allclose(OPY.repel5_forces(x), OPY.repel5_forces(x, np.float64), rtol=2e-5, atol=2e-5)


def test_first_and_last_bead_do_not_repel():
    x = np.zeros((1, 5, 3))
    x[0, :, 0] = [0.0, 0.8, 1.6, 2.4, 0.1]                  # bead 4 sits almost on bead 0
    f = OPY.repel5_forces(x, np.float64)
    x2 = x.copy()
    x2[0, 0, 1] = 50.0                                       # move bead 0 far away sideways
    f2 = OPY.repel5_forces(x2, np.float64)
    # the force on bead 4 from bead 0 is absent in both: only beads 1, 2 (repulsion) and 3 (bond) act on it
    np.testing.assert_allclose(f[0, 4], f2[0, 4], rtol=1e-12)


@pytest.mark.parametrize("nsteps", [0, 1, 2, 9])
def test_single_bead_without_noise_follows_the_closed_form(nsteps):
    """n = 1: no forces.  Half kick v(1 - g dt/2), then max(nsteps, 1) drifts with full kicks v(1 - g dt) between,
    then the last half kick."""
    g, dt, v0, x0 = 0.7, 0.05, np.array([1.0, -2.0, 0.5]), np.array([0.1, 0.2, 0.3])
    drifts = max(nsteps, 1)
    x, v = OPY.repel5_sim(x0[None, None], v0[None, None], [g], 0.0, dt, nsteps, np.zeros((drifts + 1, 1, 1, 3)), np.float64)
    vh = v0 * (1 - 0.5 * g * dt)
    xs = x0 + dt * vh * sum((1 - g * dt) ** s for s in range(drifts))
    vs = vh * (1 - g * dt) ** (drifts - 1) * (1 - 0.5 * g * dt)
    np.testing.assert_allclose(x[0, 0], xs, rtol=1e-13)
    np.testing.assert_allclose(v[0, 0], vs, rtol=1e-13)


def test_noise_enters_each_kick_with_its_weight():
    """Single bead, zero drag would zero the noise (noise = sqrt(2 g T dt)), so keep drag and check linearity in the
    normals: v(normals) - v(0) = noise * (sqrt(.5)/2 g_first decayed + sum g_mid decayed + sqrt(.5)/2 g_last)."""
    g, T, dt, nsteps = 0.3, 1.7, 0.02, 4
    rng = np.random.default_rng(1)
    normals = rng.normal(size=(nsteps + 1, 1, 1, 3))
    z = np.zeros((1, 1, 3))
    _, v1 = OPY.repel5_sim(z, z, [g], T, dt, nsteps, normals, np.float64)
    noise = np.sqrt(2 * g * T * dt)
    a, h = 1 - g * dt, 1 - 0.5 * g * dt
    want = 0.5 * np.sqrt(0.5) * noise * normals[0] * a ** (nsteps - 1) * h
    for s in range(1, nsteps):
        want = want + noise * normals[s] * a ** (nsteps - 1 - s) * h
    want = want + 0.5 * np.sqrt(0.5) * noise * normals[nsteps]
    np.testing.assert_allclose(v1, want, rtol=1e-12)


def test_energy_is_conserved_without_drag_and_time_reverses():
    rng = np.random.default_rng(2)
    n = 8
    x0 = np.zeros((1, n, 3))
    x0[0, :, 0] = 0.9 * np.arange(n)                        # a stretched, slightly kinked chain: moderate forces
    x0 += rng.normal(size=(1, n, 3)) * 0.05
    v0 = rng.normal(size=(1, n, 3)) * 0.3
    drag = np.zeros(n)
    e0 = OPY.repel5_energy(x0) + 0.5 * np.sum(v0 ** 2)
    errs = []
    for dt, steps in ((2e-3, 200), (1e-3, 400)):
        x, v = OPY.repel5_sim(x0, v0, drag, 0.0, dt, steps, np.zeros((steps + 1, 1, n, 3)), np.float64)
        errs.append(abs(float((OPY.repel5_energy(x) + 0.5 * np.sum(v ** 2) - e0)[0])))
    assert errs[0] < 1e-3 * abs(float(e0[0])) and errs[1] < 0.35 * errs[0] + 1e-12        # second order in dt
    xb, vb = OPY.repel5_sim(x, -v, drag, 0.0, 1e-3, 400, np.zeros((401, 1, n, 3)), np.float64)
    np.testing.assert_allclose(xb, x0, atol=1e-9)
    np.testing.assert_allclose(-vb, v0, atol=1e-9)


def test_philox_known_answers():
    """Known-answer vectors of Philox4x32-10 from the reference implementation of Salmon et al. (Random123
    kat_vectors: counter, key -> output)."""
    kat = [tuple(tuple(int(w, 16) for w in v[k]) for k in ("counter", "key", "output"))
           for v in load_golden("philox4x32_10")["vectors"]]
    assert len(kat) == 3
    for counter, key, want in kat:
        got = OPY.philox4x32_10(np.array(counter, dtype=np.uint32), np.array(key, dtype=np.uint32))
        assert tuple(int(g) for g in got) == want


def test_normals_have_unit_moments_and_depend_on_every_index():
    g = OPY.philox_normals(0x1234567_89abcdef, batch=16, n=64, first_kick=5, kicks=40).astype(np.float64)
    flat = g.reshape(-1)
    assert abs(flat.mean()) < 5e-3 and abs(flat.var() - 1) < 1e-2 and abs((flat ** 4).mean() - 3) < 5e-2
    # components, beads and kicks are uncorrelated
    assert abs(np.mean(g[..., 0] * g[..., 1])) < 1e-2 and abs(np.mean(g[..., 0] * g[..., 2])) < 1e-2
    assert abs(np.mean(g[:, :, 1:] * g[:, :, :-1])) < 1e-2 and abs(np.mean(g[1:] * g[:-1])) < 1e-2
    # a shifted first_kick shifts the stream; another seed gives another one
    g2 = OPY.philox_normals(0x1234567_89abcdef, batch=16, n=64, first_kick=6, kicks=3)
    np.testing.assert_array_equal(g2, OPY.philox_normals(0x1234567_89abcdef, 16, 64, 5, 4)[1:])
    assert not np.array_equal(OPY.philox_normals(1, 2, 8, 0, 1), OPY.philox_normals(1 << 32, 2, 8, 0, 1))

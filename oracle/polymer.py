"""TEST INFRASTRUCTURE ONLY — CPU restatement (numpy) of the bead-chain Langevin generator `repel5_sim`.

Follows (relative to the reference checkout):
  extensions/polymer_sims_cuda/polymer_sims_kern.cu:5-8      constants (REPEL_SCALE, K, R0, LJ_EPSILON)
  extensions/polymer_sims_cuda/polymer_sims_kern.cu:72-81    bond_force, repel_force
  extensions/polymer_sims_cuda/polymer_sims_kern.cu:83-104   repel5_ff: bonds to i-1 and i+1, then k = (i + j - 1) % n, j = 3..n-1
  extensions/polymer_sims_cuda/polymer_sims_kern.cu:106-142  repel5_sim_kern: half kick, (nsteps - 1) x [drift, kick], drift, half kick

The reference draws its noise from XORWOW states seeded from the wall clock (polymer_sims.cpp:39), so no run of it
is reproducible and its stream is not part of the contract.  The integrator here takes the normals as an argument;
`philox_normals` restates the counter-based stream the HIP kernel uses (Philox4x32-10, Salmon et al., "Parallel
random numbers: as easy as 1, 2, 3", SC'11; checked against the known-answer vectors of its reference
implementation in tests/test_oracle_polymer.py) followed by Box-Muller.

How it is pinned (tests/test_oracle_polymer.py): forces against the numerical gradient of an independently written
pair energy; the force-free integrator against its closed form; energy conservation at zero drag; Philox against
the published known-answer vectors; moments of the normals.
"""
import numpy as np

REPEL_SCALE, BOND_K, BOND_R0, LJ_EPSILON = 20.0, 20.0, 0.8, 0.2


def repel5_forces(x, dtype=np.float32):
    """x (batch, n, 3) -> forces (batch, n, 3), summed per bead in the reference's order."""
    x = np.asarray(x, dtype=dtype)
    B, n, _ = x.shape
    f = np.zeros_like(x)

    def bond(d):
        # the reference evaluates `1 - R0/sqrt(...)` and `-K*factor` in double (R0 and K are double literals) and
        # rounds when the factor meets the float3
        r = np.sqrt(np.sum(d * d, axis=-1, dtype=dtype), dtype=dtype)
        factor = (1.0 - BOND_R0 / r.astype(np.float64)).astype(dtype)
        return ((-BOND_K * factor.astype(np.float64)).astype(dtype))[..., None] * d

    if n > 1:
        f[:, 1:] += bond(x[:, 1:] - x[:, :-1])
        f[:, :-1] += bond(x[:, :-1] - x[:, 1:])
    idx = np.arange(n)
    for j in range(3, n):
        k = (idx + j - 1) % n
        d = x - x[:, k]
        q = (np.sum(d * d, axis=-1, dtype=dtype) + dtype(LJ_EPSILON)).astype(dtype)
        q2 = q * q
        p6 = q2 * (q2 * q2)
        factor = (REPEL_SCALE / p6.astype(np.float64)).astype(dtype)
        f += factor[..., None] * d
    return f


def repel5_energy(x):
    """Potential whose negative gradient repel5_forces is, written pair by pair in float64 (for pinning only):
    bonds K/2 (|d| - R0)^2 between chain neighbours, 2 (|d|^2 + eps)^-5 between every pair of beads that are
    neither equal nor cyclic neighbours."""
    x = np.asarray(x, dtype=np.float64)
    B, n, _ = x.shape
    e = np.zeros(B)
    for i in range(n):
        for k in range(i + 1, n):
            d = np.linalg.norm(x[:, i] - x[:, k], axis=-1)
            if k == i + 1:
                e += 0.5 * BOND_K * (d - BOND_R0) ** 2
            if (k - i) % n not in (0, 1, n - 1):
                e += (REPEL_SCALE / 10.0) * (d * d + LJ_EPSILON) ** -5
    return e


def repel5_sim(x, v, drag, T, dt, nsteps, normals, dtype=np.float32):
    """Returns (x, v) after the reference's integrator.  normals: (max(nsteps, 1) + 1, batch, n, 3), one set per
    velocity update in the order they happen."""
    x, v = np.array(x, dtype=dtype), np.array(v, dtype=dtype)
    drag = np.asarray(drag, dtype=dtype)[None, :, None]
    dt = dtype(dt)
    noise = np.sqrt(dtype(2) * drag * dtype(T) * dt, dtype=dtype)
    normals = np.asarray(normals, dtype=dtype)
    drifts = max(int(nsteps), 1)
    assert normals.shape[0] == drifts + 1
    half = dtype(np.sqrt(0.5))

    def kick(g, w, c):
        a = repel5_forces(x, dtype)
        return (v + dtype(w) * (dt * (a - drag * v) + (dtype(c) * noise) * g)).astype(dtype)

    v = kick(normals[0], 0.5, half)
    for s in range(1, drifts):
        x = (x + dt * v).astype(dtype)
        v = kick(normals[s], 1.0, 1.0)
    x = (x + dt * v).astype(dtype)
    v = kick(normals[drifts], 0.5, half)
    return x, v


# ------------------------------------------------------------------ the kernel's noise stream
def philox4x32_10(counter, key):
    """counter (..., 4) uint32, key (..., 2) uint32 -> (..., 4) uint32."""
    c = np.array(np.broadcast_arrays(*[np.asarray(counter, dtype=np.uint32)[..., i] for i in range(4)]), dtype=np.uint64)
    k0 = np.asarray(key, dtype=np.uint32)[..., 0].astype(np.uint64)
    k1 = np.asarray(key, dtype=np.uint32)[..., 1].astype(np.uint64)
    m32 = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c[0]
        p1 = np.uint64(0xCD9E8D57) * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & m32
        hi1, lo1 = p1 >> np.uint64(32), p1 & m32
        c = np.array([hi1 ^ c[1] ^ k0, lo1, hi0 ^ c[3] ^ k1, lo0], dtype=np.uint64)
        k0 = (k0 + np.uint64(0x9E3779B9)) & m32
        k1 = (k1 + np.uint64(0xBB67AE85)) & m32
    return np.stack([c[i] for i in range(4)], axis=-1).astype(np.uint32)


def philox_normals(seed, batch, n, first_kick, kicks):
    """(kicks, batch, n, 3) float32: normals of bead b = chain * n + i at kick first_kick + s from
    Philox(counter = (b, kick, 0, 0), key = (seed low word, seed high word)): with u = ((r >> 8) + 0.5) 2^-24,
    (sqrt(-2 ln u0) cos(2 pi u1), sqrt(-2 ln u0) sin(2 pi u1), sqrt(-2 ln u2) cos(2 pi u3))."""
    bead = np.arange(batch * n, dtype=np.uint32)
    kick = (np.uint64(first_kick) + np.arange(kicks, dtype=np.uint64)).astype(np.uint32)
    counter = np.zeros((kicks, batch * n, 4), dtype=np.uint32)
    counter[..., 0] = bead[None, :]
    counter[..., 1] = kick[:, None]
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint32)
    r = philox4x32_10(counter, key)
    u = ((r >> np.uint32(8)).astype(np.float32) + np.float32(0.5)) * np.float32(2.0 ** -24)
    two_pi = np.float32(6.28318530717958647692)
    r0 = np.sqrt(np.float32(-2) * np.log(u[..., 0]), dtype=np.float32)
    r1 = np.sqrt(np.float32(-2) * np.log(u[..., 2]), dtype=np.float32)
    a0, a1 = two_pi * u[..., 1], two_pi * u[..., 3]
    g = np.stack([r0 * np.cos(a0), r0 * np.sin(a0), r1 * np.cos(a1)], axis=-1).astype(np.float32)
    return g.reshape(kicks, batch, n, 3)

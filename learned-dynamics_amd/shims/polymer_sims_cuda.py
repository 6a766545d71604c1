"""Drop-in for the reference's `polymer_sims_cuda` extension (extensions/polymer_sims_cuda/polymer_sims.cpp:49-54):
`polymer_sim(SimId.REPEL5, x, v, drag, T, dt, nsteps)` integrates the chains in place.  Like the reference, every
call takes a fresh seed from the wall clock; pass `seed=` (and `first_kick=` to continue a stream) for a
reproducible run."""
import enum
import importlib
import time

_ops = importlib.import_module("learned-dynamics_amd.ops")


class SimId(enum.Enum):
    REPEL5 = 0


def polymer_sim(sim_id, x, v, drag, T, dt, nsteps, seed=None, first_kick=0):
    if sim_id is not SimId.REPEL5:
        raise RuntimeError("unrecognized simulation id!")
    if seed is None:
        seed = time.time_ns()
    _ops.repel5_sim(x, v, drag, T, dt, nsteps, seed, first_kick)

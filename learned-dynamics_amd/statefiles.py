"""On-disk formats of the reference, so that its trajectories and trained weights can be fed to this path.

Dataset chunk (managan/statefiles.py:16-42): three lengths as big-endian uint32 (`!III`), then three sub-files of
those lengths: the pickled metadata, the pickled per-item shape, and the trajectory as an `.npy` payload written
without pickling.  Checkpoint (managan/config.py:125-137): a `torch.save`d dict with "args", "kwargs" (the model's
configuration) and "states" (for the denoisers `{"dn": state_dict}`, archs/diffuser_atoms15.py:493-496,
archs/meanflow_painn8.py:252-255).  The mirrored modules keep the reference's attribute names, so a sub-tree of such
a state dict loads into them by name.

Nothing here executes code from a file: the two pickles are decoded by an unpickler that builds plain containers,
numbers, strings and bytes only and turns every other object into an inert `OpaqueObject` record; checkpoints are
read with `torch.load(weights_only=True)`.
"""
import io
import os
import pickle
import random
import struct
from dataclasses import dataclass, field
from typing import Any, Optional, Tuple

import numpy as np
import torch

_HEADER = struct.Struct("!III")


class DatasetError(Exception):
    """A chunk file that does not follow the format (managan/statefiles.py:13-14)."""


class OpaqueObject:
    """What a pickled instance of a class (or the result of a pickled function call) becomes when read here: a
    record of its class path (`module`, `name`), the arguments, state and items the pickle carried for it; never
    an instance of that class, and nothing of it is imported."""
    module = name = ""

    def __new__(cls, *args, **kwargs):
        obj = object.__new__(cls)
        obj.args, obj.kwargs, obj.state, obj.items = args, kwargs, None, []
        return obj

    def __init__(self, *args, **kwargs):
        pass

    def __setstate__(self, state):                # BUILD
        self.state = state

    def __setitem__(self, key, value):            # SETITEM(S) on dict-like classes
        self.items.append((key, value))

    def append(self, value):                      # APPEND on list-like classes
        self.items.append(value)

    def extend(self, values):                     # APPENDS
        self.items.extend(values)

    def __repr__(self):
        return f"<opaque {self.module}.{self.name} args={self.args!r} state={self.state!r} items={self.items!r}>"


class _InertUnpickler(pickle.Unpickler):
    """Plain containers and scalars decode as themselves (the pickle machine builds them without a lookup);
    every global a pickle names resolves to a fresh subclass of OpaqueObject instead of being imported."""

    def find_class(self, module, name):
        return type(str(name), (OpaqueObject,), {"module": str(module), "name": str(name)})

    def persistent_load(self, pid):
        raise DatasetError("persistent ids are not part of the chunk format")


def _inert_loads(data: bytes):
    try:
        return _InertUnpickler(io.BytesIO(data)).load()
    except DatasetError:
        raise
    except Exception as e:
        raise DatasetError(f"undecodable pickle in chunk file: {e}") from e


@dataclass
class TrajectoryState:
    """What `ModelState` (managan/predictor.py:132-156) holds: the per-item shape, the tensor `x` of shape
    size + shape, and the metadata."""
    shape: Tuple[int, ...]
    x: torch.Tensor
    metadata: Any = None
    size: Tuple[int, ...] = field(init=False)

    def __post_init__(self):
        self.shape = tuple(int(s) for s in self.shape)
        nd = len(self.shape)
        if self.x.dim() < nd or tuple(self.x.shape[self.x.dim() - nd:]) != self.shape:
            raise DatasetError(f"tensor of shape {tuple(self.x.shape)} does not end in the item shape {self.shape}")
        self.size = tuple(self.x.shape[:self.x.dim() - nd])

    def __getitem__(self, key):
        return TrajectoryState(self.shape, self.x[key], self.metadata)


def save_state_to_file(file, state: TrajectoryState):
    """Write one chunk (managan/statefiles.py:16-30).  Metadata must be plain data (dicts, lists, tuples, numbers,
    strings, bytes, None): that is what reads back unchanged here."""
    payload = io.BytesIO()
    np.save(payload, state.x.detach().cpu().numpy(), allow_pickle=False)
    subfiles = [pickle.dumps(state.metadata), pickle.dumps(tuple(state.shape)), payload.getvalue()]
    file.write(_HEADER.pack(*(len(s) for s in subfiles)))
    for s in subfiles:
        file.write(s)


def read_state_from_file(file, device: Optional[str] = None) -> TrajectoryState:
    """Read one chunk (managan/statefiles.py:32-42).  device None: "cuda" when a GPU is present (as the reference
    does), else "cpu"."""
    head = file.read(_HEADER.size)
    if len(head) != _HEADER.size:
        raise DatasetError("chunk file shorter than its 12-byte header")
    subfiles = []
    for n in _HEADER.unpack(head):
        data = file.read(n)
        if len(data) != n:
            raise DatasetError(f"chunk file truncated: wanted {n} bytes, got {len(data)}")
        subfiles.append(data)
    metadata = _inert_loads(subfiles[0])
    shape = _inert_loads(subfiles[1])
    if not isinstance(shape, (tuple, list)) or not all(isinstance(s, int) for s in shape):
        raise DatasetError(f"item shape must be a tuple of ints, got {shape!r}")
    try:
        x_npy = np.load(io.BytesIO(subfiles[2]), allow_pickle=False)
    except Exception as e:
        raise DatasetError(f"bad .npy payload: {e}") from e
    if device is None:
        device = "cuda" if torch.cuda.is_available() else "cpu"
    return TrajectoryState(tuple(shape), torch.tensor(x_npy, device=device), metadata)


# ------------------------------------------------------------------ checkpoints
def load_checkpoint(path, map_location="cpu"):
    """The dict of managan/config.py:131-137 read without unpickling arbitrary objects.  Raises if the file holds
    anything but tensors and plain containers (a checkpoint whose configuration arguments are class instances
    cannot be read this way; its "states" can be re-saved alone from the reference side)."""
    data = torch.load(path, map_location=map_location, weights_only=True)
    if not isinstance(data, dict) or "states" not in data:
        raise DatasetError('not a model checkpoint: expected a dict with "args", "kwargs" and "states"')
    return data


def states_under(state_dict, prefix: str):
    """The entries of a state dict below `prefix` ("blocks.3.messages_0."), with the prefix removed."""
    if prefix and not prefix.endswith("."):
        prefix += "."
    return {k[len(prefix):]: v for k, v in state_dict.items() if k.startswith(prefix)}


def load_module_states(module: torch.nn.Module, state_dict, prefix: str = "", strict: bool = True):
    """Copy the reference's trained parameters below `prefix` into a mirrored module, by name.  strict: every
    parameter of the module must be present with the same shape and nothing may be left over."""
    sub = states_under(state_dict, prefix)
    if not sub:
        raise KeyError(f"no entries below {prefix!r} in the state dict")
    return module.load_state_dict(sub, strict=strict)


# ------------------------------------------------------------------ dataset directories
def save_predictor_params_to_file(file, box, shape, name):
    """`predictor_params.pickle` of a dataset directory (managan/statefiles.py:44-50): box, item shape and the
    predictor's name."""
    pickle.dump({"box": box, "shape": tuple(shape), "name": name}, file)


def read_predictor_params_from_file(file):
    """managan/statefiles.py:52-54, decoded without instantiating anything."""
    params = _inert_loads(file.read())
    if not isinstance(params, dict) or "box" not in params or "shape" not in params:
        raise DatasetError('predictor parameters must be a dict with "box" and "shape"')
    return params


class DatasetState:
    """One chunk file as a trajectory with a cursor (managan/statefiles.py:57-74): `x` is frame `t` of the first
    `batch` saved trajectories."""

    def __init__(self, fnm, batch=1, device=None):
        with open(fnm, "rb") as f:
            self.traj = read_state_from_file(f, device)
        if len(self.traj.size) < 2:
            raise DatasetError("a dataset chunk holds (time, batch, ...) trajectories")
        self.L, saved_batch, *rest = self.traj.size
        if batch > saved_batch:
            raise DatasetError(f"requested batch {batch} cannot exceed saved batch {saved_batch}")
        self.size = (batch,) + tuple(rest)
        self.shape = self.traj.shape
        self.batch = batch
        self.t = 0

    @property
    def x(self):
        return self.traj.x[self.t, :self.batch]

    @property
    def metadata(self):
        return self.traj.metadata

    def to_model_predictor_state(self):
        return TrajectoryState(self.shape, self.x.clone(), self.metadata)


class DatasetPredictor:
    """Walks the `.bin` chunks of a dataset directory in shuffled order (managan/statefiles.py:76-113).  rng: a
    `random.Random` for the shuffle (the reference uses the global one)."""

    def __init__(self, dataset_dir, stride=1, repeat=False, rng=None, device=None):
        self.dataset_dir, self.stride, self.repeat, self.device = dataset_dir, stride, repeat, device
        self._rng = rng if rng is not None else random
        with open(os.path.join(dataset_dir, "predictor_params.pickle"), "rb") as f:
            params = read_predictor_params_from_file(f)
        self._box, self._shape = params["box"], params["shape"]
        self.file_list = sorted(fnm for fnm in os.listdir(dataset_dir) if fnm.endswith(".bin"))
        self._rng.shuffle(self.file_list)
        self.file_index = 0

    def get_box(self):
        return self._box

    def shape(self):
        return self._shape

    def sample_q(self, batch):
        if self.file_index >= len(self.file_list):
            if not self.repeat:
                raise DatasetError("out of files in dataset!")
            self._rng.shuffle(self.file_list)
            self.file_index = 0
        ans = DatasetState(os.path.join(self.dataset_dir, self.file_list[self.file_index]), batch, self.device)
        self.file_index += 1
        return ans

    def predict(self, L, state, ret=True):
        """Advance the cursor by L strides; returns frames t + stride, ..., t + L stride of the first `batch`
        trajectories, shape (L, batch, ...)."""
        if not isinstance(state, DatasetState):
            raise DatasetError("DatasetPredictor can only handle DatasetState's")
        if not L * self.stride < state.L - state.t:
            raise DatasetError(f"DatasetPredictor tried to predict {self.stride}*{L} steps, but only "
                               f"{state.L - state.t - 1} data remains")
        t_old = state.t
        state.t += L * self.stride
        if ret:
            return state.traj.x[t_old + self.stride:state.t + 1:self.stride, :state.batch]


def get_dataset_predictor(spec):
    return DatasetPredictor(spec)


def get_strided_dataset_predictor(spec):
    """"<stride>?<directory>" (managan/statefiles.py:118-121)."""
    stride, dataset_dir = spec.split("?")
    return DatasetPredictor(dataset_dir, stride=int(stride))


def get_repeated_dataset_predictor(spec):
    stride, dataset_dir = spec.split("?")
    return DatasetPredictor(dataset_dir, stride=int(stride), repeat=True)

"""Callers of the hot path: one-step samplers and the rollout loop around them.

* meanflow_generate: archs/meanflow_painn8.py:302-310 (one denoiser call per rollout step).
* diffusion_generate: the reverse-diffusion loop of archs/diffuser_atoms15.py:536-555 (`steps`
  network calls per rollout step) with its noise schedule (archs/meanflow_painn8.py:222-223) and
  the epsilon combination rule (archs/diffuser_atoms15.py:511-516).
* rollout: ModelPredictor.predict (managan/predictor.py:164-176): L steps, each fed with the last.
* GraphedCall: a fixed launch sequence (layers on a prebuilt neighbour graph) captured once into a
  HIP graph and replayed; what makes small systems, where a forward pass is hundreds of launches
  of a few microseconds each, run at the speed of the kernels instead of the speed of the host.

Random numbers come from a torch.Generator the caller may pass (the reference's TensorRandGen
draws from the global CUDA generator)."""
import math

import torch


def nodecay_cosine_schedule(t, sigma_max):
    """archs/meanflow_painn8.py:222-223"""
    return torch.cos(0.5 * math.pi * t) / torch.sqrt(sigma_max ** -2 + torch.sin(0.5 * math.pi * t) ** 2)


def _randn_like(x, generator):
    return torch.randn(x.shape, device=x.device, dtype=x.dtype, generator=generator)


def meanflow_generate(dn, x_0, sigma_0, generator=None):
    """x_0 (..., atoms, 3) -> the next frame.  dn(st, x_0, z_1) -> v_pred is the denoiser with box and
    per-system inputs already bound.  One network call: z_1 = x_0 + sigma_0 * noise; ans = z_1 - v."""
    *lead, atoms, three = x_0.shape
    if three != 3:
        raise RuntimeError("x_0 must have shape (..., atoms, 3)")
    flat = x_0.reshape(-1, atoms, 3)
    batch = flat.shape[0]
    z_1 = flat + sigma_0 * _randn_like(flat, generator)
    st = (torch.zeros(batch, device=flat.device), torch.ones(batch, device=flat.device))
    ans = z_1 - dn(st, flat, z_1)
    return ans.reshape(*lead, atoms, 3)


def diffusion_generate(dn, x_0, sigma_max, zeta, steps=12, generator=None):
    """dn(t, x_0, x_1_noised) -> (epsilon_pred, x1_pred).  `steps` network calls from t = 0 to t = 1."""
    *lead, atoms, three = x_0.shape
    if three != 3:
        raise RuntimeError("x_0 must have shape (..., atoms, 3)")
    flat = x_0.reshape(-1, atoms, 3)
    dev = flat.device

    def sigma(t):
        return nodecay_cosine_schedule(t, sigma_max)[:, None, None]

    ans = flat + sigma(torch.zeros(1, device=dev)) * _randn_like(flat, generator)
    for i in range(steps):
        t = torch.full((1,), i / steps, device=dev, dtype=torch.float32)
        t_next = torch.full((1,), (i + 1) / steps, device=dev, dtype=torch.float32)
        s_t, s_next = sigma(t), sigma(t_next)
        d_sigma = torch.sqrt(s_t ** 2 - s_next ** 2)
        eps_pred, x1_pred = dn(t, flat, ans)
        eps_comb = (zeta * eps_pred + (ans - x1_pred)) / (zeta + s_t)
        ans = ans - (d_sigma ** 2 / s_t) * eps_comb
        ans = ans + (d_sigma * s_next / s_t) * _randn_like(ans, generator)
    return ans.reshape(*lead, atoms, 3)


def rollout(step, length, x, ret=True):
    """x <- step(x), `length` times, under no_grad.  Returns the (length, *x.shape) trajectory when
    ret is true; x is overwritten with the last frame either way (the reference mutates its state)."""
    traj = torch.zeros(length, *x.shape, dtype=x.dtype, device=x.device) if ret else None
    with torch.no_grad():
        for i in range(length):
            new_x = step(x)
            x.copy_(new_x)
            if ret:
                traj[i] = new_x
    return traj


class GraphedCall:
    """fn(*tensors) -> tensor or tuple of tensors, captured into a HIP graph.

    fn must be a fixed sequence of launches on the current stream for inputs of these shapes: no
    host synchronisation, no data-dependent shapes (so: layers on an already built neighbour graph,
    not the neighbour search, whose edge count goes through the host).  Inputs are copied into
    static buffers before every replay; outputs are the static buffers of the capture and are
    overwritten by the next call.  Parameters are read in place: an optimizer step is seen by the
    next replay, but pre-split weight planes are not rebuilt (inference use)."""

    def __init__(self, fn, *example_inputs, warmup=2):
        self.static_in = [t.detach().clone() for t in example_inputs]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):          # fills the per-parameter caches and the allocator's pool
                fn(*self.static_in)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self.static_out = fn(*self.static_in)

    def __call__(self, *inputs):
        if len(inputs) != len(self.static_in):
            raise RuntimeError(f"expected {len(self.static_in)} inputs, got {len(inputs)}")
        for dst, src in zip(self.static_in, inputs):
            if dst.shape != src.shape or dst.dtype != src.dtype:
                raise RuntimeError("inputs must keep the shapes and dtypes of the capture")
            dst.copy_(src)
        self.graph.replay()
        return self.static_out

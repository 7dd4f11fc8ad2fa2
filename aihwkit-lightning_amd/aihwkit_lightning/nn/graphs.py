"""Replaying analog layers from HIP graphs.

A layer call is a handful of kernel launches (weight preparation, DAC pass, product, and their
backward counterparts); between them the GPU waits for Python. Recorded once into a HIP graph
and replayed, the launches follow each other without the host in between. Nothing in the
library allocates, copies or synchronises outside kernels, so a whole forward + backward of a
module can be recorded with ``torch.cuda.make_graphed_callables``.

Noise under replay: a seed passed by value would be baked into the graph. While a stream is
being captured, the layers read their Philox key and call counter from a device-resident state
(:func:`prepare_noise_state`) and record one counter increment per call, so every replay draws
fresh noise, as every eager call does with its host-drawn seed (the reference draws one seed per
call, ``triton_utils/triton_linear.py:541,617``).

Not for layers that still initialise their input range from data (``init_from_data > 0`` and the
counter below it): that phase asks the device for its progress from the host.
"""
from typing import Tuple, Union

import torch
from torch import Tensor
from torch.nn import Module

from .modules.hip_utils import ops as _ops


def prepare_noise_state(device: Union[torch.device, str, int] = "cuda") -> Tensor:
    """Create (once per device) and return the device noise state ``int64[2]`` = (Philox key,
    call counter). Must run before a capture that contains noisy layers; the key comes from
    torch's CPU generator."""
    dev = torch.device(device) if not isinstance(device, int) else torch.device("cuda", device)
    return _ops.noise_state(dev)


def graphed_module(module: Module, sample_args: Tuple[Tensor, ...], num_warmup_iters: int = 3):
    """``module`` as a callable whose forward and backward each replay one HIP graph.

    ``sample_args``: tensors of the shapes, dtypes and ``requires_grad`` flags of the real
    arguments (as for ``torch.cuda.make_graphed_callables``, which does the recording). The
    returned callable takes the place of ``module(*args)`` in a training step; parameter
    gradients arrive in the parameters' ``.grad`` as usual."""
    for arg in sample_args:
        if isinstance(arg, Tensor) and arg.is_cuda:
            prepare_noise_state(arg.device)
            break
    return torch.cuda.make_graphed_callables(module, tuple(sample_args),
                                             num_warmup_iters=num_warmup_iters)


class CapturedStep:
    """A whole step -- ``step_fn()``, typically forward + backward (+ optimizer) on fixed tensors --
    recorded into ONE HIP graph; calling the object replays it and returns what ``step_fn``
    returned at capture time (the same tensors, refilled by the replay).

    ``step_fn`` must read its inputs from tensors that stay where they are (copy new data into
    them between replays) and must set gradients to None before its forward, so that they are
    allocated inside the recording. A few eager warm-up runs on a side stream come first, as
    torch asks for before a capture."""

    def __init__(self, step_fn, warmup_iters: int = 3):
        prepare_noise_state(torch.cuda.current_device())
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup_iters):
                step_fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.result = step_fn()

    def __call__(self):
        self.graph.replay()
        return self.result

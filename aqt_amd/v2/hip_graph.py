"""A quantized call recorded once into a HIP graph and replayed.

The reference runs under `jax.jit`: a layer call costs one executable launch however much Python
built it (aqt_flax.py:517-590 builds the quantized dot_general per call, config.py:66-90 copies the
configuration per call).  Here the same Python runs per call and issues each kernel itself, which
for small-batch serving costs ten times the kernels' own time.  `GraphedCall` records the kernels
of one call, made on fixed-shape inputs, into a HIP graph; a replay is one launch.

What a recorded call may do: launch kernels of this library and torch device ops on the current
stream.  What it may not: read device data on the host, or change Python-side state that later calls
depend on (calibration statistics, freezing: no conversion calls, no stateful calibrators).  A key
given as host data is a kernel argument fixed at recording time; a key held in a device tensor
(`config.set_context(cfg, key_tensor, ...)`: the fan-out runs as a kernel, the quantizers read their keys
from device memory) is read anew by every replay, which is how a training step with stochastic
rounding is recorded: `GraphedStep`.
"""
from __future__ import annotations

from typing import Any, Callable

import torch

from aqt_amd import ops


def _map_tensors(tree: Any, fn: Callable[[torch.Tensor], Any]) -> Any:
  if isinstance(tree, torch.Tensor):
    return fn(tree)
  if isinstance(tree, (list, tuple)):
    return type(tree)(_map_tensors(t, fn) for t in tree)
  if isinstance(tree, dict):
    return {k: _map_tensors(v, fn) for k, v in tree.items()}
  return tree


class GraphedCall:
  """`fn(*args)` as a HIP graph.

  Tensor arguments (also inside lists, tuples and dicts) become fixed input buffers: a call copies
  the new values in (same shapes and dtypes as at recording), replays, and returns the recorded
  output tensors, which the next call overwrites.  Other arguments are constants of the recording.
  Arguments named in `static_argnums` are used in place, not copied (weights that stay where they
  are): replays read whatever those tensors hold at that time.
  """

  def __init__(self, fn: Callable, *example_args, static_argnums=(), warmup: int = 2):
    if not torch.cuda.is_available():
      raise RuntimeError('GraphedCall needs a GPU')
    self._static = set(static_argnums)
    self._inputs = [
        a if i in self._static else _map_tensors(a, lambda t: t.detach().clone())
        for i, a in enumerate(example_args)
    ]
    for t in self._flat(self._inputs):
      if not t.is_cuda:
        raise ValueError('GraphedCall: tensor arguments must live on the GPU')
    # A first pass on a side stream, as torch.cuda.graph requires, so that the recording finds
    # torch's allocator warm and this library's one-time work (kernel-layout copies of frozen
    # weights) done.  The abs-max workspaces of the recorded kernels belong to this graph: they
    # are allocated, and cleared, inside the recording.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad(), ops.private_workspaces({}):
      for _ in range(max(1, warmup)):
        fn(*self._inputs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    self._workspaces = {}
    self._graph = torch.cuda.CUDAGraph()
    with torch.no_grad(), ops.private_workspaces(self._workspaces), torch.cuda.graph(self._graph):
      self._outputs = fn(*self._inputs)

  @staticmethod
  def _flat(tree):
    out = []
    _map_tensors(tree, out.append)
    return out

  @property
  def inputs(self):
    """The fixed input buffers: a caller may fill them in place and call `replay()`."""
    return self._inputs

  @property
  def outputs(self):
    return self._outputs

  def replay(self):
    self._graph.replay()
    return self._outputs

  def __call__(self, *args):
    if len(args) != len(self._inputs):
      raise ValueError(f'GraphedCall: recorded with {len(self._inputs)} arguments, called with {len(args)}')
    for i, (buf, new) in enumerate(zip(self._inputs, args)):
      if i in self._static:
        continue
      dst, src = self._flat(buf), self._flat(new)
      if len(dst) != len(src):
        raise ValueError(f'GraphedCall: argument {i} has a different structure than at recording')
      for d, s in zip(dst, src):
        if d.shape != s.shape or d.dtype != s.dtype:
          raise ValueError(f'GraphedCall: argument {i} is {tuple(s.shape)} {s.dtype}, '
                           f'recorded as {tuple(d.shape)} {d.dtype}')
        if d.data_ptr() != s.data_ptr():
          d.copy_(s)
    return self.replay()


class GraphedStep:
  """`fn()` as a HIP graph, recorded with gradients enabled: a forward + backward pass over tensors the
  caller keeps (inputs, parameters, the output gradient, a PRNG key in a device tensor).  The caller
  refills those tensors in place and calls `replay()`; what `fn` returned (and the `.grad` tensors its
  backward pass created) are overwritten by every replay.  Before recording, set the `.grad` of the
  leaves to None so that the backward pass writes, not accumulates."""

  def __init__(self, fn: Callable, warmup: int = 3):
    if not torch.cuda.is_available():
      raise RuntimeError('GraphedStep needs a GPU')
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), ops.private_workspaces({}):
      for _ in range(max(1, warmup)):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    self._workspaces = {}
    self._graph = torch.cuda.CUDAGraph()
    with ops.private_workspaces(self._workspaces), torch.cuda.graph(self._graph):
      self._outputs = fn()

  @property
  def outputs(self):
    return self._outputs

  def replay(self):
    self._graph.replay()
    return self._outputs

"""Noise functions for stochastic rounding (mirrors aqt/jax/v2/stochastic_rounding.py).

The instances are descriptors: the quantize kernel generates the same noise
in-kernel from the PRNG key (threefry2x32 in the jax.random layout), so calling
them here returns the noise tensor only for inspection and tests.
"""
from __future__ import annotations

import dataclasses
from typing import Sequence

import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import utils


def _degenerate_noise_shape(shape, noise_sharing_axes=()):
  """stochastic_rounding.py:25-32."""
  return tuple(1 if axis in noise_sharing_axes else s for axis, s in enumerate(shape))


@dataclasses.dataclass
class JaxUniform:
  """jax.random.uniform(key, shape) - 0.5 (stochastic_rounding.py:36-46)."""
  kernel_noise = L.NOISE_JAX_UNIFORM

  def __call__(self, shape, key, noise_sharing_axes: Sequence[int] = ()):
    ns = _degenerate_noise_shape(shape, noise_sharing_axes)
    n = 1
    for s in ns:
      n *= s
    bits = ops.random_bits(key, n, 32, utils.threefry_partitionable)
    fb = torch.bitwise_or(torch.bitwise_right_shift(bits.view(torch.int32) & 0x7FFFFFFF, 9)
                          | ((bits.view(torch.int32) < 0).to(torch.int32) << 22), 0x3F800000)
    u = torch.clamp_min(fb.view(torch.float32) - 1.0, 0.0)
    return (u - 0.5).reshape(ns)


@dataclasses.dataclass
class RandomCenteredUniform:
  """16 random bits in the f32 mantissa, centred (stochastic_rounding.py:50-78)."""
  kernel_noise = L.NOISE_CUSTOM1

  def __call__(self, shape, key, noise_sharing_axes: Sequence[int] = ()):
    ns = _degenerate_noise_shape(shape, noise_sharing_axes)
    n = 1
    for s in ns:
      n *= s
    bits = ops.random_bits(key, n, 16, utils.threefry_partitionable).to(torch.int32) & 0xFFFF
    pat = (bits << 7) | 0x3F800000
    return (pat.view(torch.float32) - (1.5 - 2.0 ** -17)).reshape(ns)

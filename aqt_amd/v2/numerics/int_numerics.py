"""Symmetric integer numerics (mirrors aqt/jax/v2/numerics/int_numerics.py:25-125)."""
from __future__ import annotations

import dataclasses
from typing import Any

import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import utils
from aqt_amd.v2.numerics import numerics


@dataclasses.dataclass(kw_only=True)
class IntSymmetric(numerics.AqtNumerics):
  """sint8 / sint4 / ... numerics; same fields as the reference (int_numerics.py:25-40)."""

  bits: int
  preserve_zero: bool
  preserve_max_val: bool
  clip: bool
  clip_gradient: bool
  round: bool
  noise_fn: Any  # None | stochastic_rounding.JaxUniform | RandomCenteredUniform | partial
  dtype: Any = None

  def __deepcopy__(self, memo):
    # every field is immutable (numbers, flags, dtype tags, a noise function): a field-wise copy
    # is a deep copy, at a fraction of the cost (configurations are copied on every layer call)
    out = utils.clone_fields(self)
    memo[id(self)] = out
    return out

  def get_edge_of_last_int_bucket(self):
    ret = 2.0 ** (self.bits - 1)
    if self.preserve_zero:
      ret -= 0.5
    return ret

  def get_center_of_last_int_bucket(self):
    return self.get_edge_of_last_int_bucket() - 0.5

  def get_quant_bound(self):
    if self.preserve_max_val:
      return self.get_center_of_last_int_bucket()
    return self.get_edge_of_last_int_bucket()

  def _get_fwd_clip_bound(self):
    fwd_clip_bound = self.get_edge_of_last_int_bucket()
    if self.round:
      fwd_clip_bound -= 0.5
    return fwd_clip_bound

  def get_dtype(self):
    return self.dtype

  def kernel_spec(self, held_float: bool = False):
    """Fields of the quantize plan, or None if the kernels do not cover this setting.

    held_float: the caller also takes numerics that keep the rounded values in the float dtype
    (dtype None, the usual setting of fake quantization) when they fit an int8: the kernel then
    writes int8 and the caller casts, which gives the same values; the plan says so in 'held_float'."""
    if not (self.clip and self.round and self.preserve_zero):
      return None
    held = False
    if self.dtype is utils.int8:
      out = L.I8
    elif self.dtype is utils.int4:
      out = L.I4
    elif self.dtype is None and held_float and self.bits <= 8:
      out, held = L.I8, True
    else:
      return None
    noise, sharing = _noise_kind(self.noise_fn)
    if noise is None or sharing:
      return None
    spec = dict(out_dtype=out, quant_bound=float(self.get_quant_bound()),
                clip_bound=float(self._get_fwd_clip_bound()), noise=noise)
    if held:
      spec['held_float'] = True
    return spec

  def vjp_fwd(self, x, context):
    """Noise, clip, round, cast of an already scaled tensor (int_numerics.py:81-111)."""
    spec = self.kernel_spec()
    assert self.bits <= 22, 'Too many bits, float32 has less precision.'
    if spec is None:
      return self._vjp_fwd_stepwise(x, context)
    if spec['noise'] != L.NOISE_NONE:
      assert context.key is not None, (
          'noise_fn is set, requestic stochastic rounding, but RNG was not passed in Context.key')
    x3 = x.contiguous().reshape(1, 1, -1)
    ones = torch.ones((1, 1, 1), dtype=torch.float32, device=x.device)
    q, _ = ops.quantize(x3, reduce=L.REDUCE_COLS, scale=ones, key=context.key,
                        partitionable=utils.threefry_partitionable, **spec)
    return q.reshape(x.shape), (x,)

  def _vjp_fwd_stepwise(self, x, context):
    """The settings the fused kernel leaves out (no rounding or clipping, buckets centred on
    halves, float-held values, wider integers), one elementwise step each."""
    res = (x,)
    input_dtype = x.dtype
    if self.noise_fn:
      assert context.key is not None, (
          'noise_fn is set, requestic stochastic rounding, but RNG was not passed in Context.key')
      x = (x + self.noise_fn(x.shape, context.key)).to(input_dtype)
    if self.clip:
      fwd_clip_bound = self._get_fwd_clip_bound()
      x = torch.clamp(x, -fwd_clip_bound, fwd_clip_bound)
    if self.round:
      x = torch.round(x) if self.preserve_zero else torch.floor(x) + 0.5
    dtype = self.get_dtype()
    if dtype is utils.int4:
      dtype = torch.int8  # int4 values travel in int8 containers
    return x.to(dtype if dtype is not None else input_dtype), res

  def vjp_bwd(self, res, grad):
    ret = grad
    if self.clip_gradient:
      (x,) = res
      clip_bound = self._get_fwd_clip_bound()
      ret = ret * ((-clip_bound <= x) & (x <= clip_bound)).to(ret.dtype)
    return (ret, None)


def _noise_kind(noise_fn):
  """(kernel noise id, noise_sharing_axes) of a noise_fn; (None, ()) if unknown."""
  import functools
  sharing = ()
  if isinstance(noise_fn, functools.partial):
    sharing = tuple(noise_fn.keywords.get('noise_sharing_axes', ()))
    noise_fn = noise_fn.func
  if noise_fn is None:
    return L.NOISE_NONE, sharing
  kind = getattr(noise_fn, 'kernel_noise', None)
  return kind, sharing

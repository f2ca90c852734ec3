"""Scale calibration (mirrors aqt/jax/v2/calibration.py:25-157).

The abs-max reduction runs inside the quantize kernel; these classes carry the
settings and, when called on their own, run that kernel for the scale only.
"""
from __future__ import annotations

import abc
import dataclasses
from typing import Any, Optional, Sequence

import torch

from aqt_amd.v2 import utils


class State(dict):
  """Statistics of a stateful calibrator: the stand-in for a Flax variable collection.

  A config tree is deep-copied freely (`config.set_context` does it on every step); the
  statistics must stay the one shared object through those copies, as variables do.
  """

  def __copy__(self):
    return self

  def __deepcopy__(self, memo):
    return self


@dataclasses.dataclass(kw_only=True)
class Calibration(abc.ABC):
  """calibration.py:34-64."""

  # dtype of the scale arrays; None = the dtype of the input.
  dtype: Any = None
  po2_scale: bool = False

  @abc.abstractmethod
  def get_scale_and_bias_and_sparsity(self, x, shared_axes, numerics_, context=None):
    pass

  def init_calibration(self):
    pass

  def kernel_supported(self) -> bool:
    """True if the fused abs-max kernel implements exactly this calibration."""
    return False


class _UnitBound:
  """Stands in for a numerics object whose quant bound is 1."""

  def get_quant_bound(self):
    return 1.0


def _exp2_int(e):
  """2**e as float32 for an integer tensor e, written into the exponent field (ldexp and pow go
  through the device's exp2/log2 and can be one ulp off)."""
  biased = torch.clamp(e.to(torch.int32) + 127, 1, 254)
  return torch.bitwise_left_shift(biased, 23).view(torch.float32)


def ceil_to_po2(scale):
  """1 / 2**floor(log2(1 / scale)) (calibration.py:25-30), each step rounded to scale.dtype.

  The device reciprocal is not correctly rounded: one ulp at a power of two would halve the
  result or leave it one ulp off a power of two.  In float32 the result is the power of two
  at or above `scale`, read from the exponent field.  In a narrower dtype the roundings of the
  intermediate reciprocal and logarithm are part of the result (log2 can round up to the next
  integer), so those two steps are done in float64 and rounded to the dtype.
  """
  if scale.dtype == torch.float32:
    m, e = torch.frexp(scale)  # scale = m * 2**e with 0.5 <= m < 1
    e = torch.where(m == 0.5, e - 1, e)
    return _exp2_int(e)
  r = torch.reciprocal(scale.double()).to(scale.dtype)
  l = torch.log2(r.double()).to(scale.dtype)
  e = torch.floor(l.float()).to(torch.int32)
  return _exp2_int(-e).to(scale.dtype)


@dataclasses.dataclass(kw_only=True)
class AbsMaxCalibration(Calibration):
  """max(abs(x)) / quant_bound (calibration.py:107-157)."""

  clipping_scale: Optional[float] = None

  def kernel_supported(self) -> bool:
    return not self.po2_scale and not self.clipping_scale

  def get_scale_and_bias_and_sparsity(self, x, shared_axes, numerics_, context=None):
    del context
    msg = ('Perhaps you are using DequantMode.THIS_INPUT (fake_quant) and forgot to set them.')
    assert shared_axes is not None, msg
    from aqt_amd.v2 import lowering  # local import: lowering imports this module's users
    shared_axes = list(shared_axes)
    if not x.is_floating_point():
      x = x.to(torch.float32)  # integer input: the bound is a float (type promotion with the divisor)
    if self.kernel_supported() and shared_axes:
      scale = lowering.absmax_scale(x, shared_axes, numerics_, self.dtype)
      return [scale], [], None
    # clipping_scale / po2_scale: the abs-max kernel (bound 1 leaves max|x|, zeros replaced by
    # ones), then the remaining steps one by one in x.dtype.
    dtype = self.dtype if self.dtype is not None else x.dtype
    if shared_axes:
      abs_max = lowering.absmax_scale(x, shared_axes, _UnitBound(), x.dtype)
    else:  # nothing shared: every element is its own bound
      abs_max = torch.abs(x)
      abs_max = torch.where(abs_max == 0.0, torch.ones_like(abs_max), abs_max)
    if self.clipping_scale:
      abs_max = abs_max * torch.tensor(self.clipping_scale, dtype=x.dtype, device=x.device)
    scale = abs_max / torch.tensor(float(numerics_.get_quant_bound()), dtype=x.dtype, device=x.device)
    if self.po2_scale:
      scale = ceil_to_po2(scale)
    scale = scale.to(dtype)
    return [scale], [], None


@dataclasses.dataclass(kw_only=True)
class ConstantCalibration(Calibration):
  """Constant bound (calibration.py:68-104): scale = bound / quant_bound, no reduction."""

  bound: Any = None
  bias: Any = None

  def get_scale_and_bias_and_sparsity(self, x, shared_axes, numerics_, context=None):
    del context
    if isinstance(self.bound, float) and self.bound <= 0.0:
      raise ValueError(f'{self.bound=} should be positive.')
    dtype = self.dtype if self.dtype is not None else x.dtype
    if isinstance(self.bound, torch.Tensor):
      bound = self.bound  # per-channel bounds, already in their keepdims shape
    else:
      shape = [1 if a in list(shared_axes) else s for a, s in enumerate(x.shape)]
      # bound and quant_bound are host constants; the division happens in x.dtype.
      bound = torch.full(shape, float(self.bound), dtype=x.dtype, device=x.device)
    scale = bound / torch.tensor(float(numerics_.get_quant_bound()), dtype=bound.dtype, device=x.device)
    if self.po2_scale:
      scale = ceil_to_po2(scale)
    if self.bias is None:
      bias = []
    elif isinstance(self.bias, torch.Tensor):
      bias = [self.bias.to(dtype)]
    else:
      bias = [torch.full(tuple(x.shape), float(self.bias), dtype=x.dtype, device=x.device)]
    return [scale.to(dtype)], bias, None


@dataclasses.dataclass(kw_only=True)
class AbsMeanCalibration(Calibration):
  """clipping_scale * mean(abs(x) ** p) ** (1 / p) over the non-zero entries (calibration.py:160-193).

  Reductions and elementwise steps in x.dtype; not a fused kernel (a weight-side calibration).
  """

  clipping_scale: float = None
  p: float = None

  def get_scale_and_bias_and_sparsity(self, x, shared_axes, numerics_, context=None):
    del context
    assert shared_axes is not None
    dtype = self.dtype if self.dtype is not None else x.dtype
    axes = [a % x.dim() for a in shared_axes]

    def total(t):
      return torch.sum(t, dim=axes, keepdim=True) if axes else t

    powed = torch.abs(x) if self.p == 1.0 else torch.abs(x) ** self.p
    abs_sum = total(powed)
    count = total((x != 0.0).to(torch.int32))
    count = torch.where(count == 0, torch.ones_like(count), count)
    abs_mean = abs_sum / count.to(x.dtype)
    if self.p != 1.0:
      abs_mean = abs_mean ** (1.0 / self.p)
    abs_mean = abs_mean * torch.tensor(self.clipping_scale, dtype=x.dtype, device=x.device)
    abs_mean = torch.where(abs_mean == 0.0, torch.ones_like(abs_mean), abs_mean)
    scale = abs_mean / torch.tensor(float(numerics_.get_quant_bound()), dtype=x.dtype, device=x.device)
    if self.po2_scale:
      scale = ceil_to_po2(scale)
    return [scale.to(dtype)], [], None


@dataclasses.dataclass(kw_only=True)
class SnrBasedAutoCalibration(Calibration):
  """Per group, the clipping scale out of `auto_clip_search_config` with the highest
  log(1 + sum(x**2) / sum(err**2)) of the fake-quantized tensor (calibration.py:196-399).

  One quantize / dequantize kernel pair per candidate plus elementwise steps; meant for
  weights, as in the reference.
  """

  auto_clip_search_config: Sequence[float] = None

  def get_scale_and_bias_and_sparsity(self, x, shared_axes, numerics_, context=None):
    from aqt_amd.v2 import aqt_tensor  # local import: aqt_tensor's users import this module
    from aqt_amd.v2 import lowering
    dtype = self.dtype if self.dtype is not None else x.dtype
    axes = [a % x.dim() for a in shared_axes]
    clip_shape = [1 if a in axes else s for a, s in enumerate(x.shape)]
    best = torch.ones(clip_shape, dtype=torch.float32, device=x.device)
    max_snr = torch.zeros(clip_shape, dtype=torch.float32, device=x.device)
    if axes:
      abs_max = lowering.absmax_scale(x, axes, _UnitBound(), x.dtype)
    else:
      abs_max = torch.abs(x)
      abs_max = torch.where(abs_max == 0.0, torch.ones_like(abs_max), abs_max)
    quant_bound = torch.tensor(float(numerics_.get_quant_bound()), dtype=x.dtype, device=x.device)

    def total(t):
      return torch.sum(t, dim=axes, keepdim=True) if axes else t

    signal = total(x * x)
    for clip_scale in self.auto_clip_search_config:
      bound = abs_max * torch.tensor(clip_scale, dtype=x.dtype, device=x.device)
      scale = (bound / quant_bound).to(dtype)
      qt = aqt_tensor.QTensor(qvalue=None, scale=[scale], scale_t=None, bias=[], dequant_dtype=x.dtype)
      qt = qt.quant(x)
      qt.qvalue, _ = numerics_.vjp_fwd(qt.qvalue, context)
      if numerics_.get_dtype() is utils.int4:
        qt.container_dtype = utils.int4
      err = x - qt.dequant()
      noise = total(err * err)
      snr = torch.log(1 + signal / noise)
      best = torch.where(snr > max_snr, torch.tensor(clip_scale, dtype=torch.float32, device=x.device), best)
      max_snr = torch.maximum(snr.to(torch.float32), max_snr)
    # a tensor divisor: division by a Python scalar becomes a multiplication by its reciprocal
    scale = (abs_max * best) / quant_bound.to(torch.float32)
    if self.po2_scale:
      scale = ceil_to_po2(scale)
    return [scale.to(dtype)], [], None

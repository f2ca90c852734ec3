"""Static-range calibrators (mirrors aqt/jax/v2/flax/aqt_flax_calibration.py:33-251).

The reference keeps their statistics in Flax variables of a `quant_collection`; here the
statistics are device tensors in the `state` dict the calibrator is given (pass the same dict
every time the calibrator is built, e.g. `functools.partial(..., state=calibration.State())`, which
stays one object through the deep copies of a config; it is what a checkpoint of the layer holds
under that collection).  Reductions use the abs-max kernel
and elementwise / reduction tensor arithmetic; these calibrators run in the calibration phase
and on the step-by-step path, not in the fused kernels.
"""
from __future__ import annotations

import dataclasses
from typing import Optional, Sequence

import torch

from aqt_amd.v2 import calibration
from aqt_amd.v2 import utils

_SUM_OF_ONES = 'sum_of_ones'
_SUM_OF_VALS = 'sum_of_vals'
_MAX_OF_ABS_VALS = 'max_of_abs_vals'
_SUM_OF_L1_VALS = 'sum_of_l1_vals'
_SUM_OF_LP_VALS = 'sum_of_lp_vals'


def _abs_max(x, shared_axes):
  """max(abs(x)) over shared_axes with keepdims, zeros kept (unlike AbsMaxCalibration)."""
  axes = [a % x.dim() for a in shared_axes] if shared_axes is not None else list(range(x.dim()))
  if not axes:
    return torch.abs(x)
  return torch.linalg.vector_norm(x, ord=float('inf'), dim=axes, keepdim=True)  # one reduction pass


def _scale_from_bound(self, bound, x, numerics_):
  dtype = self.dtype if self.dtype is not None else x.dtype
  scale = bound / torch.tensor(float(numerics_.get_quant_bound()), dtype=bound.dtype, device=bound.device)
  if self.po2_scale:
    scale = calibration.ceil_to_po2(scale)
  return [scale.to(dtype)], [], None


@dataclasses.dataclass(kw_only=True)
class MeanOfAbsMaxCalibration(calibration.Calibration):
  """Static range: the mean of the abs-max seen in QuantMode.CALIBRATE (:33-84)."""

  quant_collection: str = 'aqt'
  state: Optional[dict] = None

  def get_bound(self, x, shared_axes, context=None):
    abs_max = _abs_max(x, shared_axes)
    quant_mode = context.quant_mode if context else utils.QuantMode.TRAIN
    if self.state is None:
      self.state = calibration.State()
    is_initializing = 'sum_of_max' not in self.state
    if is_initializing:
      self.state['sum_of_max'] = torch.zeros_like(abs_max)
      self.state['count'] = torch.zeros((), dtype=torch.int32, device=x.device)
    if quant_mode == utils.QuantMode.CALIBRATE and not is_initializing:
      self.state['sum_of_max'] = self.state['sum_of_max'] + abs_max
      self.state['count'] = self.state['count'] + 1
    return self.state['sum_of_max'] / self.state['count']

  def get_scale_and_bias_and_sparsity(self, x, shared_axes, numerics_, context=None):
    return _scale_from_bound(self, self.get_bound(x, shared_axes, context), x, numerics_)


@dataclasses.dataclass(kw_only=True)
class WeightedStatsCalibration(calibration.Calibration):
  """Bound = l1_dev_coeff * l1_dev + lp_dev_coeff * lp_dev + max_dev_coeff * max_dev +
  const_bound_coeff over exponentially averaged statistics (:87-251)."""

  quant_collection: str = 'aqt'
  state: Optional[dict] = None

  l1_dev_coeff: float = 0.0
  lp_dev_coeff: float = 0.0
  max_dev_coeff: float = 0.0
  const_bound_coeff: float = 0.0

  update_count_prior: float = 1.0
  max_dev_prior: float = 0.0
  mean_prior: float = 0.0
  l1_dev_prior: float = 0.0
  lp_dev_prior: float = 0.0

  lp_order: int = 2
  safe_divide: bool = False
  filter_zeros: bool = True
  tpu_cross_replica_sum: bool = False
  ema_update_count: float = 100

  def _divide(self, x, y):
    if self.safe_divide:
      return torch.where(y != 0, x / y, torch.zeros_like(x))
    return x / y

  def _mean(self):
    return self._divide(self.state[_SUM_OF_VALS], self.state[_SUM_OF_ONES])

  def _max_dev(self):
    return self.state[_MAX_OF_ABS_VALS]

  def _l1_dev(self):
    return self._divide(self.state[_SUM_OF_L1_VALS], self.state[_SUM_OF_ONES])

  def _lp_dev(self):
    mean = self._divide(self.state[_SUM_OF_LP_VALS], self.state[_SUM_OF_ONES])
    if self.lp_order == 2:
      return torch.sqrt(mean)
    return mean ** (1.0 / self.lp_order)

  def _update_var(self, name, s, shared_axes, reduce_max=False):
    axes = [a % s.dim() for a in shared_axes] if shared_axes is not None else list(range(s.dim()))
    if axes:
      s = torch.amax(s, dim=axes, keepdim=True) if reduce_max else torch.sum(s, dim=axes, keepdim=True)
    if self.tpu_cross_replica_sum:
      raise NotImplementedError('support for tpu_cross_replica_sum=True is not implemented')
    rate = 1.0 / self.ema_update_count
    self.state[name] = (1.0 - rate) * self.state[name] + rate * s.to(torch.float32)

  def get_bound(self, x, shared_axes, context=None):
    if self.lp_order > 30:
      raise NotImplementedError('For higher norms we should add stabilization.')
    quant_mode = context.quant_mode if context else utils.QuantMode.TRAIN
    stats_shape = [1 if (shared_axes is None or a in [b % x.dim() for b in shared_axes]) else s
                   for a, s in enumerate(x.shape)] if shared_axes is not None else list(x.shape)
    if self.state is None:
      self.state = calibration.State()

    def make_var(name, init_val):
      if name not in self.state:
        self.state[name] = torch.full(stats_shape, float(init_val), dtype=torch.float32, device=x.device)

    make_var(_SUM_OF_ONES, self.update_count_prior)
    make_var(_SUM_OF_VALS, self.mean_prior * self.update_count_prior)
    make_var(_MAX_OF_ABS_VALS, self.max_dev_prior)
    make_var(_SUM_OF_L1_VALS, self.l1_dev_prior * self.update_count_prior)
    make_var(_SUM_OF_LP_VALS, self.lp_dev_prior ** self.lp_order * self.update_count_prior)

    if quant_mode in (utils.QuantMode.TRAIN, utils.QuantMode.CALIBRATE):
      ones = torch.where(x != 0, 1.0, 0.0).to(x.dtype) if self.filter_zeros else torch.ones_like(x)
      px = x if self.lp_order % 2 == 0 else torch.abs(x)
      self._update_var(_SUM_OF_ONES, ones, shared_axes)
      self._update_var(_SUM_OF_VALS, x, shared_axes)
      self._update_var(_MAX_OF_ABS_VALS, torch.abs(x), shared_axes, reduce_max=True)
      self._update_var(_SUM_OF_L1_VALS, torch.abs(x), shared_axes)
      self._update_var(_SUM_OF_LP_VALS, px ** self.lp_order, shared_axes)

    return (self.l1_dev_coeff * self._l1_dev() + self.lp_dev_coeff * self._lp_dev()
            + self.max_dev_coeff * self._max_dev() + self.const_bound_coeff)

  def get_scale_and_bias_and_sparsity(self, x, shared_axes, numerics_, context=None):
    return _scale_from_bound(self, self.get_bound(x, shared_axes, context), x, numerics_)

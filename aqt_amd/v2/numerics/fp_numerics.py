"""Emulated small floats in a bf16 / f32 container (mirrors aqt/jax/v2/numerics/fp_numerics.py).

`fp_round` runs the HIP kernel behind `aqtx_fp_round`; the configurations and the numerics
class keep the reference's names.  Radix-4 rounding (fp_numerics.py:653-705) is not built.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Optional

import torch

from aqt_amd import ops
from aqt_amd.v2 import utils
from aqt_amd.v2.numerics import numerics


@dataclasses.dataclass(frozen=True, kw_only=True)
class FpNumericsConfig:
  """fp_numerics.py:26-34."""
  nexp: int
  minexp: int
  nmant: int
  has_subnormals: bool
  has_two_nan: bool
  has_naninf: bool
  radix: int


def _make(nexp, nmant, has_subnormals, minexp=0, has_two_nan=False, has_naninf=False, radix=2):
  return FpNumericsConfig(nexp=nexp, minexp=minexp, nmant=nmant, has_subnormals=has_subnormals,
                          has_two_nan=has_two_nan, has_naninf=has_naninf, radix=radix)


# FP6 (fp_numerics.py:36-94)
e5m0_ocp = _make(5, 0, True)
e4m1_ocp = _make(4, 1, True)
e3m2_ocp = _make(3, 2, True)
e2m3_ocp = _make(2, 3, True)
e1m4_ocp = _make(1, 4, True)
e0m5_ocp = _make(0, 5, True)
# FP5 (fp_numerics.py:96-148)
e4m0_ocp = _make(4, 0, True)
e3m1_ocp = _make(3, 1, True)
e2m2_ocp = _make(2, 2, True)
e1m3_ocp = _make(1, 3, True)
e0m4_ocp = _make(0, 4, True)
# FP4 (fp_numerics.py:150-232)
e3m0 = _make(3, 0, False)
e3m0_ocp = _make(3, 0, True)
e2m1 = _make(2, 1, False)
e2m1_ocp = _make(2, 1, True)
e1m2 = _make(1, 2, False)
e1m2_ocp = _make(1, 2, True)
e0m3 = _make(0, 3, False)
e0m3_ocp = _make(0, 3, True)
# Misc (fp_numerics.py:234-286); the last four describe existing dtypes and cannot be rounded to
e1m0 = _make(1, 0, False)
float8_e4m3fn = _make(4, 3, True, minexp=-6, has_two_nan=True)
float8_e5m2 = _make(5, 2, True, minexp=-14, has_naninf=True)
float16 = _make(5, 10, True, minexp=-14, has_naninf=True)
RADIX4 = _make(3, 0, True, radix=4)


def fp_round(x: torch.Tensor, *, cfg: FpNumericsConfig, key, stochastic_rounding: bool,
             test_noise_axis: Optional[int] = None) -> torch.Tensor:
  """fp_numerics.py:279-459 (radix 2) and :661-706 (radix 4): x (bf16 or f32) rounded to `cfg`, same dtype."""
  assert cfg.radix == 2 or cfg.radix == 4, 'Only radix 2 and 4 are supported.'
  if cfg.radix == 4:
    assert cfg == RADIX4
    assert x.dtype == torch.bfloat16, f'Unsupported dtype for sthochastic rounding: {x.dtype}.'
  assert cfg.minexp == 0, 'minexp not implemented'
  assert not cfg.has_two_nan, 'two_nan not implemented'
  assert not cfg.has_naninf, 'naninf not implemented'
  msg = f'Unsupported dtype for sthochastic rounding: {x.dtype}.'
  assert x.dtype in (torch.bfloat16, torch.float32), msg
  container_man = 7 if x.dtype == torch.bfloat16 else 23
  assert cfg.nmant <= container_man, 'bf16 man bits'
  noise_mod = None
  if stochastic_rounding and test_noise_axis is not None:
    axis = test_noise_axis % x.dim()
    if axis != x.dim() - 1:
      # the kernel counts the equi-spaced test noise along the last axis
      y = fp_round(x.movedim(axis, -1).contiguous(), cfg=cfg, key=key, stochastic_rounding=True, test_noise_axis=-1)
      return y.movedim(-1, axis)
    noise_mod = x.shape[-1]
  return ops.fp_round(x, nexp=cfg.nexp, nmant=cfg.nmant, has_subnormals=cfg.has_subnormals, key=key,
                      stochastic_rounding=stochastic_rounding, noise_mod=noise_mod,
                      partitionable=utils.threefry_partitionable, radix=cfg.radix)


def fp_largest_representable(cfg: FpNumericsConfig):
  """fp_numerics.py:594-615."""
  nexp, nmant = cfg.nexp, cfg.nmant
  assert cfg.minexp == 0, 'minexp not implemented'
  assert not cfg.has_naninf, 'naninf not implemented'
  if cfg == RADIX4:
    return 64.0
  assert cfg.radix == 2, 'Only radix2 or radix4 is supported.'
  max_exp = 2**nexp - 1 + cfg.minexp - (1 if cfg.has_subnormals else 0)
  max_mant = 2**nmant - 1 - (1 if cfg.has_two_nan else 0)
  max_normal = 2**max_exp * (1 + (max_mant / 2**nmant))
  max_subnormal = 2**cfg.minexp * max_mant / 2**nmant
  if cfg.has_subnormals and nexp == 0:
    return max_subnormal
  return max_normal


@dataclasses.dataclass(kw_only=True)
class FpNumerics(numerics.AqtNumerics):
  """fp_numerics.py:618-650."""

  cfg: FpNumericsConfig
  stochastic_rounding: bool = False
  clip_gradient: bool = False

  def __deepcopy__(self, memo):
    # every field is immutable (numbers, flags, dtype tags, a noise function): a field-wise copy
    # is a deep copy, at a fraction of the cost (configurations are copied on every layer call)
    out = utils.clone_fields(self)
    memo[id(self)] = out
    return out

  def get_quant_bound(self):
    return fp_largest_representable(cfg=self.cfg)

  def get_dtype(self):
    return torch.bfloat16

  def vjp_fwd(self, x, context):
    x = fp_round(x.to(torch.bfloat16), cfg=self.cfg, key=context.key,
                 stochastic_rounding=self.stochastic_rounding)
    return x, (x,)

  def vjp_bwd(self, res, grad):
    ret = grad
    if self.clip_gradient:
      (x,) = res
      clip_bound = self.get_quant_bound()
      ret = ret * ((-clip_bound <= x) & (x <= clip_bound))
    return (ret, None)

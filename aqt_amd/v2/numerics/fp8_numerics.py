"""fp8 numerics (mirrors aqt/jax/v2/numerics/fp8_numerics.py:25-145)."""
from __future__ import annotations

import dataclasses
from typing import Any

import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import utils
from aqt_amd.v2.numerics import numerics

fp8_map = {'e4m3': utils.float8_e4m3fn, 'e5m2': utils.float8_e5m2}
_FINFO_MAX = {utils.float8_e4m3fn: 448.0, utils.float8_e5m2: 57344.0}


def _convert_to_fp8dtype(dtype):
  if dtype == utils.float8_e4m3fn:
    return 'e4m3'
  if dtype == utils.float8_e5m2:
    return 'e5m2'
  return None


@dataclasses.dataclass(kw_only=True)
class Fp8Numerics(numerics.AqtNumerics):
  """fp8_numerics.py:68-134."""

  dtype: Any
  exponent_bits: int = 4
  mantissa_bits: int = 3
  stochastic_rounding: bool = False

  def __deepcopy__(self, memo):
    # every field is immutable (numbers, flags, dtype tags, a noise function): a field-wise copy
    # is a deep copy, at a fraction of the cost (configurations are copied on every layer call)
    out = utils.clone_fields(self)
    memo[id(self)] = out
    return out

  def _get_edge_of_last_fp8_bucket(self):
    return _FINFO_MAX[self.dtype]

  def get_dtype(self):
    return self.dtype

  def get_quant_bound(self):
    return self._get_edge_of_last_fp8_bucket()

  def kernel_spec(self, held_float: bool = False):
    if self.dtype == utils.float8_e4m3fn:
      assert (self.exponent_bits, self.mantissa_bits) == (4, 3)
      out = L.E4M3
    elif self.dtype == utils.float8_e5m2:
      assert (self.exponent_bits, self.mantissa_bits) == (5, 2)
      out = L.E5M2
    else:
      return None
    b = float(self.get_quant_bound())
    return dict(out_dtype=out, quant_bound=b, clip_bound=b,
                noise=L.NOISE_FP8_MANTISSA if self.stochastic_rounding else L.NOISE_NONE)

  def vjp_fwd(self, x, context):
    spec = self.kernel_spec()
    if spec is None:
      raise NotImplementedError(f'no HIP kernel for {self}')
    if self.stochastic_rounding:
      assert context.key is not None, 'stochastic_rounding requires PRNGKey in Context'
    x3 = x.contiguous().reshape(1, 1, -1)
    ones = torch.ones((1, 1, 1), dtype=torch.float32, device=x.device)
    q, _ = ops.quantize(x3, reduce=L.REDUCE_COLS, scale=ones, key=context.key,
                        partitionable=utils.threefry_partitionable, **spec)
    return q.view(self.dtype).reshape(x.shape), (x,)

  def vjp_bwd(self, res, grad):
    del res
    return (grad, None)

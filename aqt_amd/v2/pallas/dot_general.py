"""QTensor | array x QTensor | array -> dequantized array (mirrors aqt/jax/v2/pallas/dot_general.py:29-137)."""
from __future__ import annotations

import torch

from aqt_amd.v2 import aqt_dot_general
from aqt_amd.v2 import aqt_tensor
from aqt_amd.v2 import utils

QTensor = aqt_tensor.QTensor
DequantMode = aqt_dot_general.DequantMode


def load_qtensor(qt: QTensor) -> QTensor:
  """pallas/dot_general.py:29-39 turns memory references into arrays; a QTensor here holds
  device tensors already."""
  return qt


def _dtype_to_bits(qt: QTensor):
  """pallas/dot_general.py:42-57 (an int4 qvalue is an int8 tensor tagged `container_dtype`)."""
  dtype = qt.qvalue.dtype
  if dtype in (torch.bfloat16, torch.float32):
    return None
  if dtype == torch.int8:
    return 4 if qt.container_dtype is utils.int4 else 8
  if dtype == torch.float8_e4m3fn:
    return 'e4m3'
  if dtype == torch.float8_e5m2:
    return 'e5m2'
  raise ValueError('dtype must be one one of {bfloat16, float32, int8, int4, float8_*}')


def dot_general(lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None,
                lhs_dequant_mode: DequantMode = DequantMode.OUTPUT,
                rhs_dequant_mode: DequantMode = DequantMode.OUTPUT) -> torch.Tensor:
  """lax.dot_general on quantized operands, always returning the dequantized result
  (pallas/dot_general.py:60-137).  `precision` is ignored, as in the reference.

  Two quantized operands with output dequantisation run the contraction kernel with the scales in
  its epilogue; every other combination follows the reference step by step (cast or dequantize,
  contract, scale the result).  The given QTensors are left as they are (the reference overwrites
  the qvalue of a QTensor met by a float operand with its float cast).
  """
  del precision
  both = isinstance(lhs, QTensor) and isinstance(rhs, QTensor)
  if isinstance(lhs, QTensor) and not both:
    lhs = lhs.replace(qvalue=lhs.qvalue.to(torch.promote_types(lhs.dequant_dtype, rhs.dtype)), container_dtype=None)
  if isinstance(rhs, QTensor) and not both:
    rhs = rhs.replace(qvalue=rhs.qvalue.to(torch.promote_types(rhs.dequant_dtype, lhs.dtype)), container_dtype=None)
  if isinstance(lhs, torch.Tensor):
    lhs = QTensor(qvalue=lhs, scale=[], scale_t=None, bias=[], dequant_dtype=lhs.dtype)
  if isinstance(rhs, torch.Tensor):
    rhs = QTensor(qvalue=rhs, scale=[], scale_t=None, bias=[], dequant_dtype=rhs.dtype)
  if preferred_element_type is None:
    preferred_element_type = torch.promote_types(lhs.dequant_dtype, rhs.dequant_dtype)

  cfg = aqt_dot_general.dot_general_raw_make(lhs_bits=_dtype_to_bits(lhs), rhs_bits=_dtype_to_bits(rhs))
  cfg.lhs.dequant_mode = lhs_dequant_mode
  cfg.rhs.dequant_mode = rhs_dequant_mode
  output_only = lhs_dequant_mode == DequantMode.OUTPUT and rhs_dequant_mode == DequantMode.OUTPUT
  if not output_only:
    cfg.dg_accumulator_dtype = None

  if both and output_only and lhs.scale and rhs.scale:
    try:
      return aqt_dot_general._qtensor_dot_general(  # pylint: disable=protected-access
          lhs, rhs, dimension_numbers, cfg, dequant_dtype=preferred_element_type)
    except aqt_dot_general._NotFused:  # pylint: disable=protected-access
      pass
  return aqt_dot_general._qtensor_dot_general_unfused(  # pylint: disable=protected-access
      lhs, rhs, dimension_numbers, cfg, dequant_dtype=preferred_element_type).dequant()

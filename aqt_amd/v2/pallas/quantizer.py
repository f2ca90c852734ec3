"""Array -> QTensor with float32 scales (mirrors aqt/jax/v2/pallas/quantizer.py:33-68)."""
from __future__ import annotations

import functools
from typing import Optional, Sequence

import torch

from aqt_amd.v2 import aqt_quantizer
from aqt_amd.v2 import aqt_tensor
from aqt_amd.v2 import calibration

QTensor = aqt_tensor.QTensor


def quant(x: torch.Tensor, n_bits, calibration_axes: Optional[Sequence[int]] = None,
          use_dummy_static_bound: bool = False) -> QTensor:
  """Channel-wise quantization of x over `calibration_axes` (the whole tensor when None).

  `use_dummy_static_bound` is accepted and, as in the reference, changes nothing: there
  (pallas/quantizer.py:62-65) the ConstantCalibration factory is stored on a quantizer whose
  abs-max calibrator quantizer_make has already built (aqt_quantizer.py:201-205), and calibrate()
  asks the built one (aqt_quantizer.py:136-140).  The same steps are taken here, with the same
  outcome: abs-max scales.
  """
  quantizer = aqt_quantizer.quantizer_make(n_bits, scale_stop_grad=False, scale_dtype=torch.float32)
  if calibration_axes is None:
    quantizer.calib_shared_axes = 'per_tensor'
  if use_dummy_static_bound:
    quantizer.calibration = functools.partial(calibration.ConstantCalibration, bound=1.0)
  qx, _ = quantizer.quant(x, calibration_axes=calibration_axes)
  qx.dequant_dtype = torch.float32
  return qx

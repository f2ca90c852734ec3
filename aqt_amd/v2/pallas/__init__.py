"""Standalone quantize / contract entry points (mirrors aqt/jax/v2/pallas/__init__.py:16-24).

The reference offers `quant` (array -> QTensor with float32 scales) and `dot_general`
(QTensor | array x QTensor | array -> dequantized array) for use inside Pallas kernels.  The
module path and the signatures are kept so that callers find them where they were; there is no
Pallas here: a QTensor holds ordinary device tensors and `dot_general` runs the HIP kernels.
"""
from aqt_amd.v2.pallas import dot_general as _aqt_dot_general
from aqt_amd.v2.pallas import quantizer as _aqt_quantizer

quant = _aqt_quantizer.quant
load_qtensor = _aqt_dot_general.load_qtensor
dot_general = _aqt_dot_general.dot_general
DequantMode = _aqt_dot_general.DequantMode


def pallas_call(*args, **kwargs):
  """pallas/pallas_call.py:65 wraps a Pallas kernel so that it takes QTensors; nothing to wrap here."""
  del args, kwargs
  raise NotImplementedError(
      'pallas_call: there are no Pallas kernels in this build; call quant() and dot_general() directly, '
      'they run whole tensors on the GPU')

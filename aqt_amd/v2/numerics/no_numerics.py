"""No quantization (mirrors aqt/jax/v2/numerics/no_numerics.py:23-43)."""
import dataclasses
from typing import Any

from aqt_amd.v2 import utils
from aqt_amd.v2.numerics import numerics


@dataclasses.dataclass(kw_only=True)
class NoNumerics(numerics.AqtNumerics):

  noise_fn: Any = None
  dtype: Any = None

  def __deepcopy__(self, memo):
    # every field is immutable (numbers, flags, dtype tags, a noise function): a field-wise copy
    # is a deep copy, at a fraction of the cost (configurations are copied on every layer call)
    out = utils.clone_fields(self)
    memo[id(self)] = out
    return out

  def get_dtype(self):
    return None

  def get_quant_bound(self):
    pass

  def vjp_fwd(self, x, context):
    pass

  def vjp_bwd(self, res, grad):
    pass

"""Abstract numerics (mirrors aqt/jax/v2/numerics/numerics.py:21-54)."""
import abc


class AqtNumerics(abc.ABC):
  """What a numerics object must provide.

  `kernel_spec()` is this build's addition: it lowers the numerics to the fields of
  the quantize kernel's plan, or returns None when no kernel implements it.
  """

  @abc.abstractmethod
  def get_dtype(self):
    pass

  @abc.abstractmethod
  def get_quant_bound(self):
    pass

  @abc.abstractmethod
  def vjp_fwd(self, x, context):
    pass

  @abc.abstractmethod
  def vjp_bwd(self, res, grad):
    pass

  def kernel_spec(self, held_float: bool = False):
    return None

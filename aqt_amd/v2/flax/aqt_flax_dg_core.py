"""dg_core as the layer modules call it (mirrors aqt/jax/v2/flax/aqt_flax_dg_core.py:22-127).

The reference wraps `dg_core_vjp_fwd` / `dg_core_vjp_bwd` in `flax.linen.custom_vjp` so that the
custom gradient survives Flax's module lifting, and returns no gradient for the variables declared
inside the layer.  Here the custom gradient is the `torch.autograd.Function` behind
`DotGeneral.dg_core` and the layer's own variables (quantized operands, calibration statistics) are
buffers outside the autograd graph, so the function reduces to the call itself; it keeps the
reference's name and argument order for callers written against it.
"""
from __future__ import annotations


def dg_core_flax_lifted(lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, mdl, cfg):
  """Returns (out, (lhs_qt, rhs_qt)) like DotGeneral.dg_core; `mdl` is the calling module."""
  del mdl
  return cfg.dg_core(lhs=lhs, rhs=rhs, lhs_qt=lhs_qt, rhs_qt=rhs_qt, dimension_numbers=dimension_numbers)

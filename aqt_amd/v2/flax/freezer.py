"""Freezer: identity that can store its input, or hand back what was stored.

Counterpart of aqt/jax/v2/flax/freezer.py.  The stored value (any pytree-like Python
object, in practice a QTensor) is an attribute of a torch module; `state()` /
`load_state()` expose it for checkpoints.  get() returns the stored value only in
READ mode; set() stores only in WRITE mode (in READ mode it merely initialises an
empty freezer, the role `self.variable(..., initializer)` plays for checkpoint
restoring in the reference, freezer.py:60-69).
"""
import enum
from typing import Any, Callable, Optional

import torch


class FreezerMode(enum.Enum):
  """freezer.py:22-26."""
  NONE = 1
  WRITE = 2
  READ = 3


_FREEZE_VAR_NAME = 'frozen'


class Freezer(torch.nn.Module):
  """freezer.py:32-100."""

  def __init__(self, *, collection: str = 'aqt', mode: FreezerMode = FreezerMode.NONE,
               axis_metadata_wrapper: Optional[Callable[[Any], Any]] = None, name: Optional[str] = None):
    super().__init__()
    self.collection = collection
    self.mode = mode
    self.axis_metadata_wrapper = axis_metadata_wrapper
    self.var_name = name
    self._frozen = None
    self._has_variable = False

  def has_variable(self) -> bool:
    return self._has_variable

  def get(self):
    if self.mode in (FreezerMode.NONE, FreezerMode.WRITE):
      return None
    if self.mode == FreezerMode.READ:
      return self._frozen if self._has_variable else None
    assert False, 'Unknown quant mode.'

  def set(self, inputs) -> None:
    if self.mode == FreezerMode.NONE:
      return None
    if self.mode == FreezerMode.WRITE:
      self._frozen, self._has_variable = inputs, True
      return None
    if self.mode == FreezerMode.READ:
      # initialiser only: a frozen value is never changed while serving
      if not self._has_variable:
        self._frozen, self._has_variable = inputs, True
      return None
    assert False, 'Unknown quant mode.'

  # ---- checkpoint access ----------------------------------------------------------------
  def state(self):
    """{collection: {'frozen': value}} or {} when nothing is stored."""
    return {self.collection: {_FREEZE_VAR_NAME: self._frozen}} if self._has_variable else {}

  def load_state(self, state) -> None:
    if self.collection in state and _FREEZE_VAR_NAME in state[self.collection]:
      self._frozen, self._has_variable = state[self.collection][_FREEZE_VAR_NAME], True

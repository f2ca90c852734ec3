"""One-tensor quantizer (mirrors aqt/jax/v2/aqt_quantizer.py:38-214)."""
from __future__ import annotations

import copy
import contextlib
import contextvars
import dataclasses
import functools
from typing import Any, Optional, Sequence

import torch

from aqt_amd import _lib as L
from aqt_amd.v2 import aqt_tensor
from aqt_amd.v2 import calibration
from aqt_amd.v2 import lowering
from aqt_amd.v2 import utils
from aqt_amd.v2.numerics import no_numerics
from aqt_amd.v2.numerics import numerics
from aqt_amd.v2.numerics import utils as numerics_utils

AbstractAqtNumerics = numerics.AqtNumerics
AbstractAqtCalibration = calibration.Calibration



# Calibration results of an abandoned fused attempt, handed to the step-by-step path that takes
# over the same call (id(quantizer) -> incomplete QTensor); None outside such a hand-over.
_REPLAY: 'contextvars.ContextVar' = contextvars.ContextVar('aqt_calibration_replay', default=None)


# Where Quantizer.calibrate leaves its results while a lowered attempt runs a whole DotGeneralQuantizer.calibrate
# step by step (id(quantizer) -> incomplete QTensor), so that a fall-back of the same call can replay them.
_RECORD: 'contextvars.ContextVar' = contextvars.ContextVar('aqt_calibration_record', default=None)


@contextlib.contextmanager
def record_calibrations(into: dict):
  """Inside, every Quantizer.calibrate also stores its result in `into` under the quantizer object's id."""
  token = _RECORD.set(into)
  try:
    yield
  finally:
    _RECORD.reset(token)


@contextlib.contextmanager
def replay_calibrations(done: dict):
  """Inside, Quantizer.calibrate returns (once) what `done` holds for that quantizer object
  instead of calibrating again."""
  token = _REPLAY.set(dict(done))
  try:
    yield
  finally:
    _REPLAY.reset(token)

@dataclasses.dataclass(kw_only=True)
class Quantizer:
  """Configuration of quantization of one tensor (aqt_quantizer.py:38-62)."""

  numerics: AbstractAqtNumerics
  calib_shared_axes: Any  # None | Sequence[int] | 'per_tensor'
  scale_stop_grad: bool
  scale_dtype: Any = None
  calibration: Any = None  # class or functools.partial producing a Calibration
  _calibrator: Any = None
  context: utils.Context = None

  def __deepcopy__(self, memo):
    # Field by field: the flags, dtype tags and the calibration factory (a class or a
    # functools.partial, never changed in place) are shared, the rest is copied.  Same result as
    # the generic deep copy; configurations are copied on every layer call.
    out = utils.clone_fields(self)
    memo[id(self)] = out
    out.numerics = copy.deepcopy(self.numerics, memo)
    if not isinstance(self.calib_shared_axes, (str, type(None))):
      out.calib_shared_axes = copy.deepcopy(self.calib_shared_axes, memo)
    out._calibrator = copy.deepcopy(self._calibrator, memo)
    out.context = copy.deepcopy(self.context, memo)
    return out

  def init_calibration(self):
    assert self._calibrator is None, 'second call to self.init_calibration()'
    if self.calibration is not None:
      self._calibrator = self.calibration(dtype=self.scale_dtype)
      self._calibrator.init_calibration()

  # ---- fused lowering (this build) ----------------------------------------------
  def kernel_spec(self, held_float: bool = False):
    """Plan fields if numerics + calibration are covered by the fused kernel, else None."""
    if isinstance(self.numerics, no_numerics.NoNumerics):
      return None
    # (a numerics class of the user's own may define kernel_spec() without the argument)
    spec = self.numerics.kernel_spec(True) if held_float else self.numerics.kernel_spec()
    if spec is None or self._calibrator is None or not self._calibrator.kernel_supported():
      return None
    return spec

  def quant_view(self, v: lowering.OperandView, dtype, *, calibration_axes, prescale=None,
                 scale: Optional[torch.Tensor] = None, scale_dtype=None, held_float: bool = False,
                 want_other_axis_absmax: bool = False, absmax_partials: Optional[torch.Tensor] = None):
    """Calibrate + quantize an operand view in one kernel sequence.

    With `scale` (float32, one value per [B, R] entry, holding values of `scale_dtype`) the
    calibration is skipped.  Returns (q [B,R,K], scale float32 [B,R] or [1], scale dtype).
    """
    if scale is None:
      spec = self.kernel_spec(held_float)
    else:
      spec = self.numerics.kernel_spec(True) if held_float else self.numerics.kernel_spec()
    assert spec is not None
    if scale is not None:
      per_tensor = False
    elif self.calib_shared_axes == 'per_tensor':
      per_tensor = True
    else:
      shared = self.calib_shared_axes or calibration_axes
      if sorted(a % len(v.shape) for a in shared) != sorted(v.k_axes):
        raise lowering.NotFused(
            f'calib_shared_axes={shared} differs from the contraction axes {v.k_axes}')
      per_tensor = False
    if scale_dtype is not None:
      sdt = scale_dtype
    else:
      sdt = self._calibrator.dtype if self._calibrator.dtype is not None else dtype
    q, s = lowering.quantize_view(v, spec=spec, compute_dtype=dtype, scale_dtype=sdt,
                                  key=None if self.context is None else self.context.key,
                                  per_tensor=per_tensor, prescale=prescale, scale=scale,
                                  want_other_axis_absmax=want_other_axis_absmax and not per_tensor,
                                  absmax_partials=None if per_tensor else absmax_partials)
    return q, s, sdt

  # ---- reference-shaped API -------------------------------------------------------
  def quant(self, x, *, calibration_axes, tiling_state=None):
    """aqt_quantizer.py:65-77."""
    qt = self.calibrate(x, calibration_axes=calibration_axes, tiling_state=tiling_state)
    return self.calculate_qvalue(x, qt)

  def calibrate(self, x, *, calibration_axes, tiling_state=None) -> aqt_tensor.QTensor:
    """Incomplete QTensor holding only the scale (aqt_quantizer.py:79-157)."""
    replay = _REPLAY.get()
    if replay is not None and id(self) in replay:
      # this quantizer has calibrated this very tensor a moment ago, in the attempt to run the
      # call on the fused kernels: a stateful calibrator must see one update per step, not two
      return replay.pop(id(self))
    if tiling_state is not None:
      x = tiling_state.apply(x)
      _, calibration_axes = tiling_state.to_tiled_axes_transposed(calibration_axes)
    if isinstance(self.numerics, no_numerics.NoNumerics):
      return aqt_tensor.QTensor(qvalue=x, scale=[], scale_t=None, bias=[], dequant_dtype=x.dtype,
                                tiling_state=tiling_state)
    if self.calib_shared_axes == 'per_tensor':
      shared_axes = list(range(x.dim()))
    else:
      shared_axes = self.calib_shared_axes or calibration_axes
    msg = f'{self.calibration = } must be set if {self.numerics = } is not NoNumerics'
    assert self.calibration is not None, msg
    assert self._calibrator is not None, 'forgot self.init_calibration()?'
    scale, bias, sparsity_mask = self._calibrator.get_scale_and_bias_and_sparsity(
        x, shared_axes, self.numerics, self.context)
    out = aqt_tensor.QTensor(qvalue=None, sparsity_mask=sparsity_mask, scale=scale, scale_t=None,
                             bias=bias, dequant_dtype=x.dtype, tiling_state=tiling_state)
    record = _RECORD.get()
    if record is not None:
      record[id(self)] = out
    return out

  def calculate_qvalue(self, x, qt: aqt_tensor.QTensor):
    """Quantize x with the scale in qt (aqt_quantizer.py:159-176)."""
    if isinstance(self.numerics, no_numerics.NoNumerics):
      return qt, None
    spec = self.numerics.kernel_spec()
    if (spec is None or qt.bias or qt.tiling_state is not None or len(qt.scale) != 1
        or qt.sparsity_mask is not None or not x.is_floating_point()):
      return self._calculate_qvalue_stepwise(x, qt)
    try:
      out, quant_grad = self._calculate_qvalue_kernel(x, qt, spec)
    except lowering.NotFused:
      return self._calculate_qvalue_stepwise(x, qt)
    if getattr(self.numerics, 'clip_gradient', False):
      quant_grad = clip_gradient_later(self.numerics, x, qt.scale)
    return out, quant_grad

  def _calculate_qvalue_stepwise(self, x, qt: aqt_tensor.QTensor):
    """No fused scale-and-round kernel for this case: scale, then the numerics' own forward."""
    q_scaled = qt.quant(x)
    x_q, res = self.numerics.vjp_fwd(q_scaled.qvalue, self.context)
    q_scaled.qvalue = x_q
    if self.numerics.get_dtype() is utils.int4:
      q_scaled.container_dtype = utils.int4
    return q_scaled, functools.partial(self.numerics.vjp_bwd, res)

  def _calculate_qvalue_kernel(self, x, qt: aqt_tensor.QTensor, spec):
    (s,) = qt.scale
    shared = [a for a in range(x.dim()) if s.shape[a] == 1 and x.shape[a] > 1]
    rest = [a for a in range(x.dim()) if a not in shared]
    v = lowering.view_operand(x, [], rest, shared)
    per_tensor = s.numel() == 1
    sv = lowering.view_operand(s, [], rest, shared)
    s32 = sv.mem.reshape(-1).float().contiguous()
    s_in = s32.reshape(1) if per_tensor else s32.reshape(1, v.R, 1) if v.k_last else s32.reshape(1, 1, v.R)
    q, _ = lowering.quantize_view(
        v, spec=spec, compute_dtype=x.dtype, scale_dtype=s.dtype,
        key=None if self.context is None else self.context.key, per_tensor=per_tensor, scale=s_in)
    qvalue = lowering.logical_from_brk(_typed(q, spec['out_dtype']), v)
    out = qt.replace(qvalue=qvalue, container_dtype=utils.int4 if spec['out_dtype'] == L.I4 else None)
    return out, functools.partial(self.numerics.vjp_bwd, (None,))


def clip_gradient_later(numerics, x, scale_list):
  """The gradient function of a numerics with clip_gradient for an input the fused kernel quantized:
  the kernel keeps no scaled copy of x (the residual the reference's vjp_bwd reads,
  numerics/int_numerics.py:113-125), so the scaled input is recomputed from x and the scale
  when the backward pass asks, with QTensor.quant's own arithmetic (aqt_tensor.py:125-159)."""
  def quant_grad(grad):
    scaled = aqt_tensor.QTensor(qvalue=None, scale=scale_list, scale_t=None, bias=[],
                                dequant_dtype=x.dtype).quant(x.detach()).qvalue
    return numerics.vjp_bwd((scaled,), grad)
  return quant_grad


def _typed(q: torch.Tensor, out_dtype: int) -> torch.Tensor:
  if out_dtype == L.E4M3:
    return q.view(torch.float8_e4m3fn)
  if out_dtype == L.E5M2:
    return q.view(torch.float8_e5m2)
  return q


def quantizer_make(n_bits, preserve_max_val: bool = False, initialize_calibration: bool = True,
                   scale_stop_grad: bool = True, scale_dtype=None) -> Quantizer:
  """aqt_quantizer.py:179-206."""
  effective_numerics = numerics_utils.get_numerics(n_bits, preserve_max_val)
  calibration_cls = None if n_bits is None else calibration.AbsMaxCalibration
  quantizer = Quantizer(numerics=effective_numerics, calib_shared_axes=None,
                        scale_stop_grad=scale_stop_grad, scale_dtype=scale_dtype,
                        calibration=calibration_cls, context=utils.Context(key=None, train_step=None))
  if initialize_calibration:
    quantizer.init_calibration()
  return quantizer


def make_fake_quant(quantizer: Quantizer, calibration_axes=None):
  """aqt_quantizer.py:209-214."""
  def fake_quant(x):
    x_q, _ = quantizer.quant(x, calibration_axes=calibration_axes)
    return x_q.dequant()
  return fake_quant

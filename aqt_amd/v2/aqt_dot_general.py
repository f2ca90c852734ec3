"""Quantized dot_general (mirrors aqt/jax/v2/aqt_dot_general.py) on HIP kernels.

Same configuration dataclasses, call signatures and assertion behaviour as the
reference; the arithmetic of one `DotGeneralRaw.__call__` is lowered to
  quantize(lhs) , quantize(rhs)  ->  MFMA contraction with fused dequantisation
(see lowering.py, csrc/quantize.hip, csrc/gemm_i8.hip).  Differentiation uses a
torch.autograd.Function in place of jax.custom_vjp.
"""
from __future__ import annotations

import abc
import contextvars
import dataclasses
import enum
import functools
import math
import os
import weakref
from typing import Any, Optional, Sequence

import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import aqt_quantizer
from aqt_amd.v2 import aqt_tensor
from aqt_amd.v2 import lowering
from aqt_amd.v2 import transpose
from aqt_amd.v2 import utils
from aqt_amd.v2.numerics import fp8_numerics
from aqt_amd.v2.numerics import int_numerics
from aqt_amd.v2.numerics import no_numerics

dtypes_allowed_for_int32_accum = [utils.int4, utils.int8]


class CalibrationMode(enum.Enum):
  """aqt_dot_general.py:51-55."""
  CONTRACTING_AXIS = 1
  REMAINING_AXIS = 2


class DequantMode(enum.Enum):
  """aqt_dot_general.py:58-70."""
  OUTPUT = 1
  THIS_INPUT = 2
  OTHER_INPUT = 3


@dataclasses.dataclass(kw_only=True)
class Tensor:
  """Configuration of quantization of one side of the op (aqt_dot_general.py:73-85)."""
  use_fwd_quant: bool = False
  dequant_mode: DequantMode = DequantMode.OUTPUT
  calibration_mode: CalibrationMode = CalibrationMode.CONTRACTING_AXIS

  def __deepcopy__(self, memo):
    return utils.deepcopy_fields(self, memo, shared=('use_fwd_quant', 'dequant_mode', 'calibration_mode'))


@dataclasses.dataclass(kw_only=True)
class LocalAqt:
  """aqt_dot_general.py:88-96."""
  contraction_axis_shard_count: Optional[int] = None
  contraction_axis_shard_size: Optional[int] = None
  tile_largest_shape: bool = False

  def __deepcopy__(self, memo):
    return utils.deepcopy_fields(self, memo, shared=(
        'contraction_axis_shard_count', 'contraction_axis_shard_size', 'tile_largest_shape'))


_FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)

# Weight-only quantization (a float lhs against an int8 / fp8 rhs) promotes the rhs to the float dtype on
# every call; for a frozen weight that is the same conversion every time, so large converted copies are
# kept for as long as the quantized tensor lives and stays unchanged (its version counter).
_PROMOTED_RHS = {}  # id(rhs) -> (key, promoted [b, k, n] copy), oldest first
# The copies cost 2 (bf16) or 4 bytes per weight element on top of the quantized tensor; together they are kept
# below this many bytes (the oldest go first), and none is made while gradients are being recorded (a quantized
# residual of a training step is not a frozen weight).
PROMOTED_RHS_MAX_BYTES = 8 << 30
# Longest tile for which the activation quantizer writes every 8 k in even-odd order (the row kernels hold a
# segment in registers up to this length).
_EVEN_ODD8_MAX_GROUP = 16384

# Weight-only serving above 64 lhs rows: False (the default) = this library's weight-only contraction kernel,
# which widens the int8 bytes in registers and keeps no float copy of the weight (1090-1170 TFLOP/s from 1024
# rows on against a 4096 x 14336 weight); True = the vendor library's bf16 product on a float copy of the weight
# kept next to the quantized tensor (2 bytes per weight element more; 1320-1490 TFLOP/s on the same shapes): a
# trade of weight memory for 20-25 % of prefill time that the caller has to ask for
# (AQTX_WEIGHT_ONLY_FLOAT_COPY=1 in the environment does so for a whole process).
WEIGHT_ONLY_FLOAT_COPY = os.environ.get('AQTX_WEIGHT_ONLY_FLOAT_COPY', '') == '1'


def _promoted_rhs(rhs, perm, shape, common):
  if rhs.dtype == common or rhs.numel() < (1 << 20) or rhs.requires_grad or torch.is_grad_enabled():
    return rhs.permute(perm).reshape(shape).to(common)
  # the storage address is part of the key: writes through .data or set_() do not move the version counter
  key = (perm, tuple(rhs.shape), common, rhs._version, rhs.data_ptr())
  hit = _PROMOTED_RHS.get(id(rhs))
  if hit is not None and hit[0] == key:
    return hit[1]
  out = rhs.permute(perm).reshape(shape).to(common)
  if hit is None:
    weakref.finalize(rhs, _PROMOTED_RHS.pop, id(rhs), None)
  _PROMOTED_RHS.pop(id(rhs), None)
  nbytes = lambda t: t.numel() * t.element_size()
  total = sum(nbytes(v[1]) for v in _PROMOTED_RHS.values()) + nbytes(out)
  for old in list(_PROMOTED_RHS):
    if total <= PROMOTED_RHS_MAX_BYTES:
      break
    total -= nbytes(_PROMOTED_RHS.pop(old)[1])
  if nbytes(out) <= PROMOTED_RHS_MAX_BYTES:
    _PROMOTED_RHS[id(rhs)] = (key, out)
  return out


def lax_dot_general(lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None):
  """dot_general with lax semantics (output axes: batch, lhs remaining, rhs remaining).

  Stands in for `jax.lax.dot_general` as the default `DotGeneralRaw.dot_general`.  int8 x int8
  and fp8 x fp8 operands go to the MFMA contraction kernels and come back as raw int32 /
  float32 accumulators; float operands (unquantized sides, fake quantization) go to the
  library GEMM through torch.  An int8 operand next to a float one is promoted to the float
  dtype first, as jnp's type promotion does.
  """
  del precision
  (lca, rca), (lba, rba) = dimension_numbers
  lca, rca, lba, rba = list(lca), list(rca), list(lba), list(rba)
  lra = utils.get_remaining_axes(lhs.dim(), lca, lba)
  rra = utils.get_remaining_axes(rhs.dim(), rca, rba)
  bshape = [lhs.shape[a] for a in lba]
  mshape = [lhs.shape[a] for a in lra]
  nshape = [rhs.shape[a] for a in rra]
  kdim = 1
  for a in lca:
    kdim *= lhs.shape[a]
  b = 1
  for s in bshape:
    b *= s
  lt = lhs.permute(tuple(lba + lra + lca)).reshape(b, -1, kdim)
  both_int = lhs.dtype == torch.int8 and rhs.dtype == torch.int8
  both_fp8 = lhs.dtype in _FP8_DTYPES and rhs.dtype in _FP8_DTYPES
  if both_int or both_fp8:
    # the kernels take both operands with the contraction axis innermost
    rt = rhs.permute(tuple(rba + rra + rca)).reshape(b, -1, kdim)
    m, n = lt.shape[1], rt.shape[1]
    acc_dtype = torch.int32 if both_int else torch.float32
    if both_int:
      assert preferred_element_type == torch.int32, (
          f'{preferred_element_type=}: int8 operands are contracted into int32 accumulators only')
    if b * m * n == 0 or kdim == 0:
      out = torch.zeros((b, m, n), dtype=acc_dtype, device=lhs.device)
    else:
      kd = lambda t: {torch.int8: L.I8, torch.float8_e4m3fn: L.E4M3, torch.float8_e5m2: L.E5M2}[t.dtype]
      raw = lambda t: t.contiguous() if t.dtype == torch.int8 else t.contiguous().view(torch.uint8)
      out = ops.gemm(raw(lt), raw(rt), row_scale=None, col_scale=None, out_dtype=acc_dtype,
                     a_dtype=kd(lt), b_dtype=kd(rt))
  else:
    common = torch.promote_types(lhs.dtype, rhs.dtype)
    pet = preferred_element_type
    if pet is not None and pet.is_floating_point and common.is_floating_point and (
        torch.finfo(pet).bits > torch.finfo(common).bits):
      common = pet  # wider accumulator asked for: keep its precision in the result
    rt = _promoted_rhs(rhs, tuple(rba + rca + rra), (b, kdim, -1), common)
    out = torch.matmul(lt.to(common), rt)
  out = out.reshape(bshape + mshape + nshape)
  if preferred_element_type is not None:
    out = out.to(preferred_element_type)
  return out


class DotGeneralQuantizer(abc.ABC):
  """Plugin point for operand quantization (aqt_dot_general.py:331-422)."""

  @abc.abstractmethod
  def init_calibration(self):
    pass

  @abc.abstractmethod
  def calibrate(self, lhs, rhs, dimension_numbers, lhs_mode, rhs_mode):
    pass

  @abc.abstractmethod
  def calculate_qvalue(self, lhs, lhs_qt, rhs, rhs_qt):
    pass

  @abc.abstractmethod
  def swap_lhs_and_rhs(self) -> None:
    pass

  @abc.abstractmethod
  def assert_calib_shared_axes_value(self, lhs_val, rhs_val, msg: str) -> None:
    pass

  @abc.abstractmethod
  def set_context(self, lhs_context, rhs_context) -> None:
    pass

  def __call__(self, lhs_quantization_info, rhs_quantization_info):
    """Calibrate then quantize (aqt_dot_general.py:334-360)."""
    lhs_input, lhs_ca = lhs_quantization_info
    rhs_input, rhs_ca = rhs_quantization_info
    dn = ((lhs_ca, rhs_ca), ((), ())) if lhs_ca is not None else None
    (lhs, lhs_qt), (rhs, rhs_qt) = self.calibrate(
        lhs_input, rhs_input, dn, CalibrationMode.CONTRACTING_AXIS, CalibrationMode.CONTRACTING_AXIS)
    return self.calculate_qvalue(lhs, lhs_qt, rhs, rhs_qt)


@dataclasses.dataclass(kw_only=True)
class DefaultDotGeneralQuantizer(DotGeneralQuantizer):
  """Default dot_general quantizer (aqt_dot_general.py:427-595)."""

  lhs: aqt_quantizer.Quantizer
  rhs: aqt_quantizer.Quantizer
  lhs_mid: aqt_quantizer.Quantizer
  rhs_mid: aqt_quantizer.Quantizer
  lhs_mid_alpha: Optional[float] = None
  rhs_mid_alpha: Optional[float] = None
  skip_mid_scales: bool = True

  def __deepcopy__(self, memo):
    return utils.deepcopy_fields(self, memo, shared=('lhs_mid_alpha', 'rhs_mid_alpha', 'skip_mid_scales'))

  def init_calibration(self):
    self.lhs.init_calibration()
    self.rhs.init_calibration()
    if self.lhs_mid_alpha is not None:
      self.lhs_mid.init_calibration()
    if self.rhs_mid_alpha is not None:
      self.rhs_mid.init_calibration()

  def calibrate(self, lhs, rhs, dimension_numbers, lhs_mode, rhs_mode):
    """aqt_dot_general.py:464-559."""
    if dimension_numbers is not None:
      (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = dimension_numbers
      lhs_ra = utils.get_remaining_axes(lhs.dim(), lhs_ca, lhs_ba)
      rhs_ra = utils.get_remaining_axes(rhs.dim(), rhs_ca, rhs_ba)

      def axes(mode, ndim, ca, ba):
        if mode == CalibrationMode.REMAINING_AXIS:
          m = 'mid-quantization is not supported for REMAINING_AXIS mode'
          assert self.lhs_mid_alpha is None and self.rhs_mid_alpha is None, m
          return utils.get_remaining_axes(ndim, ca, ba)
        if mode == CalibrationMode.CONTRACTING_AXIS:
          return ca
        raise ValueError(f'Unknown calibration mode: {mode}')

      lhs_axes = axes(lhs_mode, lhs.dim(), lhs_ca, lhs_ba)
      rhs_axes = axes(rhs_mode, rhs.dim(), rhs_ca, rhs_ba)
    else:
      lhs_ra = rhs_ra = None
      lhs_axes = rhs_axes = None

    if self.lhs_mid_alpha is None and self.rhs_mid_alpha is None:
      lhs_qt = self.lhs.calibrate(lhs, calibration_axes=lhs_axes)
      rhs_qt = self.rhs.calibrate(rhs, calibration_axes=rhs_axes)
      return ((lhs, lhs_qt), (rhs, rhs_qt))

    # "Middle" scales (SmoothQuant, AWQ): part of each side's per-contraction-channel scale moves
    # to the other side before the usual calibration.  Elementwise tensor arithmetic around the
    # abs-max kernel.
    def dezero(x):
      return torch.where(x == 0.0, torch.ones_like(x), x)

    def mid(quantizer, x, ra, alpha, transpose_fn, other_shape):
      if alpha is None:
        return 1.0, 1.0
      assert quantizer is not None
      qt = quantizer.calibrate(x, calibration_axes=ra)
      assert len(qt.scale) == 1, 'you must set some numerics'
      scale = dezero(qt.scale[0])
      # x ** alpha; the two usual exponents avoid the device pow (a few ulp off)
      scale = scale if alpha == 1.0 else torch.sqrt(scale) if alpha == 0.5 else scale ** alpha
      return scale, transpose_fn(scale, dimension_numbers, other_shape)

    lhs_mid_scale, lhs_mid_scale_t = mid(self.lhs_mid, lhs, lhs_ra, self.lhs_mid_alpha,
                                         transpose.lhs_scale_transpose_for_rhs_input, rhs.shape)
    rhs_mid_scale, rhs_mid_scale_t = mid(self.rhs_mid, rhs, rhs_ra, self.rhs_mid_alpha,
                                         transpose.rhs_scale_transpose_for_lhs_input, lhs.shape)
    lhs_mid_scale_combined = lhs_mid_scale / rhs_mid_scale_t
    rhs_mid_scale_combined = rhs_mid_scale / lhs_mid_scale_t
    lhs_mid = lhs / lhs_mid_scale_combined
    rhs_mid = rhs / rhs_mid_scale_combined
    lhs_qt = self.lhs.calibrate(lhs_mid, calibration_axes=lhs_axes)
    rhs_qt = self.rhs.calibrate(rhs_mid, calibration_axes=rhs_axes)
    assert lhs_qt.scale is not None
    assert rhs_qt.scale is not None
    if not self.skip_mid_scales:
      lhs_qt.scale.append(lhs_mid_scale_combined)
      rhs_qt.scale.append(rhs_mid_scale_combined)
    return ((lhs, lhs_qt), (rhs, rhs_qt))

  def calculate_qvalue(self, lhs, lhs_qt, rhs, rhs_qt):
    """aqt_dot_general.py:561-575."""
    lhs_qt, lhs_grad = self.lhs.calculate_qvalue(lhs, lhs_qt)
    rhs_qt, rhs_grad = self.rhs.calculate_qvalue(rhs, rhs_qt)
    return (lhs_qt, lhs_grad), (rhs_qt, rhs_grad)

  def swap_lhs_and_rhs(self) -> None:
    self.lhs, self.rhs = self.rhs, self.lhs

  def assert_calib_shared_axes_value(self, lhs_val, rhs_val, msg: str) -> None:
    assert self.lhs.calib_shared_axes == lhs_val, msg
    assert self.rhs.calib_shared_axes == rhs_val, msg

  def set_context(self, lhs_context, rhs_context) -> None:
    self.lhs.context = lhs_context
    self.rhs.context = rhs_context


def _quant(lhs, rhs, lhs_qt, rhs_qt, dg_quantizer, lhs_cfg, rhs_cfg, dimension_numbers,
           allow_dummy_gradient_into_qtensor):
  """quant() below, also returning the operands as the quantizer's calibrate step left them."""
  (lhs, lhs_incomplete), (rhs, rhs_incomplete) = dg_quantizer.calibrate(
      lhs, rhs, dimension_numbers, lhs_cfg.calibration_mode, rhs_cfg.calibration_mode)
  if lhs_qt is not None and not lhs_qt.is_full():
    lhs_incomplete, lhs_qt = lhs_qt, None  # an incomplete QTensor (scales only) was handed in
  if rhs_qt is not None and not rhs_qt.is_full():
    rhs_incomplete, rhs_qt = rhs_qt, None
  (lhs_calc, lhs_grad), (rhs_calc, rhs_grad) = dg_quantizer.calculate_qvalue(lhs, lhs_incomplete, rhs, rhs_incomplete)

  def postprocess(given, calculated, quant_grad):
    if given is None:
      return calculated, quant_grad
    return given, (quant_grad if allow_dummy_gradient_into_qtensor else _POISON)

  return postprocess(lhs_qt, lhs_calc, lhs_grad), postprocess(rhs_qt, rhs_calc, rhs_grad), (lhs, rhs)


def quant(lhs, rhs, lhs_qt, rhs_qt, dg_quantizer, lhs_cfg, rhs_cfg, dimension_numbers,
          allow_dummy_gradient_into_qtensor):
  """Quantizes lhs and rhs with dg_quantizer (aqt_dot_general.py:598-672): calibrate, take over
  scales handed in as incomplete QTensors, compute the qvalues, and keep a QTensor that was
  handed in whole (its gradient function is then poisoned unless dummy gradients are allowed).
  Returns ((lhs_qt, lhs_quant_grad), (rhs_qt, rhs_quant_grad))."""
  l, r, _ = _quant(lhs, rhs, lhs_qt, rhs_qt, dg_quantizer, lhs_cfg, rhs_cfg, dimension_numbers,
                   allow_dummy_gradient_into_qtensor)
  return l, r


def dot_general_raw_make(lhs_bits=None, rhs_bits=None, local_aqt=None, jax_scope_name='aqt',
                         initialize_calibration=True, allow_dummy_gradients=False) -> 'DotGeneralRaw':
  """aqt_dot_general.py:99-156."""
  lhs_cfg, rhs_cfg = Tensor(), Tensor()
  if (isinstance(lhs_bits, int) and 2 <= lhs_bits <= 8 and isinstance(rhs_bits, int)
      and 2 <= rhs_bits <= 8):
    dg_accumulator_dtype = utils.int32
  elif lhs_bits in fp8_numerics.fp8_map and rhs_bits in fp8_numerics.fp8_map:
    dg_accumulator_dtype = utils.float32
  else:
    dg_accumulator_dtype = None
  mk = functools.partial(aqt_quantizer.quantizer_make, initialize_calibration=initialize_calibration)
  dg_quantizer = DefaultDotGeneralQuantizer(lhs=mk(lhs_bits), rhs=mk(rhs_bits), lhs_mid=mk(None),
                                            rhs_mid=mk(None))
  return DotGeneralRaw(lhs=lhs_cfg, rhs=rhs_cfg, dg_quantizer=dg_quantizer,
                       dg_accumulator_dtype=dg_accumulator_dtype, local_aqt=local_aqt,
                       jax_scope_name=jax_scope_name,
                       allow_dummy_gradient_into_qtensor=allow_dummy_gradients)


def dot_general_make(lhs_bits=None, rhs_bits=None, bwd_bits=None, use_fwd_quant: bool = True,
                     dlhs_local_aqt=None, drhs_local_aqt=None,
                     allow_dummy_gradients: bool = False) -> 'DotGeneral':
  """aqt_dot_general.py:161-203."""
  fwd = dot_general_raw_make(lhs_bits, rhs_bits, jax_scope_name='aqt_fwd',
                             initialize_calibration=False, allow_dummy_gradients=allow_dummy_gradients)
  dlhs = dot_general_raw_make(bwd_bits, bwd_bits, local_aqt=dlhs_local_aqt, jax_scope_name='aqt_dlhs',
                              initialize_calibration=False, allow_dummy_gradients=allow_dummy_gradients)
  drhs = dot_general_raw_make(bwd_bits, bwd_bits, local_aqt=drhs_local_aqt, jax_scope_name='aqt_drhs',
                              initialize_calibration=False, allow_dummy_gradients=allow_dummy_gradients)
  cfg = DotGeneral(fwd=fwd, dlhs=dlhs, drhs=drhs)
  # Surprising: lhs quantization determines what drhs can do.
  if lhs_bits is not None:
    cfg.drhs.rhs.use_fwd_quant = use_fwd_quant
  if rhs_bits is not None:
    cfg.dlhs.rhs.use_fwd_quant = use_fwd_quant
  assert cfg.fwd.local_aqt is None, 'local_aqt is not yet supported in fwd.'
  return cfg


@dataclasses.dataclass(kw_only=True)
class MultiTensor:
  """aqt_dot_general.py:209-213."""
  x: Any
  qx: aqt_tensor.QTensor


@dataclasses.dataclass(kw_only=True)
class TensorRes:
  """What the forward pass hands to the backward pass (aqt_dot_general.py:215-220)."""
  mt: MultiTensor
  quant_grad: Any


@dataclasses.dataclass(kw_only=True)
class DotGeneralRes:
  lhs: TensorRes
  rhs: TensorRes


def _parse_einsum(eqn: str):
  ins, out = eqn.replace(' ', '').split('->')
  l, r = ins.split(',')
  return l, r, out


def einsum(eqn: str, lhs, rhs, dg=lax_dot_general):
  """Two-operand einsum through an injectable dot_general (aqt_dot_general.py:229-241).

  Letters shared by both operands and the output are batch axes, letters shared by
  the operands only are contracted; the dot_general output (batch, lhs free, rhs
  free) is then permuted to the requested order.  Like jnp.einsum, the operands are
  handed over as (rhs, lhs) when the output is exactly (batch, rhs free, lhs free).
  """
  l, r, out = _parse_einsum(eqn)
  assert len(set(l)) == len(l) and len(set(r)) == len(r), 'repeated indices are not supported'
  batch = [c for c in l if c in r and c in out]
  contract = [c for c in l if c in r and c not in out]
  lfree = [c for c in l if c not in r]
  rfree = [c for c in r if c not in l]
  for c in lfree + rfree:
    assert c in out, 'summing a free index is not supported'
  if batch + rfree + lfree == list(out):
    # jnp.einsum tries (rhs, lhs) first and keeps that order when it needs no transpose
    # afterwards; callers (AqtEinsum) mirror the swap in their per-side settings.
    dn = ((tuple(r.index(c) for c in contract), tuple(l.index(c) for c in contract)),
          (tuple(r.index(c) for c in batch), tuple(l.index(c) for c in batch)))
    return dg(rhs, lhs, dn, None, None)
  dn = ((tuple(l.index(c) for c in contract), tuple(r.index(c) for c in contract)),
        (tuple(l.index(c) for c in batch), tuple(r.index(c) for c in batch)))
  res = dg(lhs, rhs, dn, None, None)
  names = batch + lfree + rfree
  perm = [names.index(c) for c in out]
  if perm != list(range(len(perm))):
    res = res.permute(tuple(perm))
  return res


def _get_scale_t(qt, transpose_fn, dimension_numbers, lhs_shape, rhs_shape):
  return [transpose_fn(s, dimension_numbers, lhs_shape, rhs_shape) for s in qt.scale]


def _local_aqt_split(local_aqt, shape, ca, ba):
  """Which contraction axis LocalAqt splits, and into what (aqt_dot_general.py:259-328).

  Returns (axis, shard_count, shard_size, new_ca, new_ba) or None without contraction axes:
  the axis becomes (shard_count, shard_size) in place, the shard-count axis is the new leading
  batch axis and the shard-size axis stays a contraction axis.  With tile_largest_shape the
  (first) largest contraction axis is split into shards of contraction_axis_shard_size, else
  the first contraction axis into contraction_axis_shard_count shards.
  """
  ca, ba = list(ca), list(ba)
  if local_aqt.tile_largest_shape:
    msg = 'When tile_largest_shape is True, must set shard_size.'
    assert local_aqt.contraction_axis_shard_size is not None, msg
    assert local_aqt.contraction_axis_shard_count is None, msg
  else:
    msg = 'You are using the original local aqt. Please only set shard_count.'
    assert local_aqt.contraction_axis_shard_count is not None, msg
    assert local_aqt.contraction_axis_shard_size is None, msg
  if not ca:
    return None
  if local_aqt.tile_largest_shape:
    extent = max(shape[a] for a in ca)
    axis = list(shape).index(extent)   # the reference looks the extent up in the whole shape
    assert axis in ca, 'the largest contraction extent also occurs on an earlier, non-contraction axis'
    size = local_aqt.contraction_axis_shard_size
    assert extent % size == 0
    count = extent // size
  else:
    axis = ca[0]
    count = local_aqt.contraction_axis_shard_count
    assert shape[axis] % count == 0
    size = shape[axis] // count
  new_ca = [a + (a >= axis) for a in ca]
  new_ba = [axis] + [a + (a > axis) for a in ba]
  return axis, count, size, new_ca, new_ba


def _split_axis(x, axis, count, size):
  """Reshapes axis `axis` of x into (count, size); an extent-1 axis (a keepdims scale) into (1, 1)."""
  shape = list(x.shape)
  shape[axis:axis + 1] = [count, size] if shape[axis] != 1 else [1, 1]
  return x.reshape(shape)


def _apply_local_aqt(local_aqt, lhs, rhs, dimension_numbers):
  """Both operands with the contraction axis sharded, and the matching dimension numbers.

  lhs may be a deferred `g * scale_t` (_Prescaled) and rhs a quantized residual (QTensor):
  their payloads are reshaped alike.
  """
  (lca, rca), (lba, rba) = dimension_numbers

  def one(x, ca, ba):
    arr = x.x if isinstance(x, _Prescaled) else x.qvalue if isinstance(x, aqt_tensor.QTensor) else x
    plan = _local_aqt_split(local_aqt, tuple(arr.shape), ca, ba)
    if plan is None:
      return x, list(ca), list(ba)
    axis, count, size, new_ca, new_ba = plan
    if isinstance(x, _Prescaled):
      x = _Prescaled(x=_split_axis(x.x, axis, count, size), scale_t=_split_axis(x.scale_t, axis, count, size))
    elif isinstance(x, aqt_tensor.QTensor):
      x = x.replace(qvalue=_split_axis(x.qvalue, axis, count, size),
                    scale=[_split_axis(sc, axis, count, size) for sc in x.scale])
    else:
      x = _split_axis(x, axis, count, size)
    return x, new_ca, new_ba

  lhs, lca, lba = one(lhs, lca, lba)
  rhs, rca, rba = one(rhs, rca, rba)
  return lhs, rhs, ((lca, rca), (lba, rba))


# A frozen operand that arrives in another memory order than the kernels read (e.g. a weight
# restored from a checkpoint in its logical [K, N] order) is re-laid out once, not on every call:
# the copy is remembered for as long as the frozen tensor itself lives.
_KERNEL_LAYOUT_CACHE = {}   # id(frozen tensor) -> (key, re-laid-out copy); entries die with the tensor


def _kernel_layout_of(qvalue: torch.Tensor, v: 'lowering.OperandView', pack_int4: bool = False,
                      fragments: bool = False) -> torch.Tensor:
  """The operand as the kernels read it ([B, R, K], contraction axis contiguous); with
  pack_int4 additionally packed two values per byte ([B, R, K/2] uint8), which halves the bytes
  a serving call streams from HBM; with fragments (B = 1 only) further re-laid in MFMA fragment
  order (ops.tile_weight: a flat buffer), which the serving kernels stream 20-25 % faster.
  Copies are made once per frozen tensor and kept as long as it lives."""
  key = (tuple(v.b_axes), tuple(v.r_axes), tuple(v.k_axes), qvalue._version)
  slot = (pack_int4, fragments)
  hit = _KERNEL_LAYOUT_CACHE.get(id(qvalue))
  if hit is not None and hit[0] == key and slot in hit[1]:
    return hit[1][slot]
  def rows():
    r = v.mem if v.k_last else v.mem.transpose(1, 2).contiguous()
    return ops.pack_i4(r.contiguous()) if pack_int4 else r
  if fragments:
    # from the rows copy if one is kept already, else from a passing one: the fragment order is then the
    # only copy of the weight next to the caller's own
    base = hit[1].get((pack_int4, False)) if hit is not None and hit[0] == key else None
    base = base if base is not None else rows()
    assert base.shape[0] == 1
    q = ops.tile_weight(base[0].contiguous(), L.I4P if pack_int4 else L.I8)
  else:
    q = rows()
  hit = _KERNEL_LAYOUT_CACHE.get(id(qvalue))
  if hit is None:
    weakref.finalize(qvalue, _KERNEL_LAYOUT_CACHE.pop, id(qvalue), None)
  if hit is None or hit[0] != key:
    hit = (key, {})
    _KERNEL_LAYOUT_CACHE[id(qvalue)] = hit
  hit[1][slot] = q
  return q


def _scale_f32(scale: torch.Tensor) -> torch.Tensor:
  """A frozen operand's scale in float32, same shape.  A scale kept in another dtype is converted
  once per tensor, not on every call."""
  src = getattr(scale, 'f32_copy', None)
  if src is None:
    src = scale
  if src.dtype != torch.float32:
    key = ('scale_f32', scale._version)
    hit = _KERNEL_LAYOUT_CACHE.get(id(scale))
    if hit is not None and hit[0] == key:
      src = hit[1]
    else:
      src = scale.float()
      if hit is None:
        weakref.finalize(scale, _KERNEL_LAYOUT_CACHE.pop, id(scale), None)
      _KERNEL_LAYOUT_CACHE[id(scale)] = (key, src)
  return src


def _scale_vector_f32(scale: torch.Tensor, ba, ra, ca) -> torch.Tensor:
  """A frozen operand's scale as the flat float32 vector the kernels read."""
  return lowering.view_operand(_scale_f32(scale), ba, ra, ca).mem.reshape(-1).contiguous()


_POISON = ('Poison. Gradients are not generally expected in serving. Please set '
           'allow_dummy_gradient_into_qtensor to True if this is the intended behavior.')


@dataclasses.dataclass(kw_only=True)
class _Prescaled:
  """`lhs * scale_t` of _maybe_use_fwd_quant, deferred so the quantize kernel can fuse it."""
  x: Any
  scale_t: Any


def _maybe_use_fwd_quant(lhs, rhs: MultiTensor, dimension_numbers, use_fwd_quant: bool):
  """aqt_dot_general.py:675-729.  Returns (lhs | _Prescaled, rhs array)."""
  scale_count = -1
  if rhs.qx.scale is not None:
    scale_count = len(rhs.qx.scale)
  msg = (f'Found use_fwd_quant is {use_fwd_quant} in bwd. It is supported only if there is '
         f'exactly one scale in a good shape.\n{scale_count=}')
  if use_fwd_quant:
    assert scale_count == 1, msg
    if rhs.qx.bias:
      raise NotImplementedError('Quantization biases are not supported in forward quantization.')
    # the float32 copy of the scale, when the quantizer left one, spares a cast launch
    scale0 = getattr(rhs.qx.scale[0], 'f32_copy', None)
    if scale0 is None:
      scale0 = rhs.qx.scale[0]
    scale_t = transpose.rhs_scale_transpose_for_lhs_input(scale0, dimension_numbers, lhs.shape)
    lhs = _Prescaled(x=lhs, scale_t=scale_t)
    # The quantized residual is quantized again; the kernel reads the int8/fp8 values as
    # floats of the dequant dtype (qvalue.astype(dequant_dtype) in the reference).
    rhs_arr = rhs.qx
  else:
    rhs_arr = rhs.x
  return lhs, rhs_arr


def _canonical_pairs(lhs, rhs, dimension_numbers):
  """Orders the contraction and batch axis pairs by lhs memory position.

  The pairing is what matters to dot_general; the listed order only fixes the order of
  batch axes in the output, which the caller restores.
  """
  (lca, rca), (lba, rba) = dimension_numbers
  del rhs
  order, _ = lowering.memory_rank(lhs)
  pos = {a: i for i, a in enumerate(order)}

  def sort_pairs(la, ra):
    pairs = sorted(zip(la, ra), key=lambda p: (pos.get(p[0], 10**6), p[0]))
    return [p[0] for p in pairs], [p[1] for p in pairs]

  lca2, rca2 = sort_pairs(list(lca), list(rca))
  lba2, rba2 = sort_pairs(list(lba), list(rba))
  return ((lca2, rca2), (lba2, rba2))


_NotFused = lowering.NotFused

# (lhs, rhs): whether the forward quantizers of this call should leave, next to the values they write, the partial
# maxima with which the backward pass calibrates those values over the other axis (DotGeneralRaw._quant_side); set
# by the differentiable entry point for the operands whose residual a backward contraction re-quantizes.
_RESIDUAL_ABSMAX: 'contextvars.ContextVar' = contextvars.ContextVar('aqt_residual_absmax', default=(False, False))
# False (AQTX_RESIDUAL_ABSMAX=0 in the environment): the backward pass reads the residuals for their abs-max; same results
RESIDUAL_ABSMAX = os.environ.get('AQTX_RESIDUAL_ABSMAX', '1') != '0'


def _ragged_sizes(dot_general_hook):
  """The group sizes of a ragged-contraction hook (aqt_ragged_dot.RaggedDot), else None."""
  if getattr(dot_general_hook, 'is_ragged_dot', False):
    return dot_general_hook.group_sizes
  return None


@dataclasses.dataclass(kw_only=True)
class DotGeneralRaw:
  """Configuration of quantization of one dot_general without gradient (aqt_dot_general.py:732-749)."""

  lhs: Tensor
  rhs: Tensor
  dg_quantizer: DotGeneralQuantizer
  dg_accumulator_dtype: Any
  local_aqt: Optional[LocalAqt]
  jax_scope_name: str
  allow_dummy_gradient_into_qtensor: bool = False
  dot_general: Any = lax_dot_general

  def __deepcopy__(self, memo):
    # the accumulator dtype tag, the scope name and the inner dot_general (a function) are shared
    return utils.deepcopy_fields(self, memo, shared=(
        'dg_accumulator_dtype', 'jax_scope_name', 'allow_dummy_gradient_into_qtensor', 'dot_general'))

  @classmethod
  def make(cls, *args, **kwargs):
    return dot_general_raw_make(*args, **kwargs)

  # ------------------------------------------------------------------------------
  def __call__(self, lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, _out_transpose_axes=None, _bwd_memo=None):
    """A quantized dot_general without custom gradient (aqt_dot_general.py:757-840).

    Returns (out, DotGeneralRes).  `rhs` may be a MultiTensor (bwd calls).
    `_out_transpose_axes` (this build): the caller is going to transpose the result with these
    axes; when that transpose merely swaps the lhs-remaining and rhs-remaining groups the
    contraction kernel writes the transposed result directly and `out` comes back already
    transposed (and contiguous).  `_bwd_memo` (this build): a dict owned by one backward pass, in
    which its two contractions share per-tensor scales of the gradient.
    """
    with torch.profiler.record_function(self.jax_scope_name):
      if isinstance(rhs, MultiTensor):
        lhs, rhs = _maybe_use_fwd_quant(lhs, rhs, dimension_numbers, self.rhs.use_fwd_quant)
      if self.local_aqt is None:
        return self._dispatch(lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, _out_transpose_axes, _bwd_memo)
      # LocalAqt (aqt_dot_general.py:773-776, 833-837): every shard of the contraction axis is
      # calibrated and contracted on its own (the shard axis is a leading batch axis), the
      # dequantized shard outputs are summed; no residuals come back.
      msg = 'Custom calib_shared_axes not implemented for local AQT.'
      if isinstance(self.dg_quantizer, DefaultDotGeneralQuantizer):
        self.dg_quantizer.assert_calib_shared_axes_value(None, None, msg)
      n_ca = len(dimension_numbers[0][0])
      assert n_ca == len(dimension_numbers[0][1])
      lhs, rhs, dn = _apply_local_aqt(self.local_aqt, lhs, rhs, dimension_numbers)
      out, _ = self._dispatch(lhs, rhs, lhs_qt, rhs_qt, dn, None, _bwd_memo)
      if n_ca > 0:
        out = ops.sum_tiles(out.contiguous())
      if _out_transpose_axes is not None:
        out = out.permute(tuple(_out_transpose_axes))
      return out, None

  def _dispatch(self, lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, out_transpose_axes, bwd_memo=None):
    """The lowered paths where they implement the configuration (_lowered_call: the int8 / fp8 kernels for
    the default modes, _float_contraction for the modes that contract in float), the step-by-step path
    otherwise."""
    # a ragged (grouped) contraction hook is lowered too: same kernels, rows looked up per group
    fusable = ((self.dot_general is lax_dot_general or _ragged_sizes(self.dot_general) is not None)
               and type(self.dg_quantizer) is DefaultDotGeneralQuantizer)  # pylint: disable=unidiomatic-typecheck
    calibrated = {}  # id(quantizer) -> scales found step by step during the fused attempt
    if fusable:
      try:
        return self._lowered_call(lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, out_transpose_axes,
                                  _bwd_memo=bwd_memo, _calibrated=calibrated)
      except _NotFused:
        pass
    # The attempt may have run a calibration before it found out that the call has no fused form
    # (the reference updates a stateful calibrator once per call): those results are handed over.
    with aqt_quantizer.replay_calibrations(calibrated):
      return self._unfused_call(lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, out_transpose_axes)

  # ------------------------------------------------------------------------------
  def _unfused_call(self, lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, out_transpose_axes=None):
    """The operator one step at a time: calibrate, quantize, contract, dequantize.

    Follows aqt_dot_general.py:795-828 through the plugin points (`dg_quantizer`,
    `dot_general`), so what the lowered paths leave out still runs on the GPU: quantizers,
    numerics and contraction hooks of the user's own, biases, sparsity masks and several scales
    per tensor (mid scales kept in the QTensors).  Each step is its own kernel (the quantize and
    scale-and-cast kernels, the MFMA or library contraction) with elementwise tensor arithmetic
    in between.
    """
    if isinstance(lhs, _Prescaled):
      lhs = lhs.x * lhs.scale_t.to(lhs.x.dtype)
    if isinstance(rhs, aqt_tensor.QTensor):
      rhs = rhs.qvalue.to(rhs.dequant_dtype)

    (lhs_qt, lhs_grad), (rhs_qt, rhs_grad), (lhs, rhs) = _quant(
        lhs, rhs, lhs_qt, rhs_qt, self.dg_quantizer, self.lhs, self.rhs, dimension_numbers,
        self.allow_dummy_gradient_into_qtensor)

    msg = ('biases are only supported in fake quant mode, but got a {arg} bias '
           'and self.{arg}.dequant_mode == {mode} != DequantMode.THIS_INPUT')
    assert not (lhs_qt.bias and self.lhs.dequant_mode != DequantMode.THIS_INPUT), msg.format(
        arg='lhs', mode=self.lhs.dequant_mode)
    assert not (rhs_qt.bias and self.rhs.dequant_mode != DequantMode.THIS_INPUT), msg.format(
        arg='rhs', mode=self.rhs.dequant_mode)

    res = DotGeneralRes(lhs=TensorRes(mt=MultiTensor(x=lhs, qx=lhs_qt), quant_grad=lhs_grad),
                        rhs=TensorRes(mt=MultiTensor(x=rhs, qx=rhs_qt), quant_grad=rhs_grad))
    out = _qtensor_dot_general_unfused(lhs_qt, rhs_qt, dimension_numbers, self,
                                       torch.promote_types(lhs.dtype, rhs.dtype)).dequant()
    if out_transpose_axes is not None:
      out = out.permute(tuple(out_transpose_axes))
    return out, res

  # ------------------------------------------------------------------------------
  def _lowered_call(self, lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, out_transpose_axes=None,
                    _dtypes=None, _bwd_memo=None, _calibrated=None):
    """`_dtypes` = (lhs dtype, rhs dtype, dequant dtype) when `lhs` and `rhs` are the qvalues of
    the given QTensors and so do not carry the dtypes of the tensors they were quantized from."""
    dq = self.dg_quantizer
    prescale_t = None
    if isinstance(lhs, _Prescaled):
      prescale_t, lhs = lhs.scale_t, lhs.x
    rhs_is_q = isinstance(rhs, aqt_tensor.QTensor)  # re-quantization of a fwd residual
    rhs_arr = rhs.qvalue if rhs_is_q else rhs
    lhs_dtype = lhs.dtype
    rhs_dtype = rhs.dequant_dtype if rhs_is_q else rhs.dtype
    dequant_dtype = torch.promote_types(lhs_dtype, rhs_dtype)
    if _dtypes is not None:
      lhs_dtype, rhs_dtype, dequant_dtype = _dtypes

    lhs_none = isinstance(dq.lhs.numerics, no_numerics.NoNumerics) if isinstance(
        dq, DefaultDotGeneralQuantizer) else False
    rhs_none = isinstance(dq.rhs.numerics, no_numerics.NoNumerics) if isinstance(
        dq, DefaultDotGeneralQuantizer) else False

    if lhs_none and rhs_none and lhs_qt is None and rhs_qt is None:
      # Unquantized: QTensors without scales around a plain float contraction
      # (aqt_quantizer.py:111-120; aqt_dot_general.py:921-927 with float operands).
      x = lhs
      if prescale_t is not None:
        x = x * prescale_t.to(x.dtype)
      y = rhs_arr.to(rhs_dtype) if rhs_is_q else rhs_arr
      out = self.dot_general(x, y, dimension_numbers, None, self.dg_accumulator_dtype)
      out = out.to(dequant_dtype)
      if out_transpose_axes is not None:
        out = out.permute(tuple(out_transpose_axes))
      mk = lambda t: aqt_tensor.QTensor(qvalue=t, scale=[], scale_t=None, bias=[], dequant_dtype=t.dtype)
      res = DotGeneralRes(lhs=TensorRes(mt=MultiTensor(x=x, qx=mk(x)), quant_grad=None),
                          rhs=TensorRes(mt=MultiTensor(x=y, qx=mk(y)), quant_grad=None))
      return out, res

    if isinstance(dq, DefaultDotGeneralQuantizer) and lhs_none and not rhs_none:
      served = self._serve_weight_only(lhs, dq, lhs_qt, rhs_arr, rhs_qt, dimension_numbers, prescale_t,
                                       out_transpose_axes, dequant_dtype)
      if served is not None:
        return served
    if not isinstance(dq, DefaultDotGeneralQuantizer):
      raise _NotFused('only DefaultDotGeneralQuantizer is lowered')
    if dq.lhs_mid_alpha is not None or dq.rhs_mid_alpha is not None:
      # Mid scales (aqt_dot_general.py:504-554): the calibration runs step by step (abs-max kernels over the
      # remaining axes and arithmetic on the per-channel vectors, one elementwise division per operand); with
      # skip_mid_scales, the reference's default, each side is left with one scale, and the quantize and
      # contraction kernels take it from there as they take any given scale.
      if lhs_qt is not None or rhs_qt is not None or rhs_is_q or lhs_none or rhs_none:
        raise _NotFused('mid scales next to a provided QTensor, a forward residual or an unquantized side')
      if prescale_t is not None:
        lhs, prescale_t = lhs * prescale_t.to(lhs.dtype), None
      record = {} if _calibrated is None else _calibrated
      with aqt_quantizer.record_calibrations(record):
        (_, lhs_qt), (_, rhs_qt) = dq.calibrate(lhs, rhs_arr, dimension_numbers, self.lhs.calibration_mode,
                                                self.rhs.calibration_mode)
      for qt in (lhs_qt, rhs_qt):
        if len(qt.scale) != 1 or qt.bias or qt.sparsity_mask is not None:
          raise _NotFused('mid scales kept in the QTensors (skip_mid_scales = False), a bias or a sparsity mask')
    default_modes = all(side.dequant_mode == DequantMode.OUTPUT
                        and side.calibration_mode == CalibrationMode.CONTRACTING_AXIS for side in (self.lhs, self.rhs))
    held_float = any(isinstance(q.numerics, int_numerics.IntSymmetric) and q.numerics.dtype is None
                     for q in (dq.lhs, dq.rhs))
    given_float = any(qt is not None and qt.is_full() and qt.qvalue.is_floating_point()
                      and qt.qvalue.dtype not in _FP8_DTYPES for qt in (lhs_qt, rhs_qt))
    if lhs_none or rhs_none or not default_modes or held_float or given_float:
      return self._float_contraction(lhs, rhs_arr, rhs_is_q, lhs_dtype, rhs_dtype, dequant_dtype, lhs_qt, rhs_qt,
                                     dimension_numbers, prescale_t, out_transpose_axes, lhs_none, rhs_none,
                                     _bwd_memo, _calibrated)

    ragged = _ragged_sizes(self.dot_general)
    if ragged is not None:
      # lhs [m, k] x rhs [g, k, n]; the dimension numbers only say which axes share a scale
      (lca, rca), (lba, rba) = dimension_numbers
      if (lhs.dim() != 2 or rhs_arr.dim() != 3 or list(lca) != [1] or list(rca) != [0, 1] or lba or rba
          or out_transpose_axes is not None or lhs.shape[1] != rhs_arr.shape[1]):
        raise _NotFused('ragged contraction in another layout')
      dn = (([1], [0, 1]), ([], []))
    else:
      dn = _canonical_pairs(lhs, rhs_arr, dimension_numbers)
    (lca, rca), (lba, rba) = dn
    lra = utils.get_remaining_axes(lhs.dim(), lca, lba)
    rra = utils.get_remaining_axes(rhs_arr.dim(), rca, rba)

    served = self._serve_small_batch(lhs, lhs_dtype, dq, lhs_qt, rhs_arr, rhs_qt, dn, prescale_t,
                                     out_transpose_axes, dequant_dtype, dimension_numbers)
    if served is not None:
      return served

    # ---- lhs ---------------------------------------------------------------------
    want_l, want_r = _RESIDUAL_ABSMAX.get()
    lq, ls, lsdt, lhs_qt_out, lhs_grad = self._quant_side(
        'lhs', lhs, lhs_dtype, False, dq.lhs, lhs_qt, lba, lra, lca, prescale_t, _bwd_memo, _calibrated,
        want_other_axis_absmax=want_l)
    # ---- rhs ---------------------------------------------------------------------
    rq, rs, rsdt, rhs_qt_out, rhs_grad = self._quant_side(
        'rhs', rhs_arr, rhs_dtype, rhs_is_q, dq.rhs, rhs_qt, rba, rra, rca, None, _bwd_memo, _calibrated,
        layout_later=rhs_qt is not None and rhs_qt.qvalue is not None and rhs_qt.qvalue.dtype == torch.int8,
        want_other_axis_absmax=want_r)
    rv_later = None  # a frozen int8 rhs that is not laid out for the kernels as the caller holds it
    if rq is None:
      rv_later = lowering.view_operand(rhs_qt.qvalue, rba, rra, rca)
      if ragged is not None:
        rq, rv_later = _kernel_layout_of(rhs_qt.qvalue, rv_later), None

    lkd = aqt_tensor.qvalue_kernel_dtype(lhs_qt_out)
    rkd = aqt_tensor.qvalue_kernel_dtype(rhs_qt_out)
    fp8 = lkd in (L.E4M3, L.E5M2)
    if fp8 != (rkd in (L.E4M3, L.E5M2)):
      raise _NotFused('mixed integer / fp8 operands')
    acc = self.dg_accumulator_dtype
    if not fp8:
      assert acc == utils.int32, (
          f'Found {self.dg_accumulator_dtype=}: integer operands are contracted with an int32 '
          'accumulator only')
    else:
      assert acc in (utils.float32, None), f'{self.dg_accumulator_dtype=} with fp8 operands'

    B, M, K = lq.shape
    N = rq.shape[1] if rq is not None else rv_later.R
    if ragged is not None:
      G = rhs_arr.shape[0]
      rq3 = rq.reshape(N, G, K).permute(1, 0, 2)  # [g, n, k] view of the quantizer's [n, g*k] rows
      if not (K % 16 == 0 and lq.data_ptr() % 16 == 0 and rq3.data_ptr() % 16 == 0 and M * N > 0):
        raise _NotFused('ragged contraction with unaligned operands')
      out = ops.gemm(lq, rq3, row_scale=ls.reshape(1, M) if ls.numel() == M else ls.reshape(1, 1).expand(1, M).contiguous(),
                     col_scale=rs.reshape(1, -1).expand(G, N).contiguous(), a_dtype=lkd, b_dtype=rkd,
                     row_scale_dtype=lsdt, col_scale_dtype=rsdt, out_dtype=dequant_dtype, dequant_dtype=dequant_dtype,
                     group_offsets=ops.ragged_offsets(ragged, M, lq.device))
      res = DotGeneralRes(lhs=TensorRes(mt=MultiTensor(x=lhs, qx=lhs_qt_out), quant_grad=lhs_grad),
                          rhs=TensorRes(mt=MultiTensor(x=rhs_arr, qx=rhs_qt_out), quant_grad=rhs_grad))
      return out.reshape(M, N), res
    if rq is not None:
      assert rq.shape[0] == B and rq.shape[2] == K, (lq.shape, rq.shape)
    else:
      assert rv_later.B == B and rv_later.K == K, (lq.shape, rv_later.B, rv_later.R, rv_later.K)
    # scales: [B, M] / [B, N] or a single per-tensor value (broadcast here, tiny)
    def expand(s, n):
      return s.reshape(1, 1).expand(B, n).contiguous() if s.numel() == 1 and B * n != 1 else s.reshape(B, n)
    if self.dot_general is not lax_dot_general:
      raise _NotFused('a custom DotGeneralRaw.dot_general hook is not lowered')  # (ragged hooks returned above)
    nb, nl, nr = len(lba), len(lra), len(rra)
    bdims = [lhs.shape[a] for a in lba]
    ldims = [lhs.shape[a] for a in lra]
    rdims = [rhs_arr.shape[a] for a in rra]
    want_lba = list(dimension_numbers[1][0])
    swap_perm = list(range(nb)) + list(range(nb + nl, nb + nl + nr)) + list(range(nb, nb + nl))
    swapped = (out_transpose_axes is not None and list(out_transpose_axes) == swap_perm
               and want_lba == lba and nl > 0 and nr > 0)
    common = dict(out_dtype=dequant_dtype, dequant_dtype=dequant_dtype)
    # a frozen int4 weight is read packed two values per byte (half the bytes of a serving call
    # and of the copy kept per weight; made once per tensor), unpacked in registers by the kernel
    pack = (not swapped and not fp8 and rhs_qt is not None and rhs_qt.is_full() and rhs_qt.container_dtype is utils.int4
            and rkd == L.I4 and K % 32 == 0 and K < 132096 and (rq is None or rq.dtype == torch.int8))
    b_layout = L.W_ROWS
    if rv_later is not None:
      # the copy the serving kernels stream (fragment order) serves the contraction kernels too, so a weight
      # used with few and with many lhs rows is kept once; the swapped product reads the weight as rows
      frag = (not swapped and not fp8 and B == 1 and K % 16 == 0 and N * K < 2 ** 31 and lq.stride(1) % 16 == 0
              and lq.data_ptr() % 16 == 0 and ops.GEMM_TUNING in (0, 8, 128))
      rq = _kernel_layout_of(rhs_qt.qvalue, rv_later, pack_int4=pack, fragments=frag)
      b_layout = L.W_FRAGMENTS if frag else L.W_ROWS
      rkd = L.I4P if pack else rkd
    elif pack:
      rq = _kernel_layout_of(rhs_qt.qvalue, lowering.view_operand(rhs_qt.qvalue, rba, rra, rca), pack_int4=True)
      rkd = L.I4P
    if swapped:
      # C^T = rhs_q . lhs_q^T; the lhs scale still multiplies first (aqt_tensor.py:182-183)
      out = ops.gemm(rq, lq, row_scale=expand(rs, N), col_scale=expand(ls, M), a_dtype=rkd, b_dtype=lkd,
                     scale_order=L.SCALE_COL_THEN_ROW, row_scale_dtype=rsdt, col_scale_dtype=lsdt, **common)
      out = out.reshape(bdims + rdims + ldims)
    else:
      out = ops.gemm(lq, rq, row_scale=expand(ls, M), col_scale=expand(rs, N), a_dtype=lkd, b_dtype=rkd,
                     row_scale_dtype=lsdt, col_scale_dtype=rsdt, b_layout=b_layout, **common)
      # [B, M, N] -> (batch..., lhs remaining..., rhs remaining...) in the caller's batch order
      out = out.reshape(bdims + ldims + rdims)
      if want_lba != lba:
        perm = [lba.index(a) for a in want_lba] + list(range(len(lba), out.dim()))
        out = out.permute(tuple(perm))
      if out_transpose_axes is not None:
        out = out.permute(tuple(out_transpose_axes))

    lhs_mt = MultiTensor(x=lhs, qx=lhs_qt_out)
    rhs_mt = MultiTensor(x=rhs_arr if not rhs_is_q else rhs.qvalue, qx=rhs_qt_out)
    res = DotGeneralRes(lhs=TensorRes(mt=lhs_mt, quant_grad=lhs_grad),
                        rhs=TensorRes(mt=rhs_mt, quant_grad=rhs_grad))
    return out, res

  def _float_contraction(self, lhs, rhs_arr, rhs_is_q, lhs_dtype, rhs_dtype, dequant_dtype, lhs_qt, rhs_qt,
                         dimension_numbers, prescale_t, out_transpose_axes, lhs_none, rhs_none,
                         bwd_memo, calibrated):
    """The configurations whose contraction is a float one (aqt_dot_general.py:843-958): fake quantization
    (DequantMode.THIS_INPUT), the scale of one operand multiplied into the other (OTHER_INPUT), calibration
    over the remaining axes, one side left unquantized.

    Per quantized side one calibrate-and-quantize kernel sequence (the residual the backward pass needs) and
    one pass of the scale-and-cast kernel that makes the side's contraction operand (its own scale and / or
    the other side's; a bare cast for an integer side next to a float one); the library's float product; one
    more scale-and-cast pass over the result when a side is dequantized there (DequantMode.OUTPUT).
    """
    dq = self.dg_quantizer
    if self.dot_general is not lax_dot_general:
      raise _NotFused('a custom DotGeneralRaw.dot_general hook is not lowered')
    dn = _canonical_pairs(lhs, rhs_arr, dimension_numbers)
    (lca, rca), (lba, rba) = dn
    lra = utils.get_remaining_axes(lhs.dim(), lca, lba)
    rra = utils.get_remaining_axes(rhs_arr.dim(), rca, rba)

    class Side:
      pass

    def mem_to_logical(t, v, rk):
      """A [B, R', K'] (rk) or [B, K', R'] tensor of the view v, indexed like the tensor the view was made from."""
      if rk:
        return lowering.logical_from_brk(t, v)
      axes = v.b_axes + v.k_axes + v.r_axes
      inv = [0] * len(axes)
      for pos, a in enumerate(axes):
        inv[a] = pos
      return t.reshape([v.shape[a] for a in axes]).permute(tuple(inv))

    def make(name, x, dtype, x_is_q, quantizer, given, cfg, ba, ra, ca, none, prescale):
      sd = Side()
      sd.cfg, sd.none = cfg, none
      sd.by_k = cfg.calibration_mode == CalibrationMode.REMAINING_AXIS  # one scale per (batch, contraction index)
      if none:
        if given is not None or x_is_q:
          raise _NotFused(f'{name}: a provided QTensor next to NoNumerics')
        if prescale is not None:
          x = x * prescale.to(x.dtype)
        sd.v = lowering.view_operand(x, ba, ra, ca)
        sd.mem, sd.x, sd.grad, sd.s32, sd.sdt = sd.v.mem, x, None, None, None
        sd.rk = sd.k_inner = sd.v.k_last  # mem is [B, R, K] (else [B, K, R])
        sd.qt = aqt_tensor.QTensor(qvalue=x, scale=[], scale_t=None, bias=[], dequant_dtype=x.dtype)
        sd.kdt = sd.held = None
        return sd
      # the quantizer's view: the axes that share a scale take the place of the contraction axes
      va, vk = (ca, ra) if sd.by_k else (ra, ca)
      if x_is_q and x.is_floating_point() and x.dtype not in _FP8_DTYPES:
        x, x_is_q = x.to(dtype), False  # a residual held in a float dtype: qvalue.astype(dequant_dtype)
      num = quantizer.numerics
      if ((given is None or not given.is_full()) and isinstance(num, int_numerics.IntSymmetric) and num.dtype is None
          and num.noise_fn is None and num.kernel_spec(True) is None and not x_is_q and x.is_floating_point()):
        # Results that are not integers (no rounding, no clipping, buckets centred off zero) and stay in the float
        # dtype: the calibration as usual, then one scale-and-cast pass with the reciprocal scale and the
        # numerics' clipping and rounding (aqt_tensor.py:125-159, int_numerics.py:81-111), in x's own layout.
        if prescale is not None:
          x = x * prescale.to(x.dtype)
        if given is not None:
          inc = given  # an incomplete QTensor: the scale is there already (aqt_dot_general.py:645-653)
        else:
          inc = quantizer.calibrate(x, calibration_axes=vk)
          if calibrated is not None:
            calibrated[id(quantizer)] = inc
        if len(inc.scale) != 1 or inc.bias or inc.sparsity_mask is not None:
          raise _NotFused(f'{name}: calibration with a bias, a sparsity mask or several scales')
        scale = inc.scale[0]
        sd.v = lowering.view_operand(x, ba, va, vk)
        n = sd.v.B * sd.v.R
        s32 = _scale_vector_f32(scale, ba, va, vk)
        if s32.numel() not in (1, n):
          raise _NotFused(f'{name}: a scale that is not shared over exactly the calibration axes')
        sd.s32 = s32.reshape(-1).expand(n).contiguous() if s32.numel() == 1 and n != 1 else s32.reshape(-1)
        sd.sdt, sd.rk = scale.dtype, sd.v.k_last
        held_dt = torch.promote_types(dtype, sd.sdt)
        if sd.v.mem.numel():
          sd.held = ops.scale_cast(
              sd.v.mem, [(sd.s32, L.FACTOR_ROWS if sd.rk else L.FACTOR_COLS, sd.sdt, False, True)], out_dtype=held_dt,
              finish_clip=num._get_fwd_clip_bound() if num.clip else None,
              finish_round=0 if not num.round else 1 if num.preserve_zero else 2)
        else:
          sd.held = torch.empty(sd.v.mem.shape, dtype=held_dt, device=x.device)
        sd.mem, sd.x, sd.kdt = sd.held, x, None
        sd.k_inner = sd.rk != sd.by_k
        sd.qt = aqt_tensor.QTensor(qvalue=mem_to_logical(sd.held, sd.v, sd.rk), scale=[scale], scale_t=None, bias=[],
                                   dequant_dtype=dtype)
        sd.grad = (aqt_quantizer.clip_gradient_later(num, x, [scale]) if num.clip_gradient
                   else functools.partial(num.vjp_bwd, (None,)))
        return sd
      q, s32, sdt, qt, grad = self._quant_side(name, x, dtype, x_is_q, quantizer, given, ba, va, vk, prescale,
                                               bwd_memo, calibrated, held_float=True)
      given_full = given is not None and given.is_full()
      sd.v = lowering.view_operand(qt.qvalue if given_full else x, ba, va, vk)
      n = sd.v.B * sd.v.R
      if s32.numel() not in (1, n):
        raise _NotFused(f'{name}: a scale that is not shared over exactly the calibration axes')
      sd.s32 = s32.reshape(-1).expand(n).contiguous() if s32.numel() == 1 and n != 1 else s32.reshape(-1)
      if qt.dequant_dtype is None:
        raise _NotFused(f'{name}: a QTensor without a dequant_dtype')
      sd.held = None  # the quantized values as the float tensor the reference holds, [B, R, K] of the view
      if not given_full and getattr(quantizer.numerics, 'dtype', 0) is None:
        # numerics that keep their integers in the float dtype (the usual fake-quant setting): the kernel
        # wrote them as int8, which holds the same values; the residual is their cast
        held_dt = torch.promote_types(dtype, sdt)
        sd.held = (ops.scale_cast(q, [], out_dtype=held_dt) if q.numel()
                   else torch.empty(q.shape, dtype=held_dt, device=q.device))
        qt = qt.replace(qvalue=lowering.logical_from_brk(sd.held, sd.v), container_dtype=None)
      elif qt.qvalue.dtype.is_floating_point and qt.qvalue.dtype not in _FP8_DTYPES:
        sd.held = q
      elif qt.qvalue.dtype != torch.int8 and qt.qvalue.dtype not in _FP8_DTYPES:
        raise _NotFused(f'{name}: quantized values held in {qt.qvalue.dtype}')
      sd.mem, sd.x, sd.grad, sd.sdt, sd.qt = q, x, grad, sdt, qt
      sd.rk = True  # the quantize kernel writes [B, R', K'] of its view
      sd.k_inner = not sd.by_k  # that is [B, R, K] with contraction-axis scales, [B, K, R] with remaining-axis ones
      sd.kdt = None if q.is_floating_point() and q.dtype not in _FP8_DTYPES else (
          L.I8 if q.dtype == torch.int8 and sd.held is not None else aqt_tensor.qvalue_kernel_dtype(qt))
      return sd

    L_ = make('lhs', lhs, lhs_dtype, False, dq.lhs, lhs_qt, self.lhs, lba, lra, lca, lhs_none, prescale_t)
    R_ = make('rhs', rhs_arr, rhs_dtype, rhs_is_q, dq.rhs, rhs_qt, self.rhs, rba, rra, rca, rhs_none, None)

    msg = ('biases are only supported in fake quant mode, but got a {arg} bias '
           'and self.{arg}.dequant_mode == {mode} != DequantMode.THIS_INPUT')
    for arg, sd in (('lhs', L_), ('rhs', R_)):
      assert not (sd.qt.bias and sd.cfg.dequant_mode != DequantMode.THIS_INPUT), msg.format(
          arg=arg, mode=sd.cfg.dequant_mode)
      if sd.qt.bias or sd.qt.sparsity_mask is not None or (not sd.none and len(sd.qt.scale) != 1):
        raise _NotFused('a bias, a sparsity mask or several scales')

    # dtypes of the two operands of the reference's lax.dot_general call
    def qin_dtype(sd, dtype):
      if sd.none or sd.cfg.dequant_mode == DequantMode.THIS_INPUT:
        return sd.qt.dequant_dtype if not sd.none else sd.x.dtype
      return sd.qt.qvalue.dtype
    ldt, rdt = qin_dtype(L_, lhs_dtype), qin_dtype(R_, rhs_dtype)
    if self.dg_accumulator_dtype == utils.int32:
      assert ldt == utils.int8 and rdt == utils.int8, (
          f'Found {self.dg_accumulator_dtype=}, lhs_qin.dtype={ldt} and rhs_qin.dtype={rdt}. Dot general '
          'accumulator dtype can only be jnp.int32 when both inputs are int8. Otherwise it is '
          'recommended to be None to let lax.dot_general automatically decide it.')
    if L_.cfg.dequant_mode == DequantMode.OTHER_INPUT and not L_.none:
      assert rdt in _DTYPES_CAN_BE_SCALED
    if R_.cfg.dequant_mode == DequantMode.OTHER_INPUT and not R_.none:
      assert ldt in _DTYPES_CAN_BE_SCALED
    if not ldt.is_floating_point and not rdt.is_floating_point or ldt in _FP8_DTYPES or rdt in _FP8_DTYPES:
      raise _NotFused('an integer or fp8 contraction outside the default modes')
    common = torch.promote_types(ldt, rdt)
    if common not in (torch.bfloat16, torch.float32):
      raise _NotFused(f'a contraction in {common}')

    def operand(sd, other, qdt):
      """This side's operand of the float product, in the layout of sd.mem; qdt: the dtype the reference holds
      it in when it reaches lax.dot_general."""
      factors = []
      if not sd.none and sd.cfg.dequant_mode == DequantMode.THIS_INPUT:
        factors.append((sd.s32, L.FACTOR_ROWS if sd.rk else L.FACTOR_COLS, sd.sdt, False))  # QTensor.dequant
      if not other.none and other.cfg.dequant_mode == DequantMode.OTHER_INPUT:
        if not other.by_k:
          raise _NotFused('DequantMode.OTHER_INPUT with a scale that varies along the remaining axes')
        k_count = sd.v.R if (not sd.none and sd.by_k) else sd.v.K
        if other.s32.numel() != sd.v.B * k_count:
          raise _NotFused('a scale that does not fit the other operand')
        # the scale is cast to the dtype of the operand it multiplies (aqt_dot_general.py:893, 902)
        t = other.s32 if qdt == torch.float32 or other.sdt == qdt else other.s32.to(qdt).float()
        factors.append((t, L.FACTOR_COLS if sd.k_inner else L.FACTOR_ROWS, qdt, True))
      if not factors:
        if sd.held is not None:
          return sd.held if sd.held.dtype == common else sd.held.to(common)
        if sd.mem.dtype == common:
          return sd.mem
        if sd.mem.is_floating_point() and sd.mem.dtype not in _FP8_DTYPES or sd.mem.numel() == 0:
          return sd.mem.to(common)
        qdt = common  # an integer operand next to a float one: jnp's type promotion casts it
      mem = sd.mem.view(torch.uint8) if sd.mem.dtype in _FP8_DTYPES else sd.mem
      if mem.numel() == 0:
        return torch.empty(mem.shape, dtype=common, device=mem.device)
      out = ops.scale_cast(mem.contiguous(), factors, out_dtype=qdt, in_dtype=sd.kdt)
      return out if out.dtype == common else out.to(common)

    def logical(t, sd):
      return mem_to_logical(t, sd.v, sd.rk)

    lop = logical(operand(L_, R_, ldt), L_)
    if (WEIGHT_ONLY_FLOAT_COPY and rhs_qt is not None and rhs_qt.is_full() and not rdt.is_floating_point
        and L_.cfg.dequant_mode != DequantMode.OTHER_INPUT):
      rop = R_.qt.qvalue  # a frozen weight: lax_dot_general keeps its float copy between calls
    else:
      rop = logical(operand(R_, L_, rdt), R_)
    out = lax_dot_general(lop, rop, dn, None, self.dg_accumulator_dtype)  # (batch..., lhs remaining..., rhs remaining...)

    nb = len(lba)
    bdims = [lhs.shape[a] for a in lba]
    ldims = [lhs.shape[a] for a in lra]
    rdims = [rhs_arr.shape[a] for a in rra]
    B, M, N = math.prod(bdims), math.prod(ldims), math.prod(rdims)
    factors = []
    for sd, axis, count in ((L_, L.FACTOR_ROWS, M), (R_, L.FACTOR_COLS, N)):
      if sd.none or sd.cfg.dequant_mode != DequantMode.OUTPUT:
        continue
      if sd.by_k or sd.s32.numel() != B * count:
        raise _NotFused('DequantMode.OUTPUT with a scale along the contraction axes')
      factors.append((sd.s32, axis, sd.sdt, False))
    if factors and out.numel():
      out = ops.scale_cast(out.reshape(B, M, N).contiguous(), factors, out_dtype=dequant_dtype)
    out = out.to(dequant_dtype).reshape(bdims + ldims + rdims)
    want_lba = list(dimension_numbers[1][0])
    if want_lba != lba:
      perm = [lba.index(a) for a in want_lba] + list(range(nb, out.dim()))
      out = out.permute(tuple(perm))
    if out_transpose_axes is not None:
      out = out.permute(tuple(out_transpose_axes))
    res = DotGeneralRes(lhs=TensorRes(mt=MultiTensor(x=L_.x, qx=L_.qt), quant_grad=L_.grad),
                        rhs=TensorRes(mt=MultiTensor(x=R_.x, qx=R_.qt), quant_grad=R_.grad))
    return out, res

  def _serve_small_batch(self, lhs, lhs_dtype, dq, lhs_qt, rhs_arr, rhs_qt, dn, prescale_t,
                         out_transpose_axes, dequant_dtype, dimension_numbers):
    """Serving with a frozen int8 rhs and at most 64 lhs rows: the fused decode kernel.

    Same arithmetic as the general path (per-token abs-max int8 quantisation of the lhs, int32
    contraction, QTensor.dequant); returns None when the call does not have that shape.
    """
    (lca, rca), (lba, rba) = dn
    if (rhs_qt is None or not rhs_qt.is_full() or lhs_qt is not None or prescale_t is not None
        or out_transpose_axes is not None or lba or rba or self.dot_general is not lax_dot_general):
      return None
    spec = dq.lhs.kernel_spec()
    if (spec is None or spec['out_dtype'] != L.I8 or spec['noise'] != L.NOISE_NONE
        or dq.lhs.calib_shared_axes is not None or getattr(dq.lhs.numerics, 'clip_gradient', False)):
      return None
    if (rhs_qt.qvalue.dtype != torch.int8 or len(rhs_qt.scale) != 1 or rhs_qt.bias
        or rhs_qt.container_dtype not in (None, utils.int4) or dequant_dtype != lhs.dtype
        or self.dg_accumulator_dtype != utils.int32):
      return None
    lra = utils.get_remaining_axes(lhs.dim(), lca, lba)
    rra = utils.get_remaining_axes(rhs_arr.dim(), rca, rba)
    lv = lowering.view_operand(lhs, [], lra, lca)
    rv = lowering.view_operand(rhs_qt.qvalue, [], rra, rca)
    if not lv.k_last or lv.copied:
      return None
    M, K, N = lv.R, lv.K, rv.R
    # int4 weights are streamed packed two per byte (a copy made once per frozen tensor)
    packed = rhs_qt.container_dtype is utils.int4 and K % 32 == 0
    if M == 0 or M > 64 or K == 0 or K % 16 != 0 or N == 0 or N * K >= 2 ** 31:
      return None
    # the frozen weight in fragment order (and packed, for int4): one copy per tensor, made on its
    # first serving call
    w_fragments = _kernel_layout_of(rhs_qt.qvalue, rv, pack_int4=packed, fragments=True)
    w_scale = rhs_qt.scale[0]
    sv = lowering.view_operand(w_scale, [], rra, rca)
    if sv.mem.numel() != N:
      return None
    sdt = dq.lhs._calibrator.dtype if dq.lhs._calibrator.dtype is not None else lhs_dtype
    out, xs, xq = ops.decode(lv.mem[0], w_fragments, _scale_vector_f32(w_scale, [], rra, rca),
                             quant_bound=spec['quant_bound'], clip_bound=spec['clip_bound'],
                             x_scale_dtype=sdt, w_scale_dtype=w_scale.dtype, want_xq=True,
                             w_dtype=L.I4P if packed else L.I4 if rhs_qt.container_dtype is utils.int4 else L.I8,
                             w_layout=L.W_FRAGMENTS)
    out = out.reshape([lhs.shape[a] for a in lra] + [rhs_arr.shape[a] for a in rra])
    qv = lowering.logical_from_brk(xq[None], lv)
    sc = lowering.logical_from_brk(xs.reshape(1, M), lv, k_keep=False).to(sdt)
    lhs_qt_out = aqt_tensor.QTensor(qvalue=qv, scale=[sc], scale_t=None, bias=[], dequant_dtype=lhs_dtype)
    lhs_grad = functools.partial(dq.lhs.numerics.vjp_bwd, (None,))
    rhs_grad = None if self.allow_dummy_gradient_into_qtensor else _POISON
    res = DotGeneralRes(lhs=TensorRes(mt=MultiTensor(x=lhs, qx=lhs_qt_out), quant_grad=lhs_grad),
                        rhs=TensorRes(mt=MultiTensor(x=rhs_arr, qx=rhs_qt), quant_grad=rhs_grad))
    return out, res

  def _serve_weight_only(self, lhs, dq, lhs_qt, rhs_arr, rhs_qt, dimension_numbers, prescale_t, out_transpose_axes,
                         dequant_dtype):
    """Serving with an unquantized bf16 lhs and a frozen int8 / int4 rhs with one scale per output channel:
    the weight-only kernels (the weight converted to bf16 in registers; the reference promotes the whole
    weight to bf16 and contracts in float, aqt_dot_general.py:843-958): the streaming kernel up to 64 lhs
    rows, above that the tiled one unless WEIGHT_ONLY_FLOAT_COPY.  Returns None when the call does not
    have that shape."""
    if (rhs_qt is None or not rhs_qt.is_full() or lhs_qt is not None or prescale_t is not None
        or out_transpose_axes is not None or self.dot_general is not lax_dot_general or self.local_aqt is not None
        or self.rhs.dequant_mode != DequantMode.OUTPUT or lhs.dtype != torch.bfloat16
        or dequant_dtype != torch.bfloat16 or (lhs.requires_grad and torch.is_grad_enabled())):
      return None
    if (rhs_qt.qvalue.dtype != torch.int8 or len(rhs_qt.scale) != 1 or rhs_qt.bias or rhs_qt.sparsity_mask is not None
        or rhs_qt.container_dtype not in (None, utils.int4)
        or rhs_qt.scale[0].dtype not in (torch.bfloat16, torch.float32)):
      return None
    dn = _canonical_pairs(lhs, rhs_arr, dimension_numbers)
    (lca, rca), (lba, rba) = dn
    if lba or rba:
      return None
    lra = utils.get_remaining_axes(lhs.dim(), lca, lba)
    rra = utils.get_remaining_axes(rhs_arr.dim(), rca, rba)
    lv = lowering.view_operand(lhs, [], lra, lca)
    rv = lowering.view_operand(rhs_qt.qvalue, [], rra, rca)
    if not lv.k_last or lv.copied:
      return None
    M, K, N = lv.R, lv.K, rv.R
    packed = rhs_qt.container_dtype is utils.int4 and K % 32 == 0
    if M == 0 or (M > 64 and WEIGHT_ONLY_FLOAT_COPY) or K == 0 or K % 16 != 0 or N == 0 or N * K >= 2 ** 31:
      return None
    w_scale = rhs_qt.scale[0]
    if lowering.view_operand(w_scale, [], rra, rca).mem.numel() != N:
      return None
    if M <= 64:
      w_fragments = _kernel_layout_of(rhs_qt.qvalue, rv, pack_int4=packed, fragments=True)
      out = ops.decode_weight_only(
          lv.mem[0], w_fragments, _scale_vector_f32(w_scale, [], rra, rca), w_scale_dtype=w_scale.dtype,
          w_dtype=L.I4P if packed else L.I4 if rhs_qt.container_dtype is utils.int4 else L.I8, w_layout=L.W_FRAGMENTS)
    else:
      if rv.k_last and not rv.copied:
        w, w_layout = rv.mem, L.W_ROWS
      else:
        w, w_layout = _kernel_layout_of(rhs_qt.qvalue, rv, fragments=True), L.W_FRAGMENTS
      out = ops.gemm_weight_only(lv.mem, w, _scale_vector_f32(w_scale, [], rra, rca).reshape(1, N),
                                 col_scale_dtype=w_scale.dtype, b_layout=w_layout)
    out = out.reshape([lhs.shape[a] for a in lra] + [rhs_arr.shape[a] for a in rra])
    lhs_qt_out = aqt_tensor.QTensor(qvalue=lhs, scale=[], scale_t=None, bias=[], dequant_dtype=lhs.dtype)
    rhs_grad = None if self.allow_dummy_gradient_into_qtensor else _POISON
    res = DotGeneralRes(lhs=TensorRes(mt=MultiTensor(x=lhs, qx=lhs_qt_out), quant_grad=None),
                        rhs=TensorRes(mt=MultiTensor(x=rhs_arr, qx=rhs_qt), quant_grad=rhs_grad))
    return out, res

  def _quant_side(self, name, x, dtype, x_is_q, quantizer, given_qt, ba, ra, ca, prescale_t,
                  bwd_memo=None, calibrated=None, layout_later=False, held_float=False,
                  want_other_axis_absmax=False):
    """Quantizes one side; returns (q [B,R,K], scale f32, scale dtype, QTensor, quant_grad).
    `bwd_memo`: the backward pass's table of per-tensor scales; `calibrated`: where a calibration
    that runs step by step leaves its result for a later fall-back of the same call; `held_float`:
    numerics that keep their integers in the float dtype are taken too (q and the QTensor come back
    as int8, the caller casts); `want_other_axis_absmax`: the backward pass is going to quantize the
    values written here once more over the other axis (_maybe_use_fwd_quant), so the kernels leave
    the partial maxima that calibration needs with the quantized tensor (ops.quantize), and the
    call that finds them there (`x_is_q`) skips its abs-max pass."""
    def numerics_spec():
      if isinstance(quantizer.numerics, no_numerics.NoNumerics):
        return None
      return quantizer.numerics.kernel_spec(True) if held_float else quantizer.numerics.kernel_spec()
    if given_qt is not None and given_qt.is_full():
      # Serving: the provided QTensor replaces the computed one (aqt_dot_general.py:614-635).
      quant_grad = None if self.allow_dummy_gradient_into_qtensor else _POISON
      if given_qt.bias or len(given_qt.scale) != 1 or given_qt.sparsity_mask is not None:
        raise _NotFused('a provided QTensor with a bias, a sparsity mask or several scales')
      v = lowering.view_operand(given_qt.qvalue, ba, ra, ca)
      if v.k_last and not v.copied:
        q = v.mem
      elif layout_later:
        q = None  # the caller picks rows or the serving kernels' fragment order (one copy kept per weight)
      else:
        q = _kernel_layout_of(given_qt.qvalue, v)
      if q is not None and q.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        q = q.view(torch.uint8)
      s = given_qt.scale[0]
      return q, _scale_vector_f32(s, ba, ra, ca), s.dtype, given_qt, quant_grad
    spec = quantizer.kernel_spec(held_float)
    if spec is None and given_qt is None:
      # The numerics have a kernel but the calibration does not (power-of-two or clipped
      # scales, constant bounds, static-range and delayed-scaling statistics...): calibrate step
      # by step, then quantize and contract in the fused kernels with that scale.
      nspec = numerics_spec()
      if nspec is None or quantizer._calibrator is None:
        raise _NotFused(f'{name}: numerics/calibration {quantizer.numerics} / '
                        f'{quantizer.calibration} have no fused HIP kernel')
      # the calibrator has to see the tensor the reference hands it: the gradient already
      # multiplied by the forward scale, the forward residual as values of the float dtype
      if x_is_q:
        x, x_is_q = x.to(dtype), False
      if prescale_t is not None:
        x, prescale_t = x * prescale_t.to(x.dtype), None
      given_qt = quantizer.calibrate(x, calibration_axes=ca)
      if calibrated is not None:
        calibrated[id(quantizer)] = given_qt
      if len(given_qt.scale) != 1 or given_qt.bias or given_qt.sparsity_mask is not None:
        raise _NotFused(f'{name}: calibration with a bias, a sparsity mask or several scales')
      spec = nspec
    elif spec is None:
      spec = numerics_spec()
    if spec is None:
      raise _NotFused(f'{name}: numerics {quantizer.numerics} have no fused HIP kernel')
    arr = x
    if x_is_q and arr.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
      raise _NotFused('re-quantizing an fp8 residual (use_fwd_quant with fp8 fwd)')
    v = lowering.view_operand(arr, ba, ra, ca)
    prescale = None
    if prescale_t is not None:
      pv = lowering.view_operand(prescale_t, ba, ra, ca)
      if pv.R != 1 and v.R != 1:
        raise _NotFused('use_fwd_quant scale that varies along the remaining axes')
      prescale = pv.mem.reshape(pv.B, -1).float().contiguous()
      if pv.B == 1 and v.B > 1:
        prescale = prescale.reshape(-1)
    scale_in, scale_dtype = None, None
    if given_qt is not None:  # incomplete QTensor: scale only (aqt_dot_general.py:645-653)
      assert len(given_qt.scale) == 1
      gs = given_qt.scale[0]
      scale_dtype = gs.dtype
      if gs.numel() == 1:
        flat = gs.reshape(1).float().expand(v.B * v.R)
      else:
        sv = lowering.view_operand(gs, ba, ra, ca)
        if sv.K != 1 or sv.mem.numel() != v.B * v.R:
          raise _NotFused(f'{name}: a scale that is not shared over exactly the contraction axes')
        flat = sv.mem.reshape(-1).float()
      scale_in = flat.contiguous().reshape(v.B, v.R, 1) if v.k_last else flat.contiguous().reshape(v.B, 1, v.R)
    # Both gradient contractions calibrate the same gradient; with one scale per tensor and no
    # forward-scale factor on it the abs-max is the same number, found once per backward pass.
    memo_key, memo_hit = None, None
    if (bwd_memo is not None and given_qt is None and prescale is None and not x_is_q
        and quantizer.calib_shared_axes == 'per_tensor' and quantizer.kernel_spec(held_float) is not None):
      memo_key = (arr.data_ptr(), arr._version, tuple(arr.shape), arr.dtype, spec['quant_bound'],
                  quantizer._calibrator.dtype)
      memo_hit = bwd_memo.get(memo_key)
      if memo_hit is not None:
        flat = memo_hit[0].reshape(1).expand(v.B * v.R)
        scale_in = flat.contiguous().reshape(v.B, v.R, 1) if v.k_last else flat.contiguous().reshape(v.B, 1, v.R)
        scale_dtype = memo_hit[2]
    partials = None
    if (x_is_q and scale_in is None and prescale is None and arr.dim() == 2 and arr.dtype == torch.int8
        and not v.k_last and not v.copied and quantizer.kernel_spec(held_float) is not None):
      left = getattr(arr, 'other_axis_absmax', None)  # (partial maxima, version of the tensor they describe)
      if left is not None and left[1] == arr._version and left[0].shape[1] == v.R and v.R % 16 == 0:
        partials = left[0]
    q, s32, sdt = quantizer.quant_view(v, dtype, calibration_axes=ca, prescale=prescale, scale=scale_in,
                                       scale_dtype=scale_dtype, held_float=held_float,
                                       want_other_axis_absmax=want_other_axis_absmax and arr.dim() == 2,
                                       absmax_partials=partials)
    qv = lowering.logical_from_brk(aqt_quantizer._typed(q, spec['out_dtype']), v)
    if getattr(q, 'other_axis_absmax', None) is not None:
      qv.other_axis_absmax = (q.other_axis_absmax, qv._version)
    if memo_hit is not None:
      s32, scale_list = memo_hit[0], memo_hit[1]
    elif given_qt is not None:
      scale_list = given_qt.scale
    else:
      scale_list = [lowering.scale_in_dtype(s32, v, sdt)]
      if memo_key is not None:
        bwd_memo[memo_key] = (s32, scale_list, sdt)
    qt = aqt_tensor.QTensor(qvalue=qv, scale=scale_list, scale_t=None, bias=[], dequant_dtype=dtype,
                            container_dtype=utils.int4 if spec['out_dtype'] == L.I4 else None)
    if getattr(quantizer.numerics, 'clip_gradient', False):
      quant_grad = aqt_quantizer.clip_gradient_later(quantizer.numerics, x, scale_list)
    else:
      quant_grad = functools.partial(quantizer.numerics.vjp_bwd, (None,))
    return q, s32, sdt, qt, quant_grad


_DTYPES_CAN_BE_SCALED = (torch.bfloat16, torch.float32, torch.float64)


def _qtensor_dot_general_unfused(lhs_qt, rhs_qt, dimension_numbers, cfg, dequant_dtype) -> aqt_tensor.QTensor:
  """QTensor x QTensor -> QTensor of accumulators and output scales (aqt_dot_general.py:843-958)."""

  def maybe_dequant(qt, tensor_cfg):
    if tensor_cfg.dequant_mode == DequantMode.THIS_INPUT:
      return qt.dequant()
    out = qt.qvalue
    if qt.sparsity_mask is not None:
      out = out * qt.sparsity_mask
    return out

  lhs_qin = maybe_dequant(lhs_qt, cfg.lhs)
  rhs_qin = maybe_dequant(rhs_qt, cfg.rhs)
  dtype_ms = (f'Found {cfg.dg_accumulator_dtype=}, {lhs_qin.dtype=} and {rhs_qin.dtype=}. Dot general '
              'accumulator dtype can only be jnp.int32 when both inputs are int8. Otherwise it is '
              'recommended to be None to let lax.dot_general automatically decide it.')
  if cfg.dg_accumulator_dtype == utils.int32:
    # int4 values travel in int8 containers, so int8 storage covers both allowed types
    assert lhs_qin.dtype == utils.int8 and rhs_qin.dtype == utils.int8, dtype_ms

  if cfg.lhs.dequant_mode == DequantMode.OTHER_INPUT:
    assert rhs_qin.dtype in _DTYPES_CAN_BE_SCALED
    for scale in lhs_qt.scale:
      t = transpose.lhs_scale_transpose_for_rhs_input(scale, dimension_numbers, rhs_qt.qvalue.shape)
      rhs_qin = rhs_qin * t.to(rhs_qin.dtype)
  if cfg.rhs.dequant_mode == DequantMode.OTHER_INPUT:
    assert lhs_qin.dtype in _DTYPES_CAN_BE_SCALED
    for scale in rhs_qt.scale:
      t = transpose.rhs_scale_transpose_for_lhs_input(scale, dimension_numbers, lhs_qt.qvalue.shape)
      lhs_qin = lhs_qin * t.to(lhs_qin.dtype)

  acc = cfg.dot_general(lhs_qin, rhs_qin, dimension_numbers, None, cfg.dg_accumulator_dtype)
  out = aqt_tensor.QTensor(qvalue=acc, scale=[], scale_t=None, bias=[], dequant_dtype=dequant_dtype)
  if cfg.lhs.dequant_mode == DequantMode.OUTPUT:
    out.scale.extend(_get_scale_t(lhs_qt, transpose.lhs_scale_transpose_to_output, dimension_numbers,
                                  lhs_qin.shape, rhs_qin.shape))
  if cfg.rhs.dequant_mode == DequantMode.OUTPUT:
    out.scale.extend(_get_scale_t(rhs_qt, transpose.rhs_scale_transpose_to_output, dimension_numbers,
                                  lhs_qin.shape, rhs_qin.shape))
  return out


def _qtensor_dot_general(lhs_qt, rhs_qt, dimension_numbers, cfg, dequant_dtype):
  """QTensor x QTensor -> dequantized array (aqt_dot_general.py:843-958 + the dequant).

  The reference returns a QTensor (accumulator + output scales) that the caller
  dequantizes; here the dequantisation is fused into the contraction kernel, so the
  dequantized array is returned directly.
  """
  raw = utils.clone_fields(cfg)
  out, _ = DotGeneralRaw._lowered_call(raw, lhs_qt.qvalue, rhs_qt.qvalue, lhs_qt, rhs_qt, dimension_numbers,
                                       _dtypes=(lhs_qt.dequant_dtype, rhs_qt.dequant_dtype, dequant_dtype))
  return out


@dataclasses.dataclass(kw_only=True)
class DotGeneral:
  """Configuration of quantization of dot_general and its gradients (aqt_dot_general.py:961-1078)."""

  fwd: DotGeneralRaw
  dlhs: DotGeneralRaw
  drhs: DotGeneralRaw
  apply_custom_vjp_on_jax: bool = True

  def __deepcopy__(self, memo):
    return utils.deepcopy_fields(self, memo, shared=('apply_custom_vjp_on_jax',))

  @classmethod
  def make(cls, *args, **kwargs):
    return dot_general_make(*args, **kwargs)

  def dg_core(self, lhs, rhs, lhs_qt, rhs_qt, dimension_numbers):
    """dot_general with expanded API (aqt_dot_general.py:975-1000)."""
    msg = 'AQT is not yet optimized to accept quantized types directly. '
    msg += f'lhs.dtype: {lhs.dtype}, rhs.dtype: {rhs.dtype}'
    assert lhs.dtype in [utils.bfloat16, utils.float32, utils.float16], msg
    assert rhs.dtype in [utils.bfloat16, utils.float32, utils.float16], msg
    self.assert_config_validity()
    if self.apply_custom_vjp_on_jax and (lhs.requires_grad or rhs.requires_grad):
      out, lq, rq = _DgCoreFn.apply(lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, self)
      return out, (lq, rq)
    (out, qret), _ = dg_core_vjp_fwd(lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, self)
    return out, qret

  def fused_tile_sum(self, lhs, rhs, dimension_numbers, n_sum_axes: int, lhs_qt=None, rhs_qt=None,
                     with_qt: bool = False, lhs_qvalue_needed: bool = True):
    """sum over the leading `n_sum_axes` output axes of self(lhs, rhs, dimension_numbers), fused.

    This is what tiled_dot_general asks of its inner dot_general when the contraction axis is
    tiled: lhs [..., T, ts] and rhs [T, ts, ...] with the tile-count axis T as the only batch
    axis, every tile calibrated on its own, tile outputs dequantized and summed.  When the
    forward quantizers are plain int8/int4 abs-max ones and no gradient is needed, the
    grouped-scale kernel does all of it without materialising the per-tile outputs.  `rhs_qt`
    may be a frozen weight (the serving case): it is read in the kernel's layout, an int4 one
    packed two values per byte, both made once per frozen tensor.  Returns None when the call
    does not have that shape (the caller then takes the unfused route); with `with_qt`,
    (out, (lhs QTensor, rhs QTensor)) like dg_core; a caller that will only look at the lhs
    QTensor's scales says so with lhs_qvalue_needed=False (it then comes without its qvalue).
    """
    if n_sum_axes != 1 or torch.is_grad_enabled() and (lhs.requires_grad or rhs.requires_grad):
      return None
    (lca, rca), (lba, rba) = dimension_numbers
    lca, rca, lba, rba = list(lca), list(rca), list(lba), list(rba)
    cfg = _fresh_cfg(self)   # calibration objects are created per call, as in dg_core_vjp_fwd
    cfg.fwd.dg_quantizer.init_calibration()
    raw, dq = cfg.fwd, cfg.fwd.dg_quantizer
    if (len(lca) != 1 or len(lba) != 1 or lhs.dtype != rhs.dtype or lhs.dtype not in (utils.bfloat16, utils.float32)
        or not isinstance(dq, DefaultDotGeneralQuantizer) or raw.dg_accumulator_dtype != utils.int32
        or raw.dot_general is not lax_dot_general or dq.lhs_mid_alpha is not None or dq.rhs_mid_alpha is not None):
      return None
    for side in (raw.lhs, raw.rhs):
      if side.dequant_mode != DequantMode.OUTPUT or side.calibration_mode != CalibrationMode.CONTRACTING_AXIS:
        return None
    specs = []
    for q in (dq.lhs, dq.rhs):
      spec = q.kernel_spec()
      if (spec is None or spec['out_dtype'] not in (L.I8, L.I4) or spec['noise'] != L.NOISE_NONE
          or q.calib_shared_axes is not None or getattr(q.numerics, 'clip_gradient', False)):
        return None
      specs.append(spec)
    nl, nr = lhs.dim(), rhs.dim()
    # lhs [remaining..., T, ts], rhs [T, ts, remaining...], both dense in that order
    if not (lba == [nl - 2] and lca == [nl - 1] and rba == [0] and rca == [1] and lhs.is_contiguous()
            and rhs.is_contiguous()):
      return None
    T, ts = lhs.shape[-2], lhs.shape[-1]
    if ts % 128 != 0 or rhs.shape[0] != T or rhs.shape[1] != ts or nl < 3 or nr < 3:
      return None
    M = int(math.prod(lhs.shape[:-2]))
    N = int(math.prod(rhs.shape[2:]))
    if M == 0 or N == 0:
      return None
    if lhs_qt is not None:
      return None  # a quantized activation handed in: the step-by-step route knows what to do
    frozen = rhs_qt is not None
    if frozen:
      sc = rhs_qt.scale[0] if rhs_qt.scale is not None and len(rhs_qt.scale) == 1 else None
      if (not rhs_qt.is_full() or sc is None or rhs_qt.bias or rhs_qt.qvalue.dtype != torch.int8
          or rhs_qt.container_dtype not in (None, utils.int4) or tuple(rhs_qt.qvalue.shape) != tuple(rhs.shape)
          or tuple(sc.shape) != (T, 1) + tuple(rhs.shape[2:]) or sc.dtype not in (utils.bfloat16, utils.float32)
          or rhs_qt.dequant_dtype not in (None, lhs.dtype)):
        return None
    self.assert_config_validity()
    sdt_l = dq.lhs._calibrator.dtype if dq.lhs._calibrator.dtype is not None else lhs.dtype
    rra = list(range(2, nr))
    int4 = frozen and rhs_qt.container_dtype is utils.int4
    packed = int4 and (T * ts) % 32 == 0
    # Against a packed weight, and when nobody asks for the quantized activation itself, the
    # activation is written with every 8 k in even-odd order: the kernel then takes the weight's
    # nibbles as they lie instead of interleaving them again.
    # (aqtx_quantize writes that order for groups of up to _EVEN_ODD8_MAX_GROUP values; longer tiles stay in k order)
    k_order = (L.K_EVEN_ODD8 if packed and ts <= _EVEN_ODD8_MAX_GROUP and not (with_qt and lhs_qvalue_needed)
               else L.K_NATURAL)
    lq, lsc = ops.quantize(lhs.reshape(1, M, T * ts), reduce=L.REDUCE_COLS, group=ts, out_dtype=specs[0]['out_dtype'],
                           quant_bound=specs[0]['quant_bound'], clip_bound=specs[0]['clip_bound'],
                           compute_dtype=lhs.dtype, scale_dtype=sdt_l, k_order=k_order)
    if frozen:
      rv = lowering.view_operand(rhs_qt.qvalue, [], rra, [0, 1])
      rq = _kernel_layout_of(rhs_qt.qvalue, rv, pack_int4=packed)     # [1, N, T*ts] (or packed)
      b_dtype = L.I4P if packed else L.I4 if int4 else L.I8
      sdt_r = sc.dtype
      col_scale = _scale_f32(sc).reshape(T, N).contiguous()
    else:
      sdt_r = dq.rhs._calibrator.dtype if dq.rhs._calibrator.dtype is not None else lhs.dtype
      rq, rsc = ops.quantize(rhs.reshape(1, T * ts, N), reduce=L.REDUCE_ROWS, group=ts, transpose_out=True,
                             out_dtype=specs[1]['out_dtype'], quant_bound=specs[1]['quant_bound'],
                             clip_bound=specs[1]['clip_bound'], compute_dtype=lhs.dtype, scale_dtype=sdt_r)
      b_dtype = specs[1]['out_dtype']
      col_scale = rsc.reshape(T, N)
    out = ops.gemm_grouped(lq[0], rq[0], row_scale=lsc.reshape(M, T), col_scale=col_scale, group=ts,
                           out_dtype=lhs.dtype, row_scale_dtype=sdt_l, col_scale_dtype=sdt_r,
                           a_dtype=specs[0]['out_dtype'], b_dtype=b_dtype, a_k_order=k_order, row_scale_by_row=True)
    out = out.reshape(tuple(lhs.shape[:-2]) + tuple(rhs.shape[2:]))
    if not with_qt:
      return out
    mk_container = lambda spec: utils.int4 if spec['out_dtype'] == L.I4 else None
    lhs_qt_out = aqt_tensor.QTensor(
        qvalue=lq.reshape(lhs.shape) if k_order == L.K_NATURAL else None, scale=[lsc.reshape(tuple(lhs.shape[:-1]) + (1,)).to(sdt_l)], scale_t=None,
        bias=[], dequant_dtype=lhs.dtype, container_dtype=mk_container(specs[0]))
    if frozen:
      rhs_qt_out = rhs_qt
    else:
      rest = tuple(rhs.shape[2:])
      n_rest = len(rest)
      # [N, T*ts] as the kernel wrote it -> [T, ts, rest...] (a view)
      qv = rq.reshape(rest + (T, ts)).permute(tuple([n_rest, n_rest + 1] + list(range(n_rest))))
      rhs_qt_out = aqt_tensor.QTensor(
          qvalue=qv, scale=[rsc.reshape((T, 1) + rest).to(sdt_r)], scale_t=None, bias=[],
          dequant_dtype=rhs.dtype, container_dtype=mk_container(specs[1]))
    return out, (lhs_qt_out, rhs_qt_out)

  def __call__(self, lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None):
    """aqt_dot_general.py:1002-1022."""
    del preferred_element_type
    assert precision is None, f'Precision {precision} requested together with quantization.'
    out, _ = self.dg_core(lhs=lhs, rhs=rhs, lhs_qt=None, rhs_qt=None,
                          dimension_numbers=dimension_numbers)
    return out

  def assert_config_validity(self):
    """aqt_dot_general.py:1024-1078."""
    expected_fwd_quant = False
    msg_fwd_quant = (f'use_fwd_quant should be set to {expected_fwd_quant} when remaining axis are '
                     'used for calibration axis. ')
    if self.fwd.rhs.calibration_mode == CalibrationMode.REMAINING_AXIS:
      assert self.dlhs.rhs.use_fwd_quant is expected_fwd_quant, msg_fwd_quant
    if self.fwd.lhs.calibration_mode == CalibrationMode.REMAINING_AXIS:
      assert self.drhs.rhs.use_fwd_quant is expected_fwd_quant, msg_fwd_quant
    unsupported = [(DequantMode.OUTPUT, CalibrationMode.REMAINING_AXIS),
                   (DequantMode.OTHER_INPUT, CalibrationMode.CONTRACTING_AXIS)]
    msg = 'Unsupported calibration mode - dequant mode combination '
    for dequant_mode, calibration_mode in unsupported:
      assert not (self.fwd.lhs.calibration_mode == calibration_mode
                  and self.fwd.lhs.dequant_mode == dequant_mode), msg + ' for lhs.'
      assert not (self.fwd.rhs.calibration_mode == calibration_mode
                  and self.fwd.rhs.dequant_mode == dequant_mode), msg + ' for rhs.'


def clone_down_to_quantizers(cfg: 'DotGeneral', reset_calibrators: bool = False) -> 'DotGeneral':
  """New DotGeneral / DotGeneralRaw / dot-general-quantizer / Quantizer objects around the same settings
  objects (Tensor, LocalAqt, numerics, calibration factories are shared with `cfg`): everything a call
  writes to (contexts, calibrators) is private to the copy."""
  cfg = utils.clone_fields(cfg)
  for name in ('fwd', 'dlhs', 'drhs'):
    raw = utils.clone_fields(getattr(cfg, name))
    dq = utils.clone_fields(raw.dg_quantizer)
    for qn in ('lhs', 'rhs', 'lhs_mid', 'rhs_mid'):
      if hasattr(dq, qn):
        q = utils.clone_fields(getattr(dq, qn))
        if reset_calibrators:
          q._calibrator = None
        setattr(dq, qn, q)
    raw.dg_quantizer = dq
    setattr(cfg, name, raw)
  return cfg


def _fresh_cfg(cfg: 'DotGeneral') -> 'DotGeneral':
  """Copy of the config tree down to the quantizers, calibrators not yet made.

  Under jax.custom_vjp the config reaches dg_core_vjp_fwd as a pytree argument, i.e. as a
  fresh copy on every call, which is why init_calibration() may assert that it runs once;
  this gives a reused config object the same behaviour.
  """
  return clone_down_to_quantizers(cfg, reset_calibrators=True)


def dg_core_vjp_fwd(lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, cfg: DotGeneral):
  """Forward pass (aqt_dot_general.py:1098-1124)."""
  assert lhs.dtype == rhs.dtype, f'Unmatched lhs and rhs dtype: {lhs.dtype} vs {rhs.dtype}'
  cfg = _fresh_cfg(cfg)
  cfg.fwd.dg_quantizer.init_calibration()
  cfg.dlhs.dg_quantizer.init_calibration()
  cfg.drhs.dg_quantizer.init_calibration()
  ret, res = cfg.fwd(lhs, rhs, lhs_qt, rhs_qt, dimension_numbers)
  ret = ret.to(lhs.dtype)
  assert res is not None, 'res cannot be None in fwd pass.'
  qret = (res.lhs.mt.qx, res.rhs.mt.qx)
  return ((ret, qret), (res, cfg))


def _update_dimension_numbers_for_backward(fwd_dimension_numbers, y_is_lhs, gradient_rank, y_rank):
  """Dimension numbers of the contraction that turns the output gradient g and the operand y into
  the gradient of the other operand x, and the permutation that brings its result into x's axis
  order (what aqt_dot_general.py:1127-1175 computes).

  The forward output, and so g, is laid out (batch, lhs free, rhs free).  The gradient of x
  contracts g's axes that came from y's free axes with those free axes, batches over the batch
  axes, and so comes out as (batch, x free, y contraction axes in y's axis order).
  """
  (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = fwd_dimension_numbers
  if y_is_lhs:
    x_ca, x_ba, y_ca, y_ba = list(rhs_ca), list(rhs_ba), list(lhs_ca), list(lhs_ba)
  else:
    x_ca, x_ba, y_ca, y_ba = list(lhs_ca), list(lhs_ba), list(rhs_ca), list(rhs_ba)
  n_batch = len(x_ba)
  y_free = [a for a in range(y_rank) if a not in y_ca and a not in y_ba]
  x_rank = gradient_rank - len(y_free) + len(x_ca)  # g has batch + x free + y free axes
  x_free = [a for a in range(x_rank) if a not in x_ca and a not in x_ba]
  # where y's free axes sit in g: straight after the batch axes when y is the lhs, last otherwise
  first = n_batch if y_is_lhs else n_batch + len(x_free)
  g_contract = tuple(range(first, first + len(y_free)))
  dims = ((g_contract, tuple(y_free)), (tuple(range(n_batch)), tuple(y_ba)))
  # axis of x that each axis of the result stands for; y's surviving (contraction) axes appear in
  # increasing y order, each paired with its x axis
  x_ca_in_y_order = [xa for _, xa in sorted(zip(y_ca, x_ca))]
  result_is_x_axis = x_ba + x_free + x_ca_in_y_order
  out_transpose_axes = tuple(result_is_x_axis.index(a) for a in range(x_rank))
  return dims, out_transpose_axes


def dg_core_vjp_bwd(fwd_dimension_numbers, res, g):
  """Backward pass (aqt_dot_general.py:1178-1221). Returns (dlhs, drhs, None, None, None)."""
  dg_res, cfg = res
  msg = 'dg_res can only be None in 2nd derivative. It is not yet supported.'
  assert dg_res is not None, msg
  g = g[0]

  def grad_dot_general(y_res: TensorRes, quant_grad, dg_raw: DotGeneralRaw, y_is_lhs):
    dims, out_transpose_axes = _update_dimension_numbers_for_backward(
        fwd_dimension_numbers, y_is_lhs, g.dim(), y_res.mt.x.dim())
    transposed_out, _ = dg_raw(g, y_res.mt, None, None, dims, _out_transpose_axes=out_transpose_axes,
                               _bwd_memo=bwd_memo)
    if quant_grad is not None:
      assert not isinstance(quant_grad, str), quant_grad
      transposed_out = quant_grad(transposed_out)[0]
    return transposed_out

  # Both contractions calibrate the same gradient; a scale that is one number per tensor is found
  # once and shared through this table, which lives as long as this backward pass.
  bwd_memo = {}
  dlhs = grad_dot_general(dg_res.rhs, dg_res.lhs.quant_grad, cfg.dlhs, False)
  drhs = grad_dot_general(dg_res.lhs, dg_res.rhs.quant_grad, cfg.drhs, True)
  return (dlhs, drhs, None, None, None)


class _DgCoreFn(torch.autograd.Function):
  """torch.autograd stand-in for jax.custom_vjp(_dg_core) (aqt_dot_general.py:993-997)."""

  @staticmethod
  def forward(ctx, lhs, rhs, lhs_qt, rhs_qt, dimension_numbers, cfg):
    # drhs re-quantizes the lhs residual, dlhs the rhs residual, when they reuse the forward quantization
    need_l, need_r = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
    token = _RESIDUAL_ABSMAX.set(
        (bool(RESIDUAL_ABSMAX and need_r and cfg.drhs.rhs.use_fwd_quant and cfg.drhs.local_aqt is None),
         bool(RESIDUAL_ABSMAX and need_l and cfg.dlhs.rhs.use_fwd_quant and cfg.dlhs.local_aqt is None)))
    try:
      (out, (lq, rq)), (res, cfg) = dg_core_vjp_fwd(lhs.detach(), rhs.detach(), lhs_qt, rhs_qt,
                                                    dimension_numbers, cfg)
    finally:
      _RESIDUAL_ABSMAX.reset(token)
    ctx.aqt_res = (res, cfg)
    ctx.dimension_numbers = dimension_numbers
    ctx.set_materialize_grads(False)
    # QTensors are plain Python objects to autograd and pass through untouched.
    return out, lq, rq

  @staticmethod
  def backward(ctx, g, *_):
    if g is None:
      return None, None, None, None, None, None
    dlhs, drhs, *_ = dg_core_vjp_bwd(ctx.dimension_numbers, ctx.aqt_res, (g.contiguous(), None))
    return dlhs, drhs, None, None, None, None

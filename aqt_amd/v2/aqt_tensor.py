"""QTensor (mirrors aqt/jax/v2/aqt_tensor.py:55-422) on torch tensors.

`qvalue` is an int8 tensor (int4 values use an int8 container, see
`container_dtype`) or a float8 tensor; `scale` is a list of keepdims arrays.  The
qvalue of a tensor quantized by this library is often a *permuted view* of a buffer
that keeps the contraction axis contiguous; its logical shape is the operand's.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, Optional, Sequence

import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import lowering
from aqt_amd.v2 import utils

GradientFn = Optional[Callable[..., Any]]
_MSG_NO_QVALUE = (
    'QTensor does not have qvalue, but it is asked to access the qvalue.'
    ' Call QTensor.quant() before using the qvalue.')


@dataclasses.dataclass(kw_only=True)
class QTensor:
  """Quantized tensor (aqt_tensor.py:55-94)."""

  qvalue: Any
  sparsity_mask: Any = None
  # (scale == None) means that scale is unknown/invalid.
  scale: Any
  # Transposed scales, used in post dot_general scaling.
  scale_t: Any
  # len(bias) == 0 means bias should not be applied.
  bias: Any
  dequant_dtype: Any = None
  tiling_state: Any = None
  # torch has no 4-bit integer dtype: utils.int4 here marks an int8-held int4 qvalue.
  container_dtype: Any = None

  @property
  def dtype(self):
    return self.dequant_dtype if self.dequant_dtype else None

  def replace(self, **kw):
    return dataclasses.replace(self, **kw)

  def _validate_tiling_state(self):
    """aqt_tensor.py:103-113."""
    if self.tiling_state is None:
      return
    if self.is_full():
      assert tuple(self.qvalue.shape) == tuple(self.tiling_state.tiled_shape), (
          'The shape of the qvalue should be the same as the tiled shape of the tiling state. '
          f'However, {tuple(self.qvalue.shape)=} and {self.tiling_state.tiled_shape=}')

  def is_full(self) -> bool:
    return self.qvalue is not None

  def without_qvalue(self):
    return self.replace(qvalue=None)

  def astype(self, dtype):
    return self.replace(dequant_dtype=dtype)

  def quant(self, x):
    """x / scale with the reciprocal trick (aqt_tensor.py:125-159); no rounding, no cast."""
    assert not self.is_full(), 'Already quantized QTensor.'
    assert self.scale is not None, 'Missing scales to be used for quantization.'
    assert isinstance(self.scale, list), f'QTensor.scale must be a list of arrays, but got {self.scale}'
    assert isinstance(self.bias, list), f'QTensor.bias must be a list of arrays, but got {self.bias}'
    if self.tiling_state is not None:
      x = self.tiling_state.apply(x)
    qvalue = x
    for b in self.bias:
      qvalue = qvalue + b
    if self.sparsity_mask is not None:
      qvalue = qvalue * self.sparsity_mask
    for s in self.scale:
      # Scaling is fused into the quantize kernel on the fast path; this standalone form is
      # plain elementwise tensor arithmetic.
      s_inv = torch.reciprocal(s)
      s_inv = torch.where(torch.isinf(s_inv), torch.ones_like(s_inv), s_inv)
      qvalue = qvalue * s_inv
    return self.replace(qvalue=qvalue)

  def dequant(self):
    """qvalue.astype(dequant_dtype) * scale (aqt_tensor.py:161-200) via the dequantize kernel."""
    assert self.scale is not None, 'Missing scales when dequantizing a QTensor.'
    assert isinstance(self.scale, list), f'QTensor.scale must be a list of arrays, but got {self.scale}'
    assert isinstance(self.bias, list), f'QTensor.bias must be a list of arrays, but got {self.bias}'
    msg = ('QTensor is manually created without setting a dequant_dtype. It can be used in '
           'dot_general, but to dequantize you need to set its dtype.')
    assert self.dequant_dtype is not None, msg
    assert self.is_full(), _MSG_NO_QVALUE
    self._validate_tiling_state()
    q = self.qvalue
    kernel_types = (torch.int8, torch.float8_e4m3fn, torch.float8_e5m2)
    if (len(self.scale) != 1 or self.bias or self.sparsity_mask is not None
        or self.tiling_state is not None or q.dtype not in kernel_types):
      # The general form, one elementwise step per scale and bias; each product takes the
      # promoted dtype of its factors.  Integers reach bf16 through float32, as the
      # accumulator conversion of the contraction does.
      ret = q.to(self.dequant_dtype) if q.dtype.is_floating_point else q.to(torch.float32).to(self.dequant_dtype)
      for s in self.scale:
        ret = ret * s
      if self.sparsity_mask is not None:
        ret = ret * self.sparsity_mask
      for b in self.bias:
        ret = ret - b
      if self.tiling_state is not None:
        ret = self.tiling_state.unapply(ret)
      return ret.to(self.dequant_dtype)
    (s,) = self.scale
    q_dtype = qvalue_kernel_dtype(self)
    shared = [a for a in range(q.dim()) if s.shape[a] == 1 and q.shape[a] > 1]
    rest = [a for a in range(q.dim()) if a not in shared]
    v = lowering.view_operand(q, [], rest, shared)
    sv = lowering.view_operand(s, [], rest, shared)
    scale_f32 = sv.mem.reshape(-1).float().contiguous()
    if v.R * v.K == 0:
      return torch.empty(q.shape, dtype=self.dequant_dtype, device=q.device)
    per_tensor = scale_f32.numel() == 1
    reduce = L.REDUCE_ALL_BATCH if per_tensor else (L.REDUCE_COLS if v.k_last else L.REDUCE_ROWS)
    mem = v.mem.view(torch.uint8) if v.mem.dtype != torch.int8 else v.mem
    out = ops.dequantize(mem, scale_f32, reduce=reduce, q_dtype=q_dtype, out_dtype=self.dequant_dtype,
                         scale_dtype=s.dtype)
    # out is [B=1, rows, cols] in the memory order of the view
    dims = [v.shape[a] for a in (v.r_axes + v.k_axes if v.k_last else v.k_axes + v.r_axes)]
    axes = v.r_axes + v.k_axes if v.k_last else v.k_axes + v.r_axes
    inv = [0] * len(axes)
    for pos, a in enumerate(axes):
      inv[a] = pos
    return out.reshape(dims).permute(tuple(inv))

  def qvalue_astype(self, dtype):
    assert self.is_full(), _MSG_NO_QVALUE
    return self.replace(qvalue=self.qvalue.to(dtype))

  def __getitem__(self, idx):
    assert self.scale_t is None, 'scale_t is not supported in __getitem__'
    assert self.is_full(), _MSG_NO_QVALUE
    self._validate_tiling_state()
    return QTensor(qvalue=self.qvalue[idx], scale=[s[idx] for s in self.scale], scale_t=self.scale_t,
                   bias=self.bias, dequant_dtype=self.dequant_dtype,
                   container_dtype=self.container_dtype)

  @property
  def ndim(self) -> int:
    assert self.is_full(), _MSG_NO_QVALUE
    self._validate_tiling_state()
    if self.tiling_state is not None:
      return len(self.tiling_state.untiled_shape)
    return self.qvalue.dim()

  @property
  def shape(self) -> Sequence[int]:
    assert self.is_full(), _MSG_NO_QVALUE
    self._validate_tiling_state()
    if self.tiling_state is not None:
      return tuple(self.tiling_state.untiled_shape)
    return tuple(self.qvalue.shape)

  def __len__(self) -> int:
    assert self.qvalue is not None, _MSG_NO_QVALUE
    return len(self.qvalue)


def qvalue_kernel_dtype(qt: QTensor) -> int:
  """Kernel element type of qt.qvalue."""
  q = qt.qvalue
  if q.dtype == torch.int8:
    return L.I4 if qt.container_dtype is utils.int4 else L.I8
  if q.dtype == torch.float8_e4m3fn:
    return L.E4M3
  if q.dtype == torch.float8_e5m2:
    return L.E5M2
  raise TypeError(f'qvalue dtype {q.dtype} is not a quantized type')


def zeros(shape, *, container_dtype, dequant_dtype=torch.bfloat16, device='cuda') -> QTensor:
  """aqt_tensor.py:245-255."""
  return QTensor(qvalue=torch.zeros(tuple(shape), dtype=container_dtype, device=device), scale=[],
                 scale_t=None, bias=[], dequant_dtype=dequant_dtype)


def zeros_with_scale(shape, calibration_axis, *, container_dtype, scale_dtype=None,
                     dequant_dtype=torch.bfloat16, device='cuda') -> QTensor:
  """aqt_tensor.py:258-280."""
  scale_shape = list(shape)
  for axis in calibration_axis:
    scale_shape[axis] = 1
  scale_dtype = scale_dtype or dequant_dtype
  return QTensor(qvalue=torch.zeros(tuple(shape), dtype=container_dtype, device=device),
                 scale=[torch.ones(scale_shape, dtype=scale_dtype, device=device)], scale_t=None,
                 bias=[], dequant_dtype=dequant_dtype)


def dynamic_slice(operand: QTensor, start_indices, slice_sizes) -> QTensor:
  """aqt_tensor.py:315-353."""
  msg = '{attribute} is not supported in the dynamic_slice of a QTensor.'
  assert operand.scale_t is None, msg.format(attribute='scale_t')
  assert not operand.bias, msg.format(attribute='bias')

  def sl(t, starts, sizes):
    return t[tuple(slice(int(b), int(b) + int(n)) for b, n in zip(starts, sizes))]

  def sliced_scale(scale):
    assert scale.dim() == len(slice_sizes), 'Slice sizes must have the same length as operand dims.'
    starts, sizes = list(start_indices), list(slice_sizes)
    for axis in range(len(sizes)):
      if scale.shape[axis] == 1:
        starts[axis], sizes[axis] = 0, 1
      assert starts[axis] + sizes[axis] <= scale.shape[axis], (
          'We do not support window overflow that is supported in jax.lax.dynamic_slices.')
    return sl(scale, starts, sizes)

  return QTensor(qvalue=sl(operand.qvalue, start_indices, slice_sizes),
                 scale=[sliced_scale(s) for s in operand.scale], scale_t=None, bias=[],
                 dequant_dtype=operand.dequant_dtype, container_dtype=operand.container_dtype)


def dynamic_update_slice(operand: QTensor, update: QTensor, start_indices) -> QTensor:
  """aqt_tensor.py:356-402: only whole slices along the calibration axis."""
  assert operand.scale_t is None, 'scale_t is not supported in dynamic_update_slice'
  assert operand.dequant_dtype == update.dequant_dtype, (
      f'Dequant dtype mismatch: {operand.dequant_dtype} != {update.dequant_dtype}')
  ndim = operand.qvalue.dim()
  assert update.qvalue.dim() == ndim
  for scale, update_scale in zip(operand.scale, update.scale):
    assert scale.dim() == ndim and update_scale.dim() == ndim
    for axis in range(ndim):
      if scale.shape[axis] == 1:
        assert update.qvalue.shape[axis] == operand.qvalue.shape[axis], (
            'Only updating an entire slice along the calibration axis is valid.')
        assert update_scale.shape[axis] == 1, (
            'Update scale and scale should be calibrated along the same axis.')

  def upd(dst, src, starts):
    out = dst.clone()
    idx = tuple(slice(int(b), int(b) + n) for b, n in zip(starts, src.shape))
    out[idx] = src
    return out

  def scale_starts(scale):
    return [0 if scale.shape[a] == 1 else start_indices[a] for a in range(ndim)]

  return QTensor(qvalue=upd(operand.qvalue, update.qvalue, start_indices),
                 scale=[upd(s, u, scale_starts(s)) for s, u in zip(operand.scale, update.scale)],
                 scale_t=None, bias=[], dequant_dtype=operand.dequant_dtype,
                 container_dtype=operand.container_dtype)


def update_frame(operand: QTensor, frame: int, update: QTensor) -> QTensor:
  """aqt_tensor.py:405-422."""
  assert operand.ndim == update.ndim + 1
  assert operand.dequant_dtype == update.dequant_dtype, 'Dequant dtype mismatch'

  def set_frame(dst, src):
    out = dst.clone()
    out[frame] = src
    return out

  return QTensor(qvalue=set_frame(operand.qvalue, update.qvalue),
                 scale=[set_frame(t, u) for t, u in zip(operand.scale, update.scale)], scale_t=None,
                 bias=[set_frame(t, u) for t, u in zip(operand.bias, update.bias)],
                 dequant_dtype=operand.dequant_dtype, container_dtype=operand.container_dtype)

"""Quantized conv_general_dilated, forward (mirrors aqt/jax/v2/aqt_conv_general.py:33-228).

The reference quantizes the input per batch element and the kernel per output feature, runs
`lax.conv_general_dilated` on the quantized values and multiplies the result by both scales.
Here the convolution is an implicit-GEMM: the (padded, strided, dilated) windows of the
quantized input are gathered (aqtx_im2col_i8) into a [batch * positions, window * features] int8 matrix and
contracted with the [out features, window * features] kernel matrix on the int8 MFMA kernel
(exact int32 accumulators, both scales applied in its epilogue); float-held or unquantized
operands take a float matrix product.
Flax layout only (NHWC input, HWIO kernel), as in the reference; no feature / batch groups and
no input dilation.
"""
from __future__ import annotations

import collections
import math
from typing import Optional, Sequence, Tuple

import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import aqt_dot_general
from aqt_amd.v2 import aqt_tensor

ConvDimensionNumbers = collections.namedtuple('ConvDimensionNumbers', ['lhs_spec', 'rhs_spec', 'out_spec'])


def flax_conv_dimension_numbers(input_shape) -> ConvDimensionNumbers:
  """The dimension numbers flax.linen.Conv uses: input N...C, kernel ...IO, output N...C."""
  ndim = len(input_shape)
  lhs_spec = (0, ndim - 1) + tuple(range(1, ndim - 1))
  rhs_spec = (ndim - 1, ndim - 2) + tuple(range(0, ndim - 2))
  return ConvDimensionNumbers(lhs_spec, rhs_spec, lhs_spec)


def _conv_weight_matrix(rq, k, cout):
  """The quantized kernel [*window, features_in, features_out] as the contraction's column operand
  [features_out, window * features_in] (k contiguous)."""
  return rq.reshape(k, cout).t().contiguous()


def _explicit_padding(padding, in_sizes, eff_kernel, strides):
  if isinstance(padding, str):
    if padding.upper() == 'VALID':
      return [(0, 0)] * len(in_sizes)
    if padding.upper() == 'SAME':
      pads = []
      for size, k, s in zip(in_sizes, eff_kernel, strides):
        out = -(-size // s)
        total = max((out - 1) * s + k - size, 0)
        pads.append((total // 2, total - total // 2))
      return pads
    raise ValueError(f'unknown padding {padding}')
  return [(int(lo), int(hi)) for lo, hi in padding]


def _windows(x: torch.Tensor, kernel, strides, pads, dilation) -> Tuple[torch.Tensor, Sequence[int]]:
  """x [N, *spatial, C] -> ([N * positions, prod(kernel) * C], output spatial sizes); the window
  axes are ordered like the kernel's spatial axes, features innermost."""
  ns = len(kernel)
  flat_pad = []
  for lo, hi in reversed(pads):  # F.pad lists the last axis first
    flat_pad += [lo, hi]
  if any(flat_pad):
    x = torch.nn.functional.pad(x, [0, 0] + flat_pad)
  for d in range(ns):
    eff = (kernel[d] - 1) * dilation[d] + 1
    x = x.unfold(1 + d, eff, strides[d])  # the window lands on a new last axis
    if dilation[d] != 1:
      x = x[..., ::dilation[d]]
  # [N, out..., C, win...] -> [N, out..., win..., C]
  out_sizes = list(x.shape[1:1 + ns])
  perm = [0] + list(range(1, 1 + ns)) + list(range(2 + ns, 2 + 2 * ns)) + [1 + ns]
  x = x.permute(perm)
  return x.reshape(x.shape[0] * math.prod(out_sizes), -1), out_sizes


def lax_conv_general_dilated(lhs, rhs, window_strides, padding, lhs_dilation=None, rhs_dilation=None,
                             dimension_numbers=None, feature_group_count=1, batch_group_count=1,
                             precision=None, preferred_element_type=None):
  """jax.lax.conv_general_dilated for the Flax layout on torch tensors."""
  del precision
  rank = lhs.dim()
  ns = rank - 2
  assert dimension_numbers is not None and tuple(dimension_numbers.lhs_spec[:2]) == (0, rank - 1)
  if feature_group_count != 1 or batch_group_count != 1:
    raise NotImplementedError('feature_group_count / batch_group_count other than 1')
  if lhs_dilation is not None and any(int(d) != 1 for d in lhs_dilation):
    raise NotImplementedError('lhs_dilation (transposed convolution)')
  strides = [int(s) for s in window_strides]
  dilation = [int(d) for d in rhs_dilation] if rhs_dilation is not None else [1] * ns
  kernel = list(rhs.shape[:ns])
  eff = [(k - 1) * d + 1 for k, d in zip(kernel, dilation)]
  pads = _explicit_padding(padding, list(lhs.shape[1:1 + ns]), eff, strides)
  n, cin, cout = lhs.shape[0], lhs.shape[-1], rhs.shape[-1]
  assert rhs.shape[-2] == cin, (lhs.shape, rhs.shape)
  both_int = lhs.dtype == torch.int8 and rhs.dtype == torch.int8
  if both_int and ns <= 3:
    a, out_sizes = ops.im2col_i8(lhs.contiguous(), kernel, strides, pads, dilation)  # [N*P, K]
  else:
    a, out_sizes = _windows(lhs, kernel, strides, pads, dilation)
  k = a.shape[1]
  b = rhs.reshape(k, cout).t().contiguous()  # [O, K]
  if both_int:
    if a.shape[0] * cout == 0 or k == 0:
      out = torch.zeros((a.shape[0], cout), dtype=torch.int32, device=lhs.device)
    else:
      out = ops.gemm(a.contiguous()[None], b[None], row_scale=None, col_scale=None, out_dtype=torch.int32,
                     a_dtype=L.I8, b_dtype=L.I8)[0]
    if preferred_element_type is not None:
      out = out.to(preferred_element_type)
  else:
    common = torch.promote_types(lhs.dtype, rhs.dtype)
    acc = preferred_element_type if preferred_element_type is not None else common
    wide = torch.float32 if common in (torch.bfloat16, torch.float16) else common
    out = torch.matmul(a.to(wide), b.to(wide).t()).to(acc)
  return out.reshape([n] + list(out_sizes) + [cout])


def _fused_int8_conv(lhs_qt, rhs_qt, out_dtype, window_strides, padding, lhs_dilation, rhs_dilation,
                     feature_group_count, batch_group_count, preferred_element_type):
  """int8 x int8 with one scale per batch element and one per output feature: the contraction
  kernel dequantizes in its epilogue (accumulator -> out dtype, times the lhs scale, times the rhs
  scale: QTensor.dequant's order, aqt_tensor.py:179-183).  None if the call is not of that form."""
  lq, rq = lhs_qt.qvalue, rhs_qt.qvalue
  rank = lq.dim()
  if not (lq.dtype == torch.int8 and rq.dtype == torch.int8 and len(lhs_qt.scale) == 1 and len(rhs_qt.scale) == 1
          and not lhs_qt.bias and not rhs_qt.bias and preferred_element_type in (None, out_dtype)
          and out_dtype in (torch.bfloat16, torch.float32)
          and feature_group_count == 1 and batch_group_count == 1
          and (lhs_dilation is None or all(int(d) == 1 for d in lhs_dilation))):
    return None
  ls, rs = lhs_qt.scale[0], rhs_qt.scale[0]
  n, cout = lq.shape[0], rq.shape[-1]
  if tuple(ls.shape) != (n,) + (1,) * (rank - 1) or tuple(rs.shape) != (1,) * (rank - 1) + (cout,):
    return None
  if ls.dtype not in (torch.bfloat16, torch.float32) or rs.dtype not in (torch.bfloat16, torch.float32):
    return None
  ns = rank - 2
  strides = [int(x) for x in window_strides]
  dilation = [int(d) for d in rhs_dilation] if rhs_dilation is not None else [1] * ns
  kernel = list(rq.shape[:ns])
  eff = [(k - 1) * d + 1 for k, d in zip(kernel, dilation)]
  pads = _explicit_padding(padding, list(lq.shape[1:1 + ns]), eff, strides)
  if ns > 3:
    return None
  lq = lq.contiguous()
  if ops.conv_i8_supported(lq) and lq.shape[0] * cout > 0:
    # features in multiples of 128: one kernel reads the windows in place, no window matrix
    k = math.prod(kernel) * lq.shape[-1]
    _, out_sizes = ops._window_plan(lq, kernel, strides, pads, dilation)  # pylint: disable=protected-access
    positions = math.prod(out_sizes)
    if positions > 0:
      b = _conv_weight_matrix(rq, k, cout)
      row_scale = ls.reshape(n, 1).float().expand(n, positions).reshape(n * positions).contiguous()
      out, out_sizes = ops.conv_i8(lq, b, kernel, strides, pads, dilation, row_scale=row_scale,
                                   col_scale=rs.reshape(cout).float().contiguous(), out_dtype=out_dtype,
                                   row_scale_dtype=ls.dtype, col_scale_dtype=rs.dtype)
      return out.reshape([n] + list(out_sizes) + [cout])
  a, out_sizes = ops.im2col_i8(lq, kernel, strides, pads, dilation)
  k = a.shape[1]
  positions = math.prod(out_sizes)
  if a.shape[0] * cout == 0 or k == 0:
    return None
  b = _conv_weight_matrix(rq, k, cout)
  row_scale = ls.reshape(n, 1).float().expand(n, positions).reshape(1, n * positions).contiguous()
  out = ops.gemm(a.contiguous()[None], b[None], row_scale=row_scale, col_scale=rs.reshape(1, cout).float().contiguous(),
                 out_dtype=out_dtype, dequant_dtype=out_dtype, row_scale_dtype=ls.dtype, col_scale_dtype=rs.dtype,
                 a_dtype=L.I8, b_dtype=L.I8)[0]
  return out.reshape([n] + list(out_sizes) + [cout])


def make_conv_general_dilated_with_qt(cfg: aqt_dot_general.DotGeneralRaw):
  """Quantized conv_general_dilated that also returns the QTensors (aqt_conv_general.py:33-135)."""
  assert cfg is not None, 'Missing config for make_conv_general_dilated'

  def my_conv_general_dilated(lhs, rhs, window_strides, padding, lhs_qt: Optional[aqt_tensor.QTensor] = None,
                              rhs_qt: Optional[aqt_tensor.QTensor] = None, lhs_dilation=None, rhs_dilation=None,
                              dimension_numbers=None, feature_group_count=1, batch_group_count=1,
                              precision=None, preferred_element_type=None):
    msg1 = ('To simplify the code, we currently assume a Flax-particular layout of the data. This makes '
            'sense, because this is the main use-case of this function. However if there is any other '
            'use, we will drop that assumption.')
    rank = lhs.dim()
    assert rhs.dim() == rank
    assert dimension_numbers is not None, msg1
    assert tuple(dimension_numbers.lhs_spec[0:2]) == (0, rank - 1), msg1
    assert tuple(dimension_numbers.rhs_spec[0:2]) == (rank - 1, rank - 2), msg1
    assert tuple(dimension_numbers.out_spec[0:2]) == (0, rank - 1), msg1
    msg = ('Convolution formula does not follow flax assumption. This could be because spatial '
           'dimensions was incorrectly set during DotGeneralRaw creation. Please double check the '
           'parameter in #conv_general_dilated_make().')
    cfg.dg_quantizer.assert_calib_shared_axes_value(list(range(1, rank)), list(range(0, rank - 1)), msg)
    (lhs, lhs_incomplete_qt), (rhs, rhs_incomplete_qt) = cfg.dg_quantizer.calibrate(lhs, rhs, None, None, None)
    if lhs_qt is not None and not lhs_qt.is_full():
      lhs_incomplete_qt, lhs_qt = lhs_qt, None
    if rhs_qt is not None and not rhs_qt.is_full():
      rhs_incomplete_qt, rhs_qt = rhs_qt, None
    (lhs_calc, _), (rhs_calc, _) = cfg.dg_quantizer.calculate_qvalue(lhs, lhs_incomplete_qt, rhs, rhs_incomplete_qt)
    lhs_qt = lhs_qt if lhs_qt is not None else lhs_calc
    rhs_qt = rhs_qt if rhs_qt is not None else rhs_calc

    # The reference casts both qvalues to the float dtype and convolves in float; integer
    # qvalues are contracted exactly on the int8 kernel instead and cast afterwards, which is
    # the same number whenever the float accumulation is exact.
    lq, rq = lhs_qt.qvalue, rhs_qt.qvalue
    out_dtype = torch.promote_types(lhs.dtype, rhs.dtype)
    both_int = lq.dtype == torch.int8 and rq.dtype == torch.int8
    fused = _fused_int8_conv(lhs_qt, rhs_qt, out_dtype, window_strides, padding, lhs_dilation, rhs_dilation,
                             feature_group_count, batch_group_count, preferred_element_type)
    if fused is not None:
      return fused, (lhs_qt, rhs_qt)
    acc = lax_conv_general_dilated(
        lq.contiguous() if both_int else lq.to(lhs.dtype), rq.contiguous() if both_int else rq.to(rhs.dtype),
        window_strides=window_strides, padding=padding, lhs_dilation=lhs_dilation, rhs_dilation=rhs_dilation,
        dimension_numbers=dimension_numbers, feature_group_count=feature_group_count,
        batch_group_count=batch_group_count, precision=precision,
        preferred_element_type=torch.int32 if both_int else preferred_element_type)
    if both_int:
      acc = acc.to(torch.float32).to(preferred_element_type if preferred_element_type is not None else out_dtype)
    out = aqt_tensor.QTensor(qvalue=acc, scale=[], scale_t=None, bias=[], dequant_dtype=out_dtype)
    out.scale.extend(lhs_qt.scale)
    out.scale.extend(rhs_qt.scale)
    return out.dequant(), (lhs_qt, rhs_qt)

  return my_conv_general_dilated


def make_conv_general_dilated(cfg: aqt_dot_general.DotGeneralRaw):
  """Quantized lax.conv_general_dilated replacement (aqt_conv_general.py:138-175)."""
  assert cfg is not None, 'Missing config for make_conv_general_dilated'
  with_qt = make_conv_general_dilated_with_qt(cfg)

  def my_conv_general_dilated(lhs, rhs, window_strides, padding, lhs_dilation=None, rhs_dilation=None,
                              dimension_numbers=None, feature_group_count=1, batch_group_count=1,
                              precision=None, preferred_element_type=None):
    out, _ = with_qt(lhs, rhs, window_strides, padding, lhs_qt=None, rhs_qt=None, lhs_dilation=lhs_dilation,
                     rhs_dilation=rhs_dilation, dimension_numbers=dimension_numbers,
                     feature_group_count=feature_group_count, batch_group_count=batch_group_count,
                     precision=precision, preferred_element_type=preferred_element_type)
    return out

  return my_conv_general_dilated


def conv_general_dilated_make(spatial_dimensions: int, lhs_bits: Optional[int] = None,
                              rhs_bits: Optional[int] = None,
                              initialize_calibration: bool = True) -> aqt_dot_general.DotGeneralRaw:
  """The DotGeneralRaw to inject as conv_general_dilated (aqt_conv_general.py:178-228): the input
  shares a scale over everything but the batch axis, the kernel over everything but the output
  features."""
  config = aqt_dot_general.dot_general_raw_make(lhs_bits, rhs_bits, initialize_calibration=initialize_calibration)
  lhs_calib_shared_axes = list(range(1, spatial_dimensions + 2)) if config.lhs else None
  rhs_calib_shared_axes = list(range(0, spatial_dimensions + 2 - 1)) if config.rhs else None
  assert isinstance(config.dg_quantizer, aqt_dot_general.DefaultDotGeneralQuantizer)
  config.dg_quantizer.lhs.calib_shared_axes = lhs_calib_shared_axes
  config.dg_quantizer.rhs.calib_shared_axes = rhs_calib_shared_axes
  return config

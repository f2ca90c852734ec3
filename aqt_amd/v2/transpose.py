"""Scale re-layout helpers (mirrors aqt/jax/v2/transpose.py:29-285). No arithmetic."""
from __future__ import annotations

from typing import Sequence

import torch

from aqt_amd.v2 import utils


def transpose(t: torch.Tensor, axes: Sequence[int]) -> torch.Tensor:
  """transpose.py:29-95 (a permute; torch views make the reshape shortcut moot)."""
  return t.permute(tuple(axes))


def _scale_trans(x, ca, ba):
  """transpose.py:98-111."""
  ca, ba = list(ca), list(ba)
  for i in ca:
    assert x.shape[i] == 1, (x.shape, ca, ba)
  ra = utils.get_remaining_axes(x.dim(), ca, ba)
  x = transpose(x, ba + ra + ca)
  return x.reshape(x.shape[: len(ba) + len(ra)])


def lhs_scale_transpose_to_output(lhs_scale, dimension_numbers, lhs_shape, rhs_shape):
  """transpose.py:114-132."""
  if lhs_scale is None:
    return None
  (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = dimension_numbers
  t = _scale_trans(lhs_scale, lhs_ca, lhs_ba)
  assert t.dim() == len(lhs_shape) - len(lhs_ca)
  n_rhs_ra = len(rhs_shape) - len(rhs_ca) - len(rhs_ba)
  return t.reshape(tuple(t.shape) + (1,) * n_rhs_ra)


def rhs_scale_transpose_to_output(rhs_scale, dimension_numbers, lhs_shape, rhs_shape):
  """transpose.py:135-148."""
  if rhs_scale is None:
    return None
  del rhs_shape
  (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = dimension_numbers
  t = _scale_trans(rhs_scale, rhs_ca, rhs_ba)
  nb = len(rhs_ba)
  n_lhs_ra = len(lhs_shape) - len(lhs_ca) - len(lhs_ba)
  return t.reshape(tuple(t.shape[:nb]) + (1,) * n_lhs_ra + tuple(t.shape[nb:]))


def _scale_trans_back(scale_t, ca, ba):
  """transpose.py:151-180."""
  ca, ba = list(ca), list(ba)
  scale = scale_t.reshape(tuple(scale_t.shape) + (1,) * len(ca))
  ra = utils.get_remaining_axes(scale.dim(), ca, ba)
  back = [-1] * len(ba + ra + ca)
  for axis_orig, axis_transposed in enumerate(ba + ra + ca):
    back[axis_transposed] = axis_orig
  assert -1 not in back
  return transpose(scale, back)


def lhs_recover_scale_from_scale_t(lhs_scale_t, dimension_numbers, lhs_shape, rhs_shape):
  """transpose.py:183-197."""
  (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = dimension_numbers
  start = len(lhs_shape) - len(lhs_ca)
  rhs_ra_ndim = len(rhs_shape) - len(rhs_ca) - len(rhs_ba)
  shape = list(lhs_scale_t.shape)
  for ax in range(start, start + rhs_ra_ndim):
    assert shape[ax] == 1
  lhs_scale = lhs_scale_t.reshape(shape[:start] + shape[start + rhs_ra_ndim:])
  return _scale_trans_back(lhs_scale, lhs_ca, lhs_ba)


def rhs_recover_scale_from_scale_t(rhs_scale_t, dimension_numbers, lhs_shape, rhs_shape):
  """transpose.py:200-215."""
  del rhs_shape
  (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = dimension_numbers
  start = len(rhs_ba)
  end = len(lhs_shape) - len(lhs_ca) - len(lhs_ba) + start
  shape = list(rhs_scale_t.shape)
  for ax in range(start, end):
    assert shape[ax] == 1
  rhs_scale = rhs_scale_t.reshape(shape[:start] + shape[end:])
  return _scale_trans_back(rhs_scale, rhs_ca, rhs_ba)


def _scale_trans_for_other_input(x, my_ca, my_ba, other_ca, other_ba, other_rank):
  """transpose.py:218-263."""
  my_ca, my_ba = list(my_ca), list(my_ba)
  other_ca, other_ba = list(other_ca), list(other_ba)
  if x.dim() < other_rank:
    x = x.reshape(list(x.shape) + [1] * (other_rank - x.dim()))
  transpose_dim = [-1] * x.dim()
  my_ra = utils.get_remaining_axes(x.dim(), my_ca, my_ba)
  for axis in my_ra:
    assert x.shape[axis] == 1
  for my_axis, other_axis in zip(my_ca + my_ba, other_ca + other_ba):
    transpose_dim[other_axis] = my_axis
  ra_idx = 0
  for i, v in enumerate(transpose_dim):
    if v == -1:
      transpose_dim[i] = my_ra[ra_idx]
      ra_idx += 1
  assert ra_idx == len(my_ra)
  x = transpose(x, transpose_dim)
  if x.dim() > other_rank:
    for idx in range(other_rank, x.dim()):
      assert x.shape[idx] == 1
    x = x.reshape(x.shape[:other_rank])
  return x


def lhs_scale_transpose_for_rhs_input(lhs_scale, dimension_numbers, rhs_shape):
  """transpose.py:266-274."""
  if lhs_scale is None:
    return None
  (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = dimension_numbers
  return _scale_trans_for_other_input(lhs_scale, lhs_ca, lhs_ba, rhs_ca, rhs_ba, len(rhs_shape))


def rhs_scale_transpose_for_lhs_input(rhs_scale, dimension_numbers, lhs_shape):
  """transpose.py:277-285."""
  if rhs_scale is None:
    return None
  (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = dimension_numbers
  return _scale_trans_for_other_input(rhs_scale, rhs_ca, rhs_ba, lhs_ca, lhs_ba, len(lhs_shape))

"""Quantized ragged_dot (mirrors aqt/jax/v2/aqt_ragged_dot.py:22-86), forward only.

`lhs` [m, k] holds the rows of `g` groups one after the other, `rhs` [g, k, n] one matrix per
group, `group_sizes` [g] the row counts: out[rows of group i] = lhs[rows of group i] @ rhs[i].
The contraction is plugged into `DotGeneralRaw.dot_general`, so calibration, quantization and
dequantisation are the ordinary ones; the int8 groups run on the MFMA contraction kernel in one
launch: every workgroup looks its group's row range up in a device-side offset table.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Optional, Sequence

import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import aqt_dot_general
from aqt_amd.v2 import config


def _host_group_sizes(group_sizes) -> Sequence[int]:
  # The launches are sized on the host: a device tensor is copied back (a synchronisation).
  if isinstance(group_sizes, torch.Tensor):
    return [int(v) for v in group_sizes.detach().cpu().tolist()]
  return [int(v) for v in group_sizes]


def lax_ragged_dot(lhs, rhs, group_sizes, precision=None, preferred_element_type=None):
  """jax.lax.ragged_dot on torch tensors: int8 x int8 -> int32 on the MFMA kernel (all groups in
  one launch, row ranges from a device-side offset table), anything else as float contractions;
  rows past sum(group_sizes) are zero."""
  del precision
  assert lhs.dim() == 2 and rhs.dim() == 3 and lhs.shape[1] == rhs.shape[1], (lhs.shape, rhs.shape)
  m, k = lhs.shape
  n = rhs.shape[2]
  assert len(group_sizes) == rhs.shape[0], (len(group_sizes), rhs.shape)
  both_int = lhs.dtype == torch.int8 and rhs.dtype == torch.int8
  if both_int:
    assert preferred_element_type == torch.int32, (
        f'{preferred_element_type=}: int8 operands are contracted into int32 accumulators only')
    if m * n == 0 or k == 0 or rhs.shape[0] == 0:
      return torch.zeros((m, n), dtype=torch.int32, device=lhs.device)
    a = lhs if lhs.stride(1) == 1 else lhs.contiguous()
    bt = rhs.permute(0, 2, 1)  # [g, n, k]: the quantizer already wrote the weights k-contiguous
    if bt.stride(2) != 1:
      bt = bt.contiguous()
    aligned = (k % 16 == 0 and a.stride(0) % 16 == 0 and bt.stride(1) % 16 == 0 and bt.stride(0) % 16 == 0
               and a.data_ptr() % 16 == 0 and bt.data_ptr() % 16 == 0)
    if aligned:
      return ops.gemm(a[None], bt, row_scale=None, col_scale=None, out_dtype=torch.int32, a_dtype=L.I8,
                      b_dtype=L.I8, group_offsets=ops.ragged_offsets(group_sizes, m, lhs.device))[0]
  # one contraction per group on row slices (sizes read on the host: a synchronisation when they
  # live on the device)
  sizes = _host_group_sizes(group_sizes)
  assert sum(sizes) <= m, f'group sizes {sizes} exceed the {m} rows of lhs'
  if both_int:
    out = torch.zeros((m, n), dtype=torch.int32, device=lhs.device)
  else:
    common = torch.promote_types(lhs.dtype, rhs.dtype)
    out_dtype = preferred_element_type if preferred_element_type is not None else common
    out = torch.zeros((m, n), dtype=out_dtype, device=lhs.device)
  start = 0
  for g, size in enumerate(sizes):
    if size == 0:
      continue
    rows = slice(start, start + size)
    if both_int:
      out[rows] = ops.gemm(a[rows][None], bt[g][None], row_scale=None, col_scale=None,
                           out_dtype=torch.int32, a_dtype=L.I8, b_dtype=L.I8)[0]
    else:
      out[rows] = torch.matmul(lhs[rows].to(common), rhs[g].to(common)).to(out.dtype)
    start += size
  return out


@dataclasses.dataclass(kw_only=True)
class RaggedDot:
  """Slot for DotGeneralRaw.dot_general (aqt_ragged_dot.py:22-46).

  Attributes:
    group_sizes: the sizes of the groups, shape [g].
  """
  group_sizes: Any
  is_ragged_dot = True  # DotGeneralRaw lowers this hook to the fused kernels when it can

  def __call__(self, lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None):
    del dimension_numbers
    return lax_ragged_dot(lhs, rhs, self.group_sizes, precision=precision,
                          preferred_element_type=preferred_element_type)


def ragged_dot(lhs, rhs, group_sizes, precision=None, preferred_element_type=None,
               cfg: Optional[aqt_dot_general.DotGeneral] = None):
  """Quantized version of jax.lax.ragged_dot (aqt_ragged_dot.py:49-86); forward pass only.

  Args:
    lhs: [m, k].
    rhs: [g, k, n].
    group_sizes: [g].
    precision: must be None when quantization is enabled.
    preferred_element_type: ignored.
    cfg: the DotGeneral configuration; config_v4() when None.
  """
  if cfg is None:
    cfg = config.config_v4()
  cfg.fwd.dot_general = RaggedDot(group_sizes=group_sizes)
  # One scale for all the experts in the rhs: the rhs calibration axes are [0, 1] although
  # only axis 1 is contracted.
  dimension_numbers = ([1], [0, 1]), ([], [])
  return cfg(lhs, rhs, dimension_numbers=dimension_numbers, precision=precision,
             preferred_element_type=preferred_element_type)

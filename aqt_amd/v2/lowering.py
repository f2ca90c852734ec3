"""Lowers an operand of dot_general to the [batch, rows, cols] plans of the HIP kernels.

Nothing here has a counterpart in the reference, where XLA picks layouts.  An
operand whose axes fall, in memory order, into (batch axes, remaining axes,
contraction axes) or (batch, contraction, remaining) is viewed in place as a 3-D
tensor; the quantize kernel then writes the quantized values with the contraction
axis contiguous (transposing through LDS in the second case), which is the layout
the MFMA contraction kernels read.  Any other axis order is first copied into the
canonical one (a plain permute copy, no arithmetic).
"""
from __future__ import annotations

import dataclasses
import math
from typing import Any, List, Optional, Sequence, Tuple

import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import utils


class NotFused(NotImplementedError):
  """The fused kernels do not implement this configuration; the step-by-step path takes it."""


def _prod(xs):
  return int(math.prod(xs))


@dataclasses.dataclass
class OperandView:
  mem: torch.Tensor            # contiguous [B, R0, R1]
  k_last: bool                 # memory is [B, R, K] (else [B, K, R])
  b_axes: List[int]
  r_axes: List[int]
  k_axes: List[int]
  shape: Tuple[int, ...]       # logical shape of the operand
  noise_strides: Optional[Tuple[int, int, int]]  # counter strides of (B, R, K), None if not mergeable
  copied: bool

  @property
  def B(self):
    return _prod(self.shape[a] for a in self.b_axes)

  @property
  def R(self):
    return _prod(self.shape[a] for a in self.r_axes)

  @property
  def K(self):
    return _prod(self.shape[a] for a in self.k_axes)


def memory_rank(x: torch.Tensor):
  """Axes of extent > 1 in memory order (outermost first), and whether x is dense."""
  big = [a for a in range(x.dim()) if x.shape[a] > 1]
  order = sorted(big, key=lambda a: (-x.stride(a), a))
  expect, dense = 1, True
  for a in reversed(order):
    if x.stride(a) != expect:
      dense = False
    expect *= x.shape[a]
  return order, dense


def _merged_stride(shape, axes):
  """Row-major counter stride of the flattened `axes` group, or None if it does not nest."""
  if not axes:
    return 0
  ls = [0] * len(shape)
  acc = 1
  for a in reversed(range(len(shape))):
    ls[a] = acc
    acc *= shape[a]
  big = [a for a in axes if shape[a] > 1]
  for a0, a1 in zip(big[:-1], big[1:]):
    if ls[a0] != ls[a1] * shape[a1]:
      return None
  return ls[big[-1]] if big else 0


def view_operand(x: torch.Tensor, ba: Sequence[int], ra: Sequence[int], ca: Sequence[int]) -> OperandView:
  """3-D view of x with the groups flattened in the listed axis orders."""
  ba, ra, ca = list(ba), list(ra), list(ca)
  shape = tuple(x.shape)
  order, dense = memory_rank(x)
  group_of = {}
  for a in ba:
    group_of[a] = 'b'
  for a in ra:
    group_of[a] = 'r'
  for a in ca:
    group_of[a] = 'k'
  seq = [group_of[a] for a in order]
  pattern = [g for i, g in enumerate(seq) if i == 0 or seq[i - 1] != g]
  within_ok = all(
      [a for a in order if group_of[a] == g] == [a for a in grp if shape[a] > 1]
      for g, grp in (('b', ba), ('r', ra), ('k', ca)))

  def is_subseq(p, full):
    it = iter(full)
    return all(any(c == f for f in it) for c in p)

  copied = False
  if dense and within_ok and len(set(pattern)) == len(pattern) and is_subseq(pattern, ['b', 'r', 'k']):
    k_last = True
  elif dense and within_ok and len(set(pattern)) == len(pattern) and is_subseq(pattern, ['b', 'k', 'r']):
    k_last = False
  else:
    x = x.permute(tuple(ba + ra + ca)).contiguous()
    # after the copy the logical axes are renumbered; keep the caller's numbering for shapes only
    b_n, r_n = len(ba), len(ra)
    mem = x.reshape(_prod(x.shape[:b_n]), _prod(x.shape[b_n:b_n + r_n]), _prod(x.shape[b_n + r_n:]))
    copied, k_last = True, True
    ns = tuple(_merged_stride(shape, g) for g in (ba, ra, ca))
    return OperandView(mem, k_last, ba, ra, ca, shape, None if None in ns else ns, copied)
  perm = ba + (ra + ca if k_last else ca + ra)
  xp = x.permute(tuple(perm))
  B, R, K = (_prod(shape[a] for a in g) for g in (ba, ra, ca))
  mem = xp.reshape(B, R, K) if k_last else xp.reshape(B, K, R)
  assert mem.is_contiguous()
  ns = tuple(_merged_stride(shape, g) for g in (ba, ra, ca))
  return OperandView(mem, k_last, ba, ra, ca, shape, None if None in ns else ns, copied)


def logical_from_brk(t: torch.Tensor, v: OperandView, k_keep: bool = True) -> torch.Tensor:
  """[B, R, K] (or [B, R] when not k_keep) kernel output -> tensor indexed like the operand.

  With k_keep False the contraction axes come back with extent 1 (keepdims).
  """
  dims = [v.shape[a] for a in v.b_axes] + [v.shape[a] for a in v.r_axes]
  dims += [v.shape[a] if k_keep else 1 for a in v.k_axes]
  t = t.reshape(dims)
  axes = v.b_axes + v.r_axes + v.k_axes
  inv = [0] * len(axes)
  for pos, a in enumerate(axes):
    inv[a] = pos
  return t.permute(tuple(inv))


_OUT_TORCH = {L.I8: torch.int8, L.I4: torch.int8, L.E4M3: torch.float8_e4m3fn, L.E5M2: torch.float8_e5m2}


def quantize_view(v: OperandView, *, spec: dict, compute_dtype, scale_dtype, key=None,
                  per_tensor: bool = False, prescale: Optional[torch.Tensor] = None,
                  scale: Optional[torch.Tensor] = None, want_other_axis_absmax: bool = False,
                  absmax_partials: Optional[torch.Tensor] = None):
  """Runs the quantize kernel on a view.

  Returns (q [B, R, K] int8/uint8, scale float32 [B, R] (or [1] per tensor)).
  `prescale` is float32 [B, K] (or [K]): the factor varies along the contraction axes.
  """
  noise = spec['noise']
  kwargs = dict(out_dtype=spec['out_dtype'], quant_bound=spec['quant_bound'],
                clip_bound=spec['clip_bound'], compute_dtype=compute_dtype, scale_dtype=scale_dtype,
                noise=noise, partitionable=utils.threefry_partitionable)
  if noise != L.NOISE_NONE:
    assert key is not None, 'stochastic rounding requested but Context.key is None'
    if v.noise_strides is None:
      raise NotFused('noise counters for this axis layout are not supported')
    nb, nr, nk = v.noise_strides
    kwargs.update(key=key, noise_total=_prod(v.shape),
                  noise_strides=(nb, nr, nk) if v.k_last else (nb, nk, nr))
  if prescale is not None:
    kwargs.update(prescale=prescale,
                  prescale_mode=L.PRESCALE_PER_COL if v.k_last else L.PRESCALE_PER_ROW)
  if per_tensor:
    reduce = L.REDUCE_ALL_BATCH
  else:
    reduce = L.REDUCE_COLS if v.k_last else L.REDUCE_ROWS
  transpose = not v.k_last
  if reduce == L.REDUCE_COLS and per_tensor is False and transpose:
    raise AssertionError('unreachable')
  q, s, typed = ops.quantize(v.mem, reduce=reduce, transpose_out=transpose, scale=scale,
                             want_typed_scale=True, want_other_axis_absmax=want_other_axis_absmax,
                             absmax_partials=absmax_partials, **kwargs)
  shape = (-1,) if per_tensor else (v.B, v.R)
  s = s.reshape(shape)
  # the same scales as elements of the scale dtype, written by the kernel (saves a cast launch)
  s.typed = typed.reshape(shape) if typed is not None else None
  return q, s


def absmax_scale(x: torch.Tensor, shared_axes: Sequence[int], numerics_, scale_dtype):
  """AbsMaxCalibration on its own: the keepdims scale array in scale_dtype (or x.dtype)."""
  shared = [a % x.dim() for a in shared_axes]
  rest = [a for a in range(x.dim()) if a not in shared]
  v = view_operand(x, [], rest, shared)
  spec = dict(out_dtype=L.I8, quant_bound=float(numerics_.get_quant_bound()), clip_bound=1.0,
              noise=L.NOISE_NONE)
  sdt = scale_dtype if scale_dtype is not None else x.dtype
  _, s = quantize_view(v, spec=spec, compute_dtype=x.dtype, scale_dtype=sdt)
  return scale_in_dtype(s, v, sdt)


def scale_in_dtype(s32: torch.Tensor, v: OperandView, sdt) -> torch.Tensor:
  """The keepdims scale array of dtype `sdt` from the [B, R] float32 scales of quantize_view."""
  typed = getattr(s32, 'typed', None)
  if s32.numel() == 1 and (v.B * v.R) != 1:  # per tensor
    src = typed if typed is not None and typed.dtype == sdt else s32
    out = src.reshape([1] * len(v.shape)).to(sdt)
    f32 = s32.reshape([1] * len(v.shape))
  else:
    src = typed if typed is not None and typed.dtype == sdt else s32
    out = logical_from_brk(src, v, k_keep=False).to(sdt)
    f32 = logical_from_brk(s32, v, k_keep=False)
  if sdt != torch.float32:
    out.f32_copy = f32  # same values, for kernels that take float32 scale vectors
  return out

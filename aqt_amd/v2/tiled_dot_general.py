"""dot_general with tiled (subchannel) contraction and remaining axes.

Counterpart of aqt/jax/v2/tiled_dot_general.py.  An axis of extent c*s is viewed
as (c tiles, s elements); tile-count axes of contraction axes become leading batch
axes of the inner dot_general, so a quantizing dot_general calibrates every tile
on its own (tiled_dot_general.py:430-435), and the per-tile outputs -- already
dequantized -- are summed afterwards (:493).  Tile-count axes of remaining axes
are batch axes too; the other operand is broadcast along them (:401-403).

The public names (AxisTiling, TensorTiling, Cfg, TilingState and its methods,
tiled_dot_general, ...) and the shapes they produce follow the reference
(tiled_shape/tile_map goldens: tiled_dot_general_test.py:256-299); the code is
written for torch tensors: tiling is a view, broadcasting an expand.
"""
from __future__ import annotations

import copy
import dataclasses
from typing import Dict, Iterable, List, Optional, Sequence, Tuple, Union

import torch

from aqt_amd.v2 import utils

AxisIdx = int
AxisSize = int
BROADCAST_PREFIX = 'broadcast_'


@dataclasses.dataclass
class AxisTiling:
  """How one axis is split (tiled_dot_general.py:45-75): give tile_count or tile_size."""
  axis: AxisIdx
  tile_count: Optional[AxisSize] = None
  tile_size: Optional[AxisSize] = None

  def __post_init__(self):
    assert not (self.tile_count is None and self.tile_size is None), (
        'At most one of tile_count and tile_size can be None')

  def complete_missing(self, shape):
    if self.axis < 0:
      self.axis += len(shape)
    extent = shape[self.axis]
    assert not (self.tile_count is None and self.tile_size is None), (
        'At most one of tile_count and tile_size can be None')
    if self.tile_count is None:
      self.tile_count = extent // self.tile_size
    if self.tile_size is None:
      self.tile_size = extent // self.tile_count
    assert self.tile_size * self.tile_count == extent, (
        f'Axis {self.axis} cannot be split into {self.tile_count} tiles.')


@dataclasses.dataclass
class TensorTiling:
  contraction_axes: List[AxisTiling]
  remaining_axes: List[AxisTiling]


@dataclasses.dataclass
class Cfg:
  """Tiling of both operands (tiled_dot_general.py:85-147)."""
  lhs: TensorTiling
  rhs: TensorTiling

  @classmethod
  def from_einsum(cls, eqn: str, einsum_tile_sizes: Dict[str, AxisSize]) -> 'Cfg':
    """Tile sizes keyed by einsum letter; a letter must be on exactly two of lhs/rhs/result."""
    args, ret = eqn.split('->')
    args = args.split(',')
    assert len(args) == 2, f'more then 2 arguments are not supported {eqn}'
    lhs_s, rhs_s = args
    assert lhs_s.isalpha(), f'unsupported lhs: {eqn}'
    assert rhs_s.isalpha(), f'unsupported rhs: {eqn}'
    assert ret.isalpha(), f'unsupported ret: {eqn}'
    cfg = cls(lhs=TensorTiling([], []), rhs=TensorTiling([], []))
    for letter, size in einsum_tile_sizes.items():
      assert letter.isalpha() and len(letter) == 1
      where = [lhs_s.find(letter), rhs_s.find(letter), ret.find(letter)]
      msg = f'We support only contraction axes and remaining axes: eqn={eqn} einsum_letter={letter}'
      assert sum(w != -1 for w in where) == 2, msg
      in_l, in_r, in_o = where
      if in_l != -1 and in_r != -1:
        cfg.lhs.contraction_axes.append(AxisTiling(axis=in_l, tile_size=size))
        cfg.rhs.contraction_axes.append(AxisTiling(axis=in_r, tile_size=size))
      else:
        assert in_o != -1, f'Should not happen. {msg}'
        if in_l != -1:
          cfg.lhs.remaining_axes.append(AxisTiling(axis=in_l, tile_size=size))
        if in_r != -1:
          cfg.rhs.remaining_axes.append(AxisTiling(axis=in_r, tile_size=size))
    return cfg

  def complete_missing(self, lhs_shape, rhs_shape) -> 'Cfg':
    out = copy.deepcopy(self)
    for side, shape in ((out.lhs, lhs_shape), (out.rhs, rhs_shape)):
      for at in (*side.contraction_axes, *side.remaining_axes):
        at.complete_missing(shape)
    return out


def get_ra(rank, ca, ba) -> List[AxisIdx]:
  return [a for a in range(rank) if a not in list(ca) + list(ba)]


def interleave(tile_count, tile_size, tile_map, remaining_axes, product=False):
  """Pairs every tile-size entry with its tile-count entry when the axis is tiled.

  `tile_count` lists entries of tiled axes only, `tile_size` one entry per remaining
  axis.  With product the pair collapses to count*size (the untiled extent).
  """
  counts = list(tile_count)
  out = []
  for ax, ts in zip(remaining_axes, tile_size):
    if len(tile_map[ax]) > 1:
      tc = counts.pop(0)
      out += [tc * ts] if product else [tc, ts]
    else:
      out.append(ts)
  assert not counts, 'Remaining axes tile count and tile size are not fully interleaved.'
  return out


def maybe_add_one(i, min_i):
  """Index i after an axis was inserted at min_i (tiled_dot_general.py:177-178)."""
  return i + int(i >= min_i)


@dataclasses.dataclass
class TilingState:
  """Axis bookkeeping of one operand while it is tiled (tiled_dot_general.py:182-294).

  tile_map[a] lists where untiled axis a went: [size axis] or [count axis, size axis];
  keys 'broadcast_i' stand for leading axes added by broadcast_to_other.
  """
  untiled_shape: Tuple[AxisSize, ...]
  tile_map: Dict[Union[AxisIdx, str], List[AxisIdx]] = dataclasses.field(default_factory=dict)
  tiled_shape: List[AxisSize] = dataclasses.field(default_factory=list)

  def __post_init__(self):
    self.untiled_shape = tuple(self.untiled_shape)
    self.tile_map = {i: [i] for i in range(len(self.untiled_shape))}
    self.tiled_shape = list(self.untiled_shape)

  def get_broadcasted_tile_map_indexes(self):
    return [k for k in self.tile_map if isinstance(k, str) and k.startswith(BROADCAST_PREFIX)]

  def tile_one_axis(self, at: AxisTiling):
    assert not self.get_broadcasted_tile_map_indexes(), (
        "Can't tile as all tiling must be done before broadcast operations.")
    where = self.tile_map[at.axis]
    assert len(where) == 1, "can't tile the same axis twice."
    pos = where[0]
    assert self.tiled_shape[pos] == at.tile_size * at.tile_count, (
        f'{self.tiled_shape[pos]=}, {at.tile_size=}, {at.tile_count=}')
    self.tiled_shape[pos:pos + 1] = [at.tile_count, at.tile_size]
    for k, v in self.tile_map.items():
      self.tile_map[k] = [p + (p >= pos) for p in v]
    self.tile_map[at.axis] = [pos, pos + 1]

  def tile_axes(self, ats: Iterable[AxisTiling]):
    for at in ats:
      self.tile_one_axis(at)

  def apply(self, x: torch.Tensor) -> torch.Tensor:
    """x in the tiled shape (a view; broadcast axes are expanded, not materialised)."""
    nb = len(self.get_broadcasted_tile_map_indexes())
    return x.reshape(self.tiled_shape[nb:]).expand(self.tiled_shape)

  def unapply(self, tiled_x: torch.Tensor) -> torch.Tensor:
    nb = len(self.get_broadcasted_tile_map_indexes())
    return tiled_x[(0,) * nb].reshape(self.untiled_shape)

  def broadcast_to_other(self, bcast_shape):
    """New leading axes of the given extents; returns their tile_map keys."""
    n = len(bcast_shape)
    for k, v in self.tile_map.items():
      self.tile_map[k] = [p + n for p in v]
    keys = []
    for i in range(n):
      key = f'{BROADCAST_PREFIX}{i}'
      assert key not in self.tile_map
      self.tile_map[key] = [i]
      keys.append(key)
    self.tiled_shape = list(bcast_shape) + self.tiled_shape
    return keys

  def axes_shape(self, axes):
    return tuple(self.tiled_shape[a] for a in axes)

  def to_tiled_axes_transposed(self, axes):
    """(tile-count axes, tile-size axes) in the tiled tensor for untiled `axes`."""
    counts, sizes = [], []
    for a in axes:
      if isinstance(a, int) and a < 0:
        a += len(self.untiled_shape)
      where = self.tile_map[a]
      if len(where) == 2:
        counts.append(where[0])
      sizes.append(where[-1])
    return counts, sizes

def generate_tiling_state(tensor, tiled_axes: Iterable[AxisTiling]) -> TilingState:
  """tiled_dot_general.py:320-331."""
  tiled_axes = list(tiled_axes)
  for at in tiled_axes:
    at.complete_missing(tuple(tensor.shape))
  st = TilingState(untiled_shape=tuple(tensor.shape))
  st.tile_axes(tiled_axes)
  return st

def generate_tiling_states_for_dot_general(cfg: Cfg, lhs, rhs, dimension_numbers):
  """Tiling states of both operands, broadcast axes included (tiled_dot_general.py:334-404)."""
  cfg = copy.deepcopy(cfg).complete_missing(tuple(lhs.shape), tuple(rhs.shape))
  (lca, rca), (lba, rba) = dimension_numbers
  lra = get_ra(lhs.dim(), list(lca), list(lba))
  rra = get_ra(rhs.dim(), list(rca), list(rba))
  assert len(cfg.lhs.contraction_axes) == len(cfg.rhs.contraction_axes), (
      f'tiling cfg has different numbers of contraction axes: {cfg}')
  for a, b in zip(cfg.lhs.contraction_axes, cfg.rhs.contraction_axes):
    assert a.tile_count == b.tile_count, (
        'Contraction axis tile counts should be the same, but found lhs axis'
        f' {a.axis} has a tile count of {a.tile_count}, and rhs axis {b.axis} has a tile count of'
        f' {b.tile_count}')
  xlhs = TilingState(untiled_shape=tuple(lhs.shape))
  xlhs.tile_axes(cfg.lhs.contraction_axes + cfg.lhs.remaining_axes)
  xrhs = TilingState(untiled_shape=tuple(rhs.shape))
  xrhs.tile_axes(cfg.rhs.contraction_axes + cfg.rhs.remaining_axes)
  l_ra_tiles, _ = xlhs.to_tiled_axes_transposed(lra)
  xrhs.broadcast_to_other(xlhs.axes_shape(l_ra_tiles))
  r_ra_tiles, _ = xrhs.to_tiled_axes_transposed(rra)
  xlhs.broadcast_to_other(xrhs.axes_shape(r_ra_tiles))
  return xlhs, xrhs

def _sum_leading(x):
  """Sum over axis 0 in float32, tile by tile, rounded once to x.dtype."""
  if x.is_cuda and x.dtype in (torch.bfloat16, torch.float32):
    from aqt_amd import ops
    return ops.sum_tiles(x.contiguous())
  acc = torch.zeros(x.shape[1:], dtype=torch.float32 if x.dtype != torch.float64 else torch.float64,
                    device=x.device)
  for t in range(x.shape[0]):
    acc = acc + x[t]
  return acc.to(x.dtype)

def _default_dot_general(lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None):
  from aqt_amd.v2 import aqt_dot_general
  return aqt_dot_general.lax_dot_general(lhs, rhs, dimension_numbers, precision, preferred_element_type)

def tiled_dot_general_with_tiling_states(lhs, xlhs: TilingState, rhs, xrhs: TilingState,
                                         untiled_dimension_numbers, precision=None,
                                         preferred_element_type=None, dot_general=_default_dot_general):
  """tiled_dot_general.py:407-543."""
  tl, tr = xlhs.apply(lhs), xrhs.apply(rhs)
  (lca, rca), (lba, rba) = untiled_dimension_numbers
  lca, rca, lba, rba = list(lca), list(rca), list(lba), list(rba)
  lra, rra = get_ra(lhs.dim(), lca, lba), get_ra(rhs.dim(), rca, rba)
  l_ca_t, l_ca = xlhs.to_tiled_axes_transposed(lca)
  l_ra_t, l_ra = xlhs.to_tiled_axes_transposed(lra)
  r_ca_t, r_ca = xrhs.to_tiled_axes_transposed(rca)
  r_ra_t, r_ra = xrhs.to_tiled_axes_transposed(rra)
  none_l, l_other = xlhs.to_tiled_axes_transposed(xlhs.get_broadcasted_tile_map_indexes())
  none_r, r_other = xrhs.to_tiled_axes_transposed(xrhs.get_broadcasted_tile_map_indexes())
  nb_l, l_ba = xlhs.to_tiled_axes_transposed(lba)
  nb_r, r_ba = xrhs.to_tiled_axes_transposed(rba)
  assert not (none_l or none_r or nb_l or nb_r), 'batch and broadcast axes cannot be tiled'

  tiled_dn = ((l_ca, r_ca), (l_ca_t + l_ba + l_ra_t + l_other, r_ca_t + r_ba + r_other + r_ra_t))
  for ax in tiled_dn[0][0] + tiled_dn[1][0]:
    assert 0 <= ax < tl.dim()
  for ax in tiled_dn[0][1] + tiled_dn[1][1]:
    assert 0 <= ax < tr.dim()

  # A quantizing dot_general may be able to contract, dequantize and sum the tiles in one kernel.
  fused = getattr(dot_general, 'fused_tile_sum', None)
  out = None
  if fused is not None and l_ca_t and precision is None:
    summed = fused(tl, tr, tiled_dn, len(l_ca_t))
    if summed is not None:
      out = summed.reshape((1,) * len(l_ca_t) + tuple(summed.shape))
  if out is None:
    out = dot_general(tl, tr, tiled_dn, precision, preferred_element_type)

  ca_t_sh = xlhs.axes_shape(l_ca_t)
  assert ca_t_sh == xrhs.axes_shape(r_ca_t)
  ba_sh = xlhs.axes_shape(l_ba)
  assert ba_sh == xrhs.axes_shape(r_ba)
  l_ra_t_sh = xlhs.axes_shape(l_ra_t)
  assert l_ra_t_sh == xrhs.axes_shape(r_other)
  r_ra_t_sh = xlhs.axes_shape(l_other)
  assert r_ra_t_sh == xrhs.axes_shape(r_ra_t)
  l_ra_sh, r_ra_sh = xlhs.axes_shape(l_ra), xrhs.axes_shape(r_ra)
  if fused is not None and tuple(out.shape[:len(ca_t_sh)]) == (1,) * len(ca_t_sh) and ca_t_sh != (1,) * len(ca_t_sh):
    ca_t_sh = (1,) * len(ca_t_sh)   # already summed by the fused kernel
  assert tuple(out.shape) == ca_t_sh + ba_sh + l_ra_t_sh + r_ra_t_sh + l_ra_sh + r_ra_sh, (
      tuple(out.shape), ca_t_sh, ba_sh, l_ra_t_sh, r_ra_t_sh, l_ra_sh, r_ra_sh)

  # Sum of the (dequantized) per-tile outputs over the contraction tile counts.  jnp.sum
  # accumulates 16-bit floats in float32 and rounds once; so does this.
  if ca_t_sh:
    rest = tuple(out.shape[len(ca_t_sh):])
    only_one = all(c == 1 for c in ca_t_sh)   # a single tile, or tiles already summed by the fused kernel
    out = out.reshape(rest) if only_one else _sum_leading(out.reshape((-1,) + rest))

  # (ba, lhs ra counts, rhs ra counts, lhs ra sizes, rhs ra sizes) -> counts next to their sizes
  n0 = len(ba_sh)
  n1, n2 = n0 + len(l_ra_t_sh), n0 + len(l_ra_t_sh) + len(r_ra_t_sh)
  n3 = n2 + len(l_ra_sh)
  n4 = n3 + len(r_ra_sh)
  perm = (list(range(n0))
          + interleave(range(n0, n1), range(n2, n3), xlhs.tile_map, lra)
          + interleave(range(n1, n2), range(n3, n4), xrhs.tile_map, rra))
  out = out.permute(tuple(perm)) if perm else out
  l_flat = interleave(l_ra_t_sh, l_ra_sh, xlhs.tile_map, lra, product=True)
  r_flat = interleave(r_ra_t_sh, r_ra_sh, xrhs.tile_map, rra, product=True)
  return out.reshape(list(ba_sh) + l_flat + r_flat)

def tiled_dot_general(cfg: Cfg, lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None,
                      dot_general=_default_dot_general):
  """dot_general over tiles of the operands (tiled_dot_general.py:546-568)."""
  xlhs, xrhs = generate_tiling_states_for_dot_general(cfg, lhs, rhs, dimension_numbers)
  return tiled_dot_general_with_tiling_states(lhs, xlhs, rhs, xrhs, dimension_numbers, precision,
                                              preferred_element_type, dot_general)

def print_dimension_numbers(dimension_numbers, lhs, rhs, label) -> None:
  """Logs the dimension numbers before and / or after tiling at debug level
  (tiled_dot_general.py:297-320)."""
  import logging
  (lhs_ca, rhs_ca), (lhs_ba, rhs_ba) = dimension_numbers
  lhs_ra = get_ra(lhs.dim(), lhs_ca, lhs_ba)
  rhs_ra = get_ra(rhs.dim(), rhs_ca, rhs_ba)
  log = logging.getLogger(__name__)
  log.debug(label)
  log.debug(' lhs.shape=%s', tuple(lhs.shape))
  log.debug(' rhs.shape=%s', tuple(rhs.shape))
  log.debug(' lhs_ca=%s rhs_ca=%s', lhs_ca, rhs_ca)
  log.debug(' lhs_ba=%s rhs_ba=%s', lhs_ba, rhs_ba)
  log.debug(' lhs_ra=%s rhs_ra=%s', lhs_ra, rhs_ra)

"""Host logic of tiled_dot_general: goldens and properties of the reference's own tests
(aqt/jax/v2/tiled_dot_general_test.py), with a float contraction as the inner dot_general."""
import itertools

import numpy as np
import pytest
import torch

from aqt_amd.v2 import aqt_dot_general
from aqt_amd.v2 import tiled_dot_general as T

AxisTiling, TensorTiling, Cfg = T.AxisTiling, T.TensorTiling, T.Cfg


def test_tiling_state_for_single_tensor():
  """tiled_dot_general_test.py:256-278."""
  shape = (31, 22, 27, 8, 27)
  axes = [AxisTiling(axis=1, tile_count=None, tile_size=11), AxisTiling(axis=2, tile_count=None, tile_size=9)]
  st = T.generate_tiling_state(torch.ones(shape), axes)
  assert st.untiled_shape == shape
  assert st.tiled_shape == [31, 2, 11, 3, 9, 8, 27]
  assert st.tile_map == {0: [0], 1: [1, 2], 2: [3, 4], 3: [5], 4: [6]}
  assert st.to_tiled_axes_transposed([a.axis for a in axes]) == ([1, 3], [2, 4])


def test_negative_axis_index():
  """tiled_dot_general_test.py:280-304."""
  shape = (31, 22, 27, 8, 27)
  axes = [AxisTiling(axis=-1, tile_count=None, tile_size=9), AxisTiling(axis=-2, tile_count=2, tile_size=None)]
  st = T.generate_tiling_state(torch.ones(shape), axes)
  assert st.tiled_shape == [31, 22, 27, 2, 4, 3, 9]
  assert st.tile_map == {0: [0], 1: [1], 2: [2], 3: [3, 4], 4: [5, 6]}
  assert st.to_tiled_axes_transposed([-1]) == ([5], [6])
  assert st.to_tiled_axes_transposed([-2]) == ([3], [4])
  assert st.to_tiled_axes_transposed([-3]) == ([], [2])


def test_apply_unapply_round_trip():
  x = torch.arange(4 * 6 * 10, dtype=torch.float32).reshape(4, 6, 10)
  st = T.generate_tiling_state(x, [AxisTiling(axis=1, tile_size=3), AxisTiling(axis=2, tile_count=5)])
  st.broadcast_to_other((7, 2))
  tx = st.apply(x)
  assert list(tx.shape) == [7, 2, 4, 2, 3, 5, 2]
  assert torch.equal(st.unapply(tx), x)
  with pytest.raises(AssertionError, match='before broadcast'):
    st.tile_one_axis(AxisTiling(axis=0, tile_size=2))


def test_single():
  """tiled_dot_general_test.py:226-254: two tiled contraction axes, a tiled rhs remaining axis."""
  lhs, rhs = torch.ones((31, 22, 9, 8, 27)), torch.ones((8, 9, 22, 27, 7, 12))
  cfg = Cfg(
      lhs=TensorTiling(contraction_axes=[AxisTiling(axis=2, tile_size=9), AxisTiling(axis=1, tile_size=11)],
                       remaining_axes=[]),
      rhs=TensorTiling(contraction_axes=[AxisTiling(axis=1, tile_size=9), AxisTiling(axis=2, tile_size=11)],
                       remaining_axes=[AxisTiling(axis=5, tile_size=4)]))
  dims = (((2, 1), (1, 2)), ((4, 3), (3, 0)))
  out = T.tiled_dot_general(cfg, lhs, rhs, dims)
  want = aqt_dot_general.lax_dot_general(lhs, rhs, dims, None, None)
  assert out.shape == want.shape
  assert torch.equal(out, want)


def _divisors(n):
  return [d for d in range(1, n + 1) if n % d == 0]


def _axis_tilings(axes, shape):
  """Every subset of `axes`, every second divisor as tile size (tiled_dot_general_test.py:57-75)."""
  out = []
  for r in range(len(axes) + 1):
    for subset in itertools.combinations(axes, r):
      choices = [[AxisTiling(a, None, ts) for ts in _divisors(shape[a])[::2]] for a in subset]
      out.extend(itertools.product(*choices))
  return out


@pytest.mark.parametrize('seed', range(6))
def test_tiled_equals_untiled_random_layouts(seed):
  """tiled_dot_general_test.py:191-224 with numpy's generator: random ranks, axis orders and
  tilings; integer-valued operands make every summation order exact."""
  rng = np.random.default_rng(seed)
  n_ca, n_ba, n_lra, n_rra = rng.integers(1, 3), rng.integers(0, 3), rng.integers(1, 3), rng.integers(1, 3)
  ca_sh = rng.integers(1, 9, n_ca).tolist()
  ba_sh = rng.integers(1, 4, n_ba).tolist()

  def place(ra_sh):
    n = n_ca + n_ba + len(ra_sh)
    axes = rng.permutation(n).tolist()
    ca, ba, ra = axes[:n_ca], axes[n_ca:n_ca + n_ba], axes[n_ca + n_ba:]
    shape = np.array(ca_sh + ba_sh + ra_sh)[np.argsort(axes)].tolist()
    return ca, ba, ra, shape

  lca, lba, lra, lsh = place(rng.integers(1, 7, n_lra).tolist())
  rca, rba, rra, rsh = place(rng.integers(1, 7, n_rra).tolist())
  lhs = torch.from_numpy(rng.integers(-3, 4, lsh).astype(np.float32))
  rhs = torch.from_numpy(rng.integers(-3, 4, rsh).astype(np.float32))
  dims = ((tuple(lca), tuple(rca)), (tuple(lba), tuple(rba)))
  want = aqt_dot_general.lax_dot_general(lhs, rhs, dims, None, None)
  l_ca_t, r_ca_t = _axis_tilings(lca, lsh), _axis_tilings(rca, rsh)
  assert len(l_ca_t) == len(r_ca_t)
  count = 0
  for ct_l, ct_r in zip(l_ca_t, r_ca_t):
    for rt_l in _axis_tilings(lra, lsh)[:4]:
      for rt_r in _axis_tilings(rra, rsh)[:4]:
        cfg = Cfg(lhs=TensorTiling(list(ct_l), list(rt_l)), rhs=TensorTiling(list(ct_r), list(rt_r)))
        got = T.tiled_dot_general(cfg, lhs, rhs, dims)
        assert got.shape == want.shape, cfg
        assert torch.equal(got, want), cfg
        count += 1
  assert count > 0


def test_from_einsum():
  cfg = Cfg.from_einsum('bsd,dhk->bshk', {'d': 128, 'h': 4})
  assert [(a.axis, a.tile_size) for a in cfg.lhs.contraction_axes] == [(2, 128)]
  assert [(a.axis, a.tile_size) for a in cfg.rhs.contraction_axes] == [(0, 128)]
  assert cfg.lhs.remaining_axes == [] and [(a.axis, a.tile_size) for a in cfg.rhs.remaining_axes] == [(1, 4)]
  with pytest.raises(AssertionError, match='only contraction axes and remaining axes'):
    Cfg.from_einsum('bsd,bdk->bsk', {'b': 2})


def test_bad_tilings_are_rejected():
  with pytest.raises(AssertionError, match='cannot be split'):
    AxisTiling(axis=0, tile_size=5).complete_missing((12,))
  with pytest.raises(AssertionError):
    AxisTiling(axis=0)
  lhs, rhs = torch.ones(4, 12), torch.ones(12, 6)
  cfg = Cfg(lhs=TensorTiling([AxisTiling(axis=1, tile_size=4)], []),
            rhs=TensorTiling([AxisTiling(axis=0, tile_size=3)], []))
  with pytest.raises(AssertionError, match='tile counts should be the same'):
    T.tiled_dot_general(cfg, lhs, rhs, (((1,), (0,)), ((), ())))

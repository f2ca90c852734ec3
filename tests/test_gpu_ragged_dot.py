"""Quantized ragged_dot: oracle pins (CPU) and GPU parity, after aqt_ragged_dot_test.py."""
import numpy as np
import pytest
import torch

from oracle import aqt_ref as R
from oracle import numerics as nm
from tests import gpu_util as U


def _args(m, k, n, num_groups, dt, balanced, seed=1234):
  """aqt_ragged_dot_test.py:88-112: uniform [0, 1) operands representable in bf16; random
  group ends drawn with replacement so that empty groups occur."""
  rng = np.random.default_rng(seed)
  lhs = nm.cast(nm.cast(rng.uniform(0, 1, (m, k)).astype(np.float32), 'bf16'), dt)
  rhs = nm.cast(nm.cast(rng.uniform(0, 1, (num_groups, k, n)).astype(np.float32), 'bf16'), dt)
  if balanced:
    sizes = [m // num_groups] * num_groups
  else:
    ends = np.concatenate([np.sort(rng.choice(m, num_groups - 1)), [m]])
    sizes = list(np.diff(np.concatenate([[0], ends])))
  assert sum(sizes) == m
  return lhs, rhs, [int(s) for s in sizes]


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('balanced', [True, False])
def test_oracle_ragged_dot_close_to_float_and_to_batched_dot_general(dt, balanced):
  """aqt_ragged_dot_test.py:114-153: within rtol 1e-2 (bf16) / 5e-3 (f32) of the float ragged
  dot, and, with equal groups, of the quantized batched dot_general on the reshaped lhs."""
  m, k, n, g = 32, 128, 16, 8
  lhs, rhs, sizes = _args(m, k, n, g, dt, balanced)
  rtol = 1e-2 if dt == 'bf16' else 5e-3
  out, lqt, rqt = R.ragged_dot_fwd(lhs, rhs, dt, sizes, R.config_v4().fwd)
  assert lqt.scale[0].shape == (m, 1) and rqt.scale[0].shape == (1, 1, n)
  want = nm.cast(R.lax_ragged_dot(lhs, rhs, sizes, np.float32), dt)
  np.testing.assert_allclose(out, want, rtol=rtol, atol=1e-5)
  if balanced:
    f = R.dg_fwd(lhs.reshape(g, m // g, k), rhs, dt, (((2,), (1,)), ((0,), (0,))), R.config_v4())
    np.testing.assert_allclose(out, f.out.reshape(m, n), rtol=rtol, atol=1e-5)


def test_oracle_ragged_dot_integer_exact():
  """Small integers quantize without loss when the abs-max is 127: the quantized ragged dot
  is then the exact integer result."""
  rng = np.random.default_rng(0)
  lhs = rng.integers(-127, 128, (12, 16)).astype(np.float32)
  lhs[:, 0] = 127.0
  rhs = rng.integers(-127, 128, (3, 16, 5)).astype(np.float32)
  rhs[0, 0, :] = 127.0
  raw = R.config_v4().fwd
  raw.lhs.preserve_max_val = raw.rhs.preserve_max_val = True  # scale = absmax / 127 = 1
  out, _, _ = R.ragged_dot_fwd(lhs, rhs, 'f32', [5, 0, 7], raw)
  want = np.concatenate([lhs[:5] @ rhs[0], lhs[5:] @ rhs[2]])
  np.testing.assert_array_equal(out, want)


@pytest.mark.gpu
@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('balanced', [True, False])
@pytest.mark.parametrize('shape', [(32, 128, 16, 8), (300, 96, 200, 5), (3000, 256, 520, 6), (66, 72, 40, 3)])
def test_ragged_dot_matches_oracle(gpu, dt, balanced, shape):
  from aqt_amd.v2 import aqt_ragged_dot
  m, k, n, g = shape
  lhs, rhs, sizes = _args(m, k, n, g, dt, balanced)
  want, _, _ = R.ragged_dot_fwd(lhs, rhs, dt, sizes, R.config_v4().fwd)
  L, Rr = U.to_dev(lhs, dt, gpu), U.to_dev(rhs, dt, gpu)
  out = aqt_ragged_dot.ragged_dot(L, Rr, torch.tensor(sizes, dtype=torch.int32, device=gpu))
  assert out.dtype == U.TORCH_DT[dt]
  np.testing.assert_array_equal(out.float().cpu().numpy(), want)
  # group sizes given on the host, rows past the last group stay zero
  short = sizes[:-1] + [max(sizes[-1] - 3, 0)]
  out2 = aqt_ragged_dot.ragged_dot(L, Rr, short)
  covered = sum(short)
  np.testing.assert_array_equal(out2[:covered].float().cpu().numpy(), want[:covered])
  assert (out2[covered:] == 0).all()


@pytest.mark.gpu
def test_ragged_dot_unquantized_and_precision(gpu):
  from aqt_amd.v2 import aqt_ragged_dot
  from aqt_amd.v2 import config
  lhs, rhs, sizes = _args(32, 128, 16, 8, 'f32', False)
  L, Rr = U.to_dev(lhs, 'f32', gpu), U.to_dev(rhs, 'f32', gpu)
  out = aqt_ragged_dot.ragged_dot(L, Rr, sizes, cfg=config.default_unquantized_config())
  np.testing.assert_allclose(out.cpu().numpy(), R.lax_ragged_dot(lhs, rhs, sizes, np.float32), rtol=1e-5)
  with pytest.raises(AssertionError):  # aqt_ragged_dot_test.py:155-166
    aqt_ragged_dot.ragged_dot(L, Rr, sizes, precision='highest')


@pytest.mark.gpu
def test_ragged_gemm_one_launch_against_integer_reference(gpu):
  """The grouped launch itself: groups that span several 256-row tiles, start in the middle of
  a tile, are empty, or leave the last rows uncovered; raw int32 accumulators."""
  from aqt_amd import ops
  rng = np.random.default_rng(3)
  m, k, n = 2000, 320, 300
  sizes = [700, 0, 257, 1, 511, 300]  # sums to 1769 < m
  a = rng.integers(-127, 128, (m, k)).astype(np.int8)
  b = rng.integers(-127, 128, (len(sizes), n, k)).astype(np.int8)
  offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
  out = ops.gemm(torch.from_numpy(a).to(gpu)[None], torch.from_numpy(b).to(gpu), row_scale=None, col_scale=None,
                 out_dtype=torch.int32, group_offsets=torch.from_numpy(offs).to(gpu))[0].cpu().numpy()
  want = np.zeros((m, n), np.int64)
  for g, (lo, hi) in enumerate(zip(offs[:-1], offs[1:])):
    want[lo:hi] = a[lo:hi].astype(np.int64) @ b[g].astype(np.int64).T
  np.testing.assert_array_equal(out, want)

"""Pins for the oracle's emulated small floats (oracle/fp_ref.py), after fp_numerics_test.py.

None of these retypes the rounding formula: they check it against the enumerated values of
each format, against exact expectations under equi-spaced noise, and against the reference's
second, independent formulation of the same rounding.
"""
import numpy as np
import pytest

from oracle import fp_ref as F
from oracle import numerics as nm
from oracle import prng

# fp_numerics_test.py:296-339 (radix 2, minexp 0)
ROUND_CFGS = [(3, 0), (2, 1), (1, 2), (0, 3), (5, 0), (4, 1), (3, 2), (2, 3), (1, 4), (0, 5), (4, 0), (3, 1), (2, 2),
              (1, 3), (0, 4)]
ROUND_CASES = [(e, m, s) for (e, m) in ROUND_CFGS for s in (False, True)] + [(2, 0, False)]


@pytest.mark.parametrize('nexp,minexp,nmant,sub,expected', [
    (3, 0, 0, False, [1, 2, 4, 8, 16, 32, 64, 128]),
    (3, 0, 0, True, [0, 1, 2, 4, 8, 16, 32, 64]),
    (3, -2, 0, False, [0.25, 0.5, 1, 2, 4, 8, 16, 32]),
    (3, -2, 0, True, [0, 0.25, 0.5, 1, 2, 4, 8, 16]),
    (2, 0, 0, False, [1, 2, 4, 8]),
    (2, 0, 1, False, [1, 1.5, 2, 3, 4, 6, 8, 12]),
    (2, 0, 1, True, [0, 0.5, 1, 1.5, 2, 3, 4, 6]),
    (1, 0, 2, True, [0, 0.25, 0.5, 0.75, 1, 1.25, 1.5, 1.75]),
    (0, 0, 3, True, [0, 0.125, 0.25, 0.375, 0.5, 0.625, 0.75, 0.875]),
])
def test_fp_values_tables(nexp, minexp, nmant, sub, expected):
  """fp_numerics_test.py:169-293: the value tables the reference's test holds."""
  cfg = F.FpNumericsConfig(nexp=nexp, minexp=minexp, nmant=nmant, has_subnormals=sub)
  want = np.array(list(expected) + [-v for v in expected], np.float32)
  np.testing.assert_array_equal(F.fp_values(cfg), want)


def _buckets(cfg):
  centers = np.sort(F.fp_values(cfg).astype(np.float64))
  centers = np.unique(centers)  # +0 and -0 are one bucket
  assert centers[-1] == F.fp_largest_representable(cfg)
  bounds = (centers[1:] + centers[:-1]) / 2
  half = centers[-1] - bounds[-1]
  edge = centers[-1] + half
  bounds = np.concatenate([[-edge], bounds, [edge]])
  return centers, bounds, edge


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('nexp,nmant,sub', ROUND_CASES)
def test_round_to_nearest_and_overflow(nexp, nmant, sub, dt):
  """fp_numerics_test.py:340-440: every interior point of a bucket rounds to its centre, and
  everything past the last bucket clamps to the largest value."""
  cfg = F.FpNumericsConfig(nexp=nexp, minexp=0, nmant=nmant, has_subnormals=sub)
  centers, bounds, edge = _buckets(cfg)
  lower, upper = bounds[:-1], bounds[1:]
  data64 = np.linspace(lower, upper, 129, endpoint=True, axis=0)
  data = nm.cast(data64.astype(np.float32), dt)
  interior = (data != lower[None].astype(np.float32)) & (data != upper[None].astype(np.float32))
  # casting to the container may move a point across a boundary only onto it; keep strict interiors
  interior &= (data > lower[None]) & (data < upper[None])
  q = F.radix2_round(data, dt, cfg)
  want = np.broadcast_to(centers[None].astype(np.float32), q.shape)
  if not sub:
    # without subnormals there is no zero: the bucket "centres" are the values themselves
    assert 0.0 not in centers
  np.testing.assert_array_equal(np.where(interior, q, 0), np.where(interior, want, 0))
  for sign in (-1.0, 1.0):
    far = nm.cast(np.linspace(sign * edge, sign * 10 * edge, 129).astype(np.float32), dt)
    far = far[np.abs(far) > edge] if dt == 'bf16' else far[1:]
    np.testing.assert_array_equal(F.radix2_round(far, dt, cfg), np.full_like(far, sign * centers[-1]))


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('nexp,nmant,sub', [(3, 0, False), (3, 0, True), (2, 1, False), (2, 1, True), (1, 2, True),
                                            (0, 3, True), (0, 3, False), (4, 1, True), (2, 3, True), (1, 4, False)])
def test_equispaced_noise_gives_exact_mean(nexp, nmant, sub, dt):
  """fp_numerics_test.py:442-460: with the 2^16 noise values each used once, the mean of the
  stochastically rounded values is the input exactly (accumulated here in float64)."""
  cfg = F.FpNumericsConfig(nexp=nexp, minexp=0, nmant=nmant, has_subnormals=sub)
  centers, _, _ = _buckets(cfg)
  x = nm.cast(np.linspace(centers[0], centers[-1], 33, endpoint=True).astype(np.float32), dt)
  bx = np.broadcast_to(x[:, None], (33, 2**16))
  q = F.radix2_round(bx, dt, cfg, stochastic_rounding=True, test_noise_axis=1)
  np.testing.assert_array_equal(q.astype(np.float64).mean(axis=1), x.astype(np.float64))
  # and each input hits at most the two neighbouring values
  for row, xv in zip(q, x):
    vals = np.unique(row)
    assert len(vals) <= 2 and vals.min() <= xv <= vals.max()
    assert all(v in centers for v in vals)


@pytest.mark.parametrize('name', sorted(F.CONFIGS))
@pytest.mark.parametrize('sr', [False, True])
def test_two_formulations_agree_on_every_bf16_pattern(name, sr):
  """fp_numerics_test.py:517-604: radix2_round == fp_round_new on all 2^16 bf16 inputs."""
  cfg = F.CONFIGS[name]
  x = (np.arange(2**16, dtype=np.uint32) << np.uint32(16)).view(np.float32)
  ok = ~np.isnan(x)
  for key_num in ([0, 42] if sr else [None]):
    key = prng.prng_key(key_num) if sr else None
    a = F.radix2_round(x, 'bf16', cfg, key, sr)
    b = F.fp_round_new(x, 'bf16', cfg, key, sr)
    np.testing.assert_array_equal(a[ok], b[ok])


@pytest.mark.parametrize('name', ['e2m1', 'e2m1_ocp', 'e3m0_ocp', 'e0m3_ocp', 'e1m0', 'e4m1_ocp'])
@pytest.mark.parametrize('sr', [False, True])
def test_two_formulations_agree_on_f32_slices(name, sr):
  """fp_numerics_test.py:525-604: the same on slices of the float32 bit patterns."""
  cfg = F.CONFIGS[name]
  vlen = 2**18
  for i in (0, 1, 100, 8191, 8192, 8193, 15900):
    x = np.arange(vlen * i, vlen * (i + 1), dtype=np.uint32).view(np.float32)
    ok = ~np.isnan(x)
    key = prng.prng_key(12) if sr else None
    a = F.radix2_round(x, 'f32', cfg, key, sr)
    b = F.fp_round_new(x, 'f32', cfg, key, sr)
    np.testing.assert_array_equal(a[ok], b[ok])


def test_unbiased_with_real_noise():
  """fp_numerics_test.py:462-515: with jax.random bits the empirical probability of rounding
  down is within two standard errors of the distance to the upper neighbour."""
  n = 100000
  for name in ('e2m1', 'e2m1_ocp'):
    cfg = F.CONFIGS[name]
    centers, _, _ = _buckets(cfg)
    x = nm.cast(np.linspace(centers[0], centers[-1], 17, endpoint=True).astype(np.float32), 'bf16')
    bx = np.broadcast_to(x[:, None], (17, n))
    q = F.radix2_round(bx, 'bf16', cfg, prng.prng_key(42), True)
    lo, hi = q.min(axis=1), q.max(axis=1)
    assert ((q == lo[:, None]) | (q == hi[:, None])).all()
    p_lo = (q == lo[:, None]).mean(axis=1)
    size = hi - lo
    want = np.where(size == 0, 1.0, (hi - x) / np.where(size == 0, 1, size))
    assert (np.abs(p_lo - want) * np.sqrt(n) < 2.0).all()


def test_e1m2_vs_e0m3():
  """fp_numerics_test.py:606-619: e1m2 (with subnormals) is e0m3 scaled by two."""
  rng = np.random.default_rng(42)
  x = nm.cast(rng.standard_normal((64, 64)).astype(np.float32), 'bf16')
  x = nm.cast(x / np.abs(x).max(), 'bf16')
  b1 = F.fp_largest_representable(F.CONFIGS['e1m2_ocp'])
  b0 = F.fp_largest_representable(F.CONFIGS['e0m3_ocp'])
  assert (b1, b0) == (1.75, 0.875)
  in1, in0 = nm.cast(x * np.float32(b1), 'bf16'), nm.cast(x * np.float32(b0), 'bf16')
  np.testing.assert_array_equal(in1, in0 * 2)
  y1 = F.fp_vjp_fwd(in1, 'bf16', F.CONFIGS['e1m2_ocp'])
  y0 = F.fp_vjp_fwd(in0, 'bf16', F.CONFIGS['e0m3_ocp'])
  # The identity holds away from ties only (the reference's random sample holds none): in
  # [1, 2) e1m2 adds half an ulp to the bit pattern (ties away from zero), e0m3 rounds the
  # scaled value half to even.
  tie = (np.abs(in1) >= 1) & (np.abs(in0 * 8) % 1 == 0.5)
  np.testing.assert_array_equal(y1[~tie], y0[~tie] * 2)
  np.testing.assert_array_equal(F.fp_vjp_fwd(np.float32([1.125, -1.125, 1.375]), 'bf16', F.CONFIGS['e1m2_ocp']),
                                np.float32([1.25, -1.25, 1.5]))
  np.testing.assert_array_equal(F.fp_vjp_fwd(np.float32([0.5625, -0.5625, 0.6875]), 'bf16', F.CONFIGS['e0m3_ocp']),
                                np.float32([0.5, -0.5, 0.75]))


def test_largest_representable():
  """fp_numerics.py:594-615 against the enumerated values."""
  for name, cfg in F.CONFIGS.items():
    assert F.fp_largest_representable(cfg) == F.fp_values(cfg).max(), name


# ---- radix 4 (fp_numerics.py:661-706) -------------------------------------------------------------
def _radix4_buckets():
  """fp_numerics_test.py:342-377 for RADIX4: centres, boundaries halfway between them, except that the
  edge of the zero bucket is where floor(log4(1.6 x)) turns -3, at (4^-3 + 4^-4) / 2."""
  centers = np.unique(F.RADIX4_VALUES.astype(np.float64))
  assert centers[-1] == 64.0
  bounds = (centers[1:] + centers[:-1]) / 2
  edge = centers[-1] + (centers[-1] - bounds[-1])
  bounds = np.concatenate([[-edge], bounds, [edge]])
  bounds = np.where(np.abs(bounds) == 4.0**-3 / 2, np.sign(bounds) * (4.0**-3 + 4.0**-4) / 2, bounds)
  return centers, bounds, edge


def test_radix4_round_to_nearest_and_overflow():
  centers, bounds, edge = _radix4_buckets()
  lower, upper = bounds[:-1], bounds[1:]
  data = nm.cast(np.linspace(lower, upper, 257, endpoint=True, axis=0).astype(np.float32), 'bf16')
  interior = (data > lower[None]) & (data < upper[None])
  assert interior.mean() > 0.9
  q = F.radix4_round(data, 'bf16')
  want = np.broadcast_to(centers[None].astype(np.float32), q.shape)
  np.testing.assert_array_equal(np.where(interior, q, 0), np.where(interior, want, 0))
  for sign in (-1.0, 1.0):
    far = nm.cast(np.linspace(sign * edge, sign * 10 * edge, 129).astype(np.float32), 'bf16')
    far = far[np.abs(far) > edge]
    np.testing.assert_array_equal(F.radix4_round(far, 'bf16'), np.full_like(far, sign * 64.0))
  np.testing.assert_array_equal(F.radix4_round(np.array([0.0, -0.0, 1e-30, -1e-30], np.float32), 'bf16'), np.zeros(4, np.float32))


def test_radix4_equispaced_noise_gives_exact_mean():
  """With the 2^16 equi-spaced noise values the mean of the rounded values is the input (to the
  spacing of the noise), for inputs inside the range of the format: P(up) is the position in the bucket."""
  xs = nm.cast(np.array([0.02, 0.05, 0.3, 0.9, 1.0, 1.7, 3.1, 5.0, 12.0, 17.0, 50.0, -2.5, -40.0], np.float32), 'bf16')
  x = np.broadcast_to(xs[:, None], (xs.size, 2**16)).copy()
  q = F.radix4_round(x, 'bf16', stochastic_rounding=True, test_noise_axis=1)
  assert set(np.unique(np.abs(q))) <= set(np.abs(F.RADIX4_VALUES))
  mean = q.astype(np.float64).mean(axis=1)
  width = 3 * 4.0**np.floor(np.log2(np.abs(xs.astype(np.float64))) / 2)
  np.testing.assert_allclose(mean, xs.astype(np.float64), rtol=0, atol=2.0**-15 * width.max())
  assert np.all(np.abs(mean - xs) <= 2.0**-15 * width)


def test_radix4_log_safety_mask_flags_the_powers_of_four():
  x = nm.cast(np.array([10.0, 2.5, 0.625, 40.0, 3.0, 1.0, 0.3], np.float32), 'bf16')  # 1.6 x = 16, 4, 1, 64: edges
  np.testing.assert_array_equal(F.radix4_log_is_safe(x), [False, False, False, False, True, True, True])
  np.testing.assert_array_equal(F.radix4_log_is_safe(x, stochastic_rounding=True, test_noise_axis=None, key=np.array([0, 1], np.uint32))[5:6], [False])

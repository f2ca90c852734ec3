"""Pins of the oracle's PRNG: Random123 vectors and values JAX documents for PRNGKey(0)."""
import numpy as np
import pytest

from oracle import prng


# Random123 known-answer vectors for Threefry-2x32-20 (kat_vectors of the Random123 distribution).
KAT = [
    ((0x00000000, 0x00000000), (0x00000000, 0x00000000), (0x6B200159, 0x99BA4EFE)),
    ((0xFFFFFFFF, 0xFFFFFFFF), (0xFFFFFFFF, 0xFFFFFFFF), (0x1CB996FC, 0xBB002BE7)),
    ((0x13198A2E, 0x03707344), (0x243F6A88, 0x85A308D3), (0xC4923A9C, 0x483DF7A0)),
]


@pytest.mark.parametrize('key,ctr,want', KAT)
def test_threefry_known_answers(key, ctr, want):
  a, b = prng.threefry2x32(key[0], key[1], [ctr[0]], [ctr[1]])
  assert (int(a[0]), int(b[0])) == want


def test_split_of_key0_matches_published_jax_values():
  # jax.random.split(jax.random.PRNGKey(0)) as printed in JAX's PRNG documentation
  # (original, non-partitionable threefry layout).
  got = prng.split(prng.prng_key(0), 2)
  np.testing.assert_array_equal(got, [[4146024105, 967050713], [2718843009, 1272950319]])


def test_uniform_of_key0_matches_published_jax_value():
  # jax.random.uniform(jax.random.PRNGKey(0)) -> 0.41845703
  u = prng.uniform(prng.prng_key(0), ())
  assert u.dtype == np.float32
  assert abs(float(u) - 0.41845703) < 5e-9


def test_prng_key_layout():
  np.testing.assert_array_equal(prng.prng_key(42), [0, 42])
  np.testing.assert_array_equal(prng.prng_key((7 << 32) | 5), [7, 5])


@pytest.mark.parametrize('n', [1, 2, 5, 8, 33])
def test_original_layout_structure(n):
  """Word i < half comes from lane 0 of block (i, i+half); odd n pads a zero counter."""
  key = prng.prng_key(9)
  bits = prng.random_bits(key, (n,), 32)
  half = (n + 1) // 2
  for i in range(n):
    if i < half:
      c1 = i + half if i + half < n else 0
      want = prng.threefry2x32(key[0], key[1], [i], [c1])[0][0]
    else:
      want = prng.threefry2x32(key[0], key[1], [i - half], [i])[1][0]
    assert bits[i] == want


def test_16bit_draws_are_low_then_high_halves():
  key = prng.prng_key(3)
  w = prng.random_bits(key, (4,), 32)
  h = prng.random_bits(key, (8,), 16)
  np.testing.assert_array_equal(h[0::2], (w & 0xFFFF).astype(np.uint16))
  np.testing.assert_array_equal(h[1::2], (w >> 16).astype(np.uint16))


def test_partitionable_layout_structure():
  key = prng.prng_key(11)
  bits = prng.random_bits(key, (3, 5), 32, partitionable=True)
  for i in range(15):
    a, b = prng.threefry2x32(key[0], key[1], [0], [i])
    assert bits.reshape(-1)[i] == a[0] ^ b[0]
  ks = prng.split(key, 4, partitionable=True)
  for i in range(4):
    a, b = prng.threefry2x32(key[0], key[1], [0], [i])
    assert tuple(ks[i]) == (a[0], b[0])


def test_uniform_range_and_mean():
  u = prng.uniform(prng.prng_key(1), (200000,))
  assert u.min() >= 0.0 and u.max() < 1.0
  assert abs(u.mean() - 0.5) < 3e-3


@pytest.mark.parametrize('partitionable', [False, True])
@pytest.mark.parametrize('total', [1, 2, 7, 64, 1001])
def test_bits_at_positions_match_the_whole_draw(total, partitionable):
  key = prng.prng_key(11)
  whole = prng.random_bits(key, (total,), 32, partitionable)
  idx = np.random.default_rng(total).integers(0, total, size=(3, 5))
  np.testing.assert_array_equal(prng.random_bits_at(key, total, idx, partitionable), whole[idx])
  np.testing.assert_array_equal(prng.uniform_at(key, total, np.arange(total), partitionable),
                                prng.uniform(key, (total,), partitionable))
  halves = prng.random_bits(key, (total,), 16, partitionable)
  np.testing.assert_array_equal(prng.random_bits_at(key, total, idx, partitionable, 16), halves[idx])


def test_noise_window_is_the_slice_of_the_full_noise():
  from oracle import aqt_ref as R
  key = prng.prng_key(5)
  full = R.jax_uniform_noise((6, 10), key)
  rows, cols = [4, 1, 5], [0, 9, 3, 2]
  got = R.jax_uniform_noise_window((3, 4), key, ((6, 10), (rows, cols)))
  np.testing.assert_array_equal(got, full[np.ix_(rows, cols)])


def test_fp8_mantissa_noise_window_is_the_slice_of_the_full_draw():
  from oracle import aqt_ref as R
  from oracle import numerics as nm
  key = prng.prng_key(8)
  x = nm.cast(np.random.default_rng(0).standard_normal((7, 9)).astype(np.float32), 'bf16')
  rows, cols = [6, 0, 3], [8, 1, 2, 5]
  for dt in ('bf16', 'f32'):
    full = R.fp_mantissa_round(x, dt, 2, key)
    got = R.fp_mantissa_round(x[np.ix_(rows, cols)], dt, 2, key, ((7, 9), (rows, cols)))
    np.testing.assert_array_equal(got, full[np.ix_(rows, cols)])

"""Threefry2x32 and the jax.random bit layouts (test infrastructure).

The reference draws all its noise from `jax.random` (third-party, version
unpinned in the reference's pyproject.toml:18-23):
  * `jax.random.split`    -- aqt/jax/v2/config.py:61-63
  * `jax.random.uniform`  -- aqt/jax/v2/stochastic_rounding.py:46
  * `jax.random.bits`     -- aqt/jax/v2/stochastic_rounding.py:65,
                             aqt/jax/v2/numerics/fp8_numerics.py:54
JAX is not vendored in the reference, so its published algorithm is restated
here: Threefry-2x32 with 20 rounds (Salmon et al., "Parallel random numbers: as
easy as 1, 2, 3", SC'11; Random123) and the two counter layouts JAX uses
(`jax_threefry_partitionable` False / True).
"""
import numpy as np

_ROT = ((13, 15, 26, 6), (17, 29, 16, 24))
_PARITY = np.uint32(0x1BD11BDA)


def _rotl(x, r):
  return (x << np.uint32(r)) | (x >> np.uint32(32 - r))


def threefry2x32(k0, k1, x0, x1):
  """Threefry-2x32-20 block function on uint32 arrays (Random123 ordering)."""
  with np.errstate(over='ignore'):
    k0 = np.uint32(k0)
    k1 = np.uint32(k1)
    x0 = np.array(x0, dtype=np.uint32, copy=True)
    x1 = np.array(x1, dtype=np.uint32, copy=True)
    ks = (k0, k1, np.uint32(k0 ^ k1 ^ _PARITY))
    x0 = x0 + ks[0]
    x1 = x1 + ks[1]
    for block in range(5):
      for r in _ROT[block % 2]:
        x0 = x0 + x1
        x1 = _rotl(x1, r)
        x1 = x1 ^ x0
      x0 = x0 + ks[(block + 1) % 3]
      x1 = x1 + ks[(block + 2) % 3] + np.uint32(block + 1)
  return x0, x1


def prng_key(seed):
  """jax.random.PRNGKey(seed): raw key data [hi32(seed), lo32(seed)]."""
  seed = int(seed) & 0xFFFFFFFFFFFFFFFF
  return np.array([seed >> 32, seed & 0xFFFFFFFF], dtype=np.uint32)


def _threefry_2x32_flat(key, count):
  """jax._src.prng.threefry_2x32: split the counts in halves as the two lanes."""
  count = np.asarray(count, np.uint32).ravel()
  odd = count.size % 2
  if odd:
    count = np.concatenate([count, np.zeros(1, np.uint32)])
  half = count.size // 2
  y0, y1 = threefry2x32(key[0], key[1], count[:half], count[half:])
  out = np.concatenate([y0, y1])
  return out[:-1] if odd else out


def split(key, num, partitionable=False):
  """jax.random.split(key, num) -> uint32[num, 2]."""
  key = np.asarray(key, np.uint32)
  if partitionable:
    idx = np.arange(num, dtype=np.uint64)
    b1, b2 = threefry2x32(key[0], key[1], (idx >> np.uint64(32)).astype(np.uint32),
                          (idx & np.uint64(0xFFFFFFFF)).astype(np.uint32))
    return np.stack([b1, b2], axis=1)
  return _threefry_2x32_flat(key, np.arange(2 * num, dtype=np.uint32)).reshape(num, 2)


def random_bits(key, shape, bit_width=32, partitionable=False):
  """jax.random.bits(key, shape, uint{bit_width}) for bit_width in {8,16,32}."""
  key = np.asarray(key, np.uint32)
  shape = tuple(int(s) for s in shape)
  size = int(np.prod(shape, dtype=np.int64)) if shape else 1
  out_dtype = {8: np.uint8, 16: np.uint16, 32: np.uint32}[bit_width]
  if partitionable:
    idx = np.arange(size, dtype=np.uint64)
    b1, b2 = threefry2x32(key[0], key[1], (idx >> np.uint64(32)).astype(np.uint32),
                          (idx & np.uint64(0xFFFFFFFF)).astype(np.uint32))
    return (b1 ^ b2).astype(out_dtype).reshape(shape)
  max_count = -(-(bit_width * size) // 32)
  words = _threefry_2x32_flat(key, np.arange(max_count, dtype=np.uint32))
  if bit_width == 32:
    return words.reshape(shape)
  per = 32 // bit_width
  shifts = (np.arange(per, dtype=np.uint32) * np.uint32(bit_width))[None, :]
  parts = (words[:, None] >> shifts) & np.uint32((1 << bit_width) - 1)
  return parts.reshape(-1)[:size].astype(out_dtype).reshape(shape)


def random_bits_at(key, total, idx, partitionable=False, bit_width=32):
  """jax.random.bits(key, (total,), uint{bit_width})[idx] without drawing the other elements.

  32 bits: word i of the first half of the counters is lane 0 of block (i, i + half), word i of
  the second half is lane 1 of block (i - half, i); an odd count pads one zero counter (see
  _threefry_2x32_flat).  16 bits: element i is the low (even i) or high half of word i // 2 of
  the ceil(total / 2) words drawn (see random_bits)."""
  key = np.asarray(key, np.uint32)
  idx = np.asarray(idx, np.int64)
  assert bit_width in (16, 32)
  assert idx.size == 0 or (idx.min() >= 0 and idx.max() < total)
  flat = idx.ravel()
  if partitionable:
    b1, b2 = threefry2x32(key[0], key[1], (flat >> 32).astype(np.uint32), (flat & 0xFFFFFFFF).astype(np.uint32))
    bits = b1 ^ b2
    return (bits & np.uint32(0xFFFF) if bit_width == 16 else bits).reshape(idx.shape)
  if bit_width == 16:
    words = random_bits_at(key, -(-int(total) // 2), flat // 2, False, 32)
    return ((words >> (np.uint32(16) * (flat % 2).astype(np.uint32))) & np.uint32(0xFFFF)).reshape(idx.shape)
  half = (int(total) + 1) // 2
  first = flat < half
  c0 = np.where(first, flat, flat - half)
  c1 = np.where(first, flat + half, flat)
  c1 = np.where(c1 < total, c1, 0)  # the padded counter of an odd total
  y0, y1 = threefry2x32(key[0], key[1], c0.astype(np.uint32), c1.astype(np.uint32))
  return np.where(first, y0, y1).reshape(idx.shape)


def uniform_at(key, total, idx, partitionable=False):
  """jax.random.uniform(key, (total,))[idx]."""
  bits = random_bits_at(key, total, idx, partitionable)
  fbits = (bits >> np.uint32(9)) | np.uint32(0x3F800000)
  return np.maximum(np.float32(0.0), fbits.view(np.float32) - np.float32(1.0))


def uniform(key, shape, partitionable=False):
  """jax.random.uniform(key, shape) (float32, [0, 1))."""
  bits = random_bits(key, shape, 32, partitionable)
  fbits = (bits >> np.uint32(9)) | np.uint32(0x3F800000)
  floats = fbits.view(np.float32) - np.float32(1.0)
  return np.maximum(np.float32(0.0), floats)

"""numpy restatement of aqt.jax.v2.numerics.fp_numerics (test infrastructure).

Emulated small floats (e2m1, e3m0, the OCP fp4/fp5/fp6 variants ...) held in a bf16 or f32
container.  Two independent formulations of the same rounding are restated, as the reference
holds two (`radix2_round`, the one `fp_round` dispatches to, fp_numerics.py:300-459, and
`fp_round_new`, fp_numerics.py:462-591) and tests them equal on every bf16 bit pattern
(fp_numerics_test.py:517-604).  Pins: that equality; round-to-nearest against the enumerated
representable values and clamping of overflows (fp_numerics_test.py:296-440); exactness of
the mean under equi-spaced noise (fp_numerics_test.py:442-460); the representable-value tables
(fp_numerics_test.py:169-293).

radix-4 rounding (`radix4_round`, fp_numerics.py:661-706) is restated as written, through float32
log(): floor(log(z) / log(4)).  Pins: every interior point of every bucket goes to the bucket's
centre, zero below 4^-3 and +-64 above (the reference's own bucket test, fp_numerics_test.py:330-440,
with its shifted edge of the lowest bucket, :364-377); the mean under equi-spaced noise.  Where z is
a power of 4 to within a float32 ulp the result depends on the last bit of the library's log():
parity unpinned at those arguments (the reference's test leaves the bucket edges out as well);
`radix4_log_is_safe` says which arguments are clear of them.

Arrays: float32 numpy arrays whose values are representable in the container dtype ('bf16' or
'f32'), like the rest of the oracle.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import numpy as np

from oracle import numerics as nm
from oracle import prng


@dataclasses.dataclass(frozen=True)
class FpNumericsConfig:
  """fp_numerics.py:26-34."""
  nexp: int
  minexp: int
  nmant: int
  has_subnormals: bool
  has_two_nan: bool = False
  has_naninf: bool = False
  radix: int = 2


def _cfg(nexp, nmant, sub):
  return FpNumericsConfig(nexp=nexp, minexp=0, nmant=nmant, has_subnormals=sub)


# fp_numerics.py:36-268 (name -> config)
CONFIGS = {
    'e5m0_ocp': _cfg(5, 0, True), 'e4m1_ocp': _cfg(4, 1, True), 'e3m2_ocp': _cfg(3, 2, True),
    'e2m3_ocp': _cfg(2, 3, True), 'e1m4_ocp': _cfg(1, 4, True), 'e0m5_ocp': _cfg(0, 5, True),
    'e4m0_ocp': _cfg(4, 0, True), 'e3m1_ocp': _cfg(3, 1, True), 'e2m2_ocp': _cfg(2, 2, True),
    'e1m3_ocp': _cfg(1, 3, True), 'e0m4_ocp': _cfg(0, 4, True),
    'e3m0': _cfg(3, 0, False), 'e3m0_ocp': _cfg(3, 0, True), 'e2m1': _cfg(2, 1, False),
    'e2m1_ocp': _cfg(2, 1, True), 'e1m2': _cfg(1, 2, False), 'e1m2_ocp': _cfg(1, 2, True),
    'e0m3': _cfg(0, 3, False), 'e0m3_ocp': _cfg(0, 3, True), 'e1m0': _cfg(1, 0, False),
}


def fp_largest_representable(cfg: FpNumericsConfig) -> float:
  """fp_numerics.py:594-615."""
  assert cfg.minexp == 0 and not cfg.has_naninf and cfg.radix == 2
  max_exp = 2**cfg.nexp - 1 + cfg.minexp - (1 if cfg.has_subnormals else 0)
  max_mant = 2**cfg.nmant - 1 - (1 if cfg.has_two_nan else 0)
  max_normal = 2**max_exp * (1 + (max_mant / 2**cfg.nmant))
  max_subnormal = 2**cfg.minexp * max_mant / 2**cfg.nmant
  if cfg.has_subnormals and cfg.nexp == 0:
    return max_subnormal
  return max_normal


def _container(dt):
  # (mantissa bits, total bits)
  return (7, 16) if dt == 'bf16' else (23, 32)


def _to_bits(x, dt):
  b = np.ascontiguousarray(x, np.float32).view(np.uint32)
  return (b >> np.uint32(16)) if dt == 'bf16' else b.copy()


def _from_bits(b, dt):
  b = b.astype(np.uint32)
  if dt == 'bf16':
    b = b << np.uint32(16)
  return b.view(np.float32)


def _noise_bits(shape, key, test_noise_axis):
  """16 random bits per element: jax.random.bits(key, shape, uint16), or the index along
  `test_noise_axis` (the reference's deterministic stand-in, fp_numerics.py:334-340)."""
  if test_noise_axis is not None:
    n = shape[test_noise_axis]
    sh = [1] * len(shape)
    sh[test_noise_axis] = n
    return np.broadcast_to(np.arange(n, dtype=np.uint32).astype(np.uint16).reshape(sh), shape).astype(np.uint32)
  return prng.random_bits(key, shape, 16, prng_partitionable()).astype(np.uint32)


def prng_partitionable():
  from oracle import aqt_ref
  return aqt_ref.PARTITIONABLE


def radix2_round(x, dt, cfg: FpNumericsConfig, key=None, stochastic_rounding=False, test_noise_axis=None):
  """fp_numerics.py:300-459.  x: float32 array of dt-representable values; returns the same."""
  nexp, nmant = cfg.nexp, cfg.nmant
  assert cfg.minexp == 0 and not cfg.has_two_nan and not cfg.has_naninf
  x = np.ascontiguousarray(x, np.float32)
  cm, total = _container(dt)
  wrap = np.uint32(0xFFFF) if total == 16 else np.uint32(0xFFFFFFFF)
  assert nmant < cm
  trunc = cm - nmant
  trunc_mask = np.uint32((1 << trunc) - 1)
  xb = _to_bits(x, dt)
  rnd = _noise_bits(x.shape, key, test_noise_axis) if stochastic_rounding else None
  if stochastic_rounding:
    noise = rnd.copy()
    if trunc > 16:
      noise = ((noise << np.uint32(1)) | np.uint32(1)) & wrap
      noise = (noise << np.uint32(trunc - 16 - 1)) & wrap
    noise = noise & trunc_mask
  else:
    noise = np.uint32(1 << (trunc - 1))
  xb = (xb + noise) & wrap  # unsigned addition in the container width; the carry may reach the exponent
  xb = xb & (~trunc_mask & wrap)

  min_exp = 127 - (1 if cfg.has_subnormals else 0)
  max_exp = min_exp + 2**nexp - 1
  min_repr = np.uint32(min_exp << cm)
  min_repr_float = _from_bits(np.array([min_repr], np.uint32), dt)[0]
  mant_mask = np.uint32((1 << cm) - 1)
  max_mant = mant_mask & ~trunc_mask
  max_repr = np.uint32((max_exp << cm) + int(max_mant))
  sign_mask = np.uint32(1 << (total - 1))
  sign = xb & sign_mask
  abs_x = xb & (~sign_mask & wrap)
  clip_x = np.clip(abs_x, min_repr, max_repr)
  out = _from_bits(sign | clip_x, dt)
  if cfg.has_subnormals:
    ob = _to_bits(x, dt)
    orig_abs = ob & (~sign_mask & wrap)
    orig_clip = np.clip(orig_abs, min_repr, max_repr)
    exp = orig_clip & (~mant_mask & wrap)
    with np.errstate(invalid='ignore', over='ignore'):
      scaled = nm.cast(x * np.float32(2**nmant), dt)
    if stochastic_rounding:
      rb = (rnd << np.uint32(7)) | np.uint32(0x3F800000)
      nz = (rb.view(np.float32) - np.float32(1.5)) + np.float32(2.0**-17)
      t = scaled + nz  # float32 in both containers: the noise is float32
      sub = np.rint(t) / np.float32(2**nmant)
    else:
      sub = np.rint(scaled) / np.float32(2**nmant)  # stays in the container dtype; exact
    with np.errstate(invalid='ignore', over='ignore'):
      sub = nm.cast(sub.astype(np.float32), dt)
    out = np.where(exp == min_repr, sub, out)
  elif stochastic_rounding:
    rb = (rnd << np.uint32(7)) | np.uint32(0x40000000)
    rnd_floats = rb.view(np.float32) - np.float32(3.0 - 2.0**-16)
    rx = np.where(x > rnd_floats, np.float32(1.0), np.float32(-1.0))
    out = np.where(np.abs(x) < min_repr_float, rx, out)
  if nexp == 0 and cfg.has_subnormals:
    max_subnormal = np.float32(2**cfg.minexp * (1 - 2.0**(-nmant)))
    out = np.clip(out, -max_subnormal, max_subnormal)
  return out.astype(np.float32)


def fp_round_new(x, dt, cfg: FpNumericsConfig, key=None, stochastic_rounding=False, test_noise_axis=None):
  """fp_numerics.py:462-591: the second formulation (sign and magnitude handled as floats)."""
  nexp, nmant = cfg.nexp, cfg.nmant
  assert cfg.minexp == 0 and not cfg.has_two_nan and not cfg.has_naninf
  x = np.ascontiguousarray(x, np.float32)
  cm, total = _container(dt)
  wrap = np.uint32(0xFFFF) if total == 16 else np.uint32(0xFFFFFFFF)
  mant_mask = np.uint32((1 << cm) - 1)
  trunc = cm - nmant
  trunc_mask = np.uint32((1 << trunc) - 1)
  sign_mask = np.uint32(1 << (total - 1))
  min_normal = np.float32(2.0**cfg.minexp)
  min_normal_repr = _to_bits(np.array([min_normal], np.float32), dt)[0]
  bias = 1 if cfg.has_subnormals else 0
  min_ctner_exp = 127 - bias
  max_ctner_exp = min_ctner_exp + 2**nexp - 1
  max_ctner_mant = mant_mask & ~trunc_mask
  max_normal = _from_bits(np.array([(max_ctner_exp << cm) + int(max_ctner_mant)], np.uint32), dt)[0]
  max_subnormal = np.float32(2**cfg.minexp * (1 - 2.0**(-nmant)))
  rnd = _noise_bits(x.shape, key, test_noise_axis) if stochastic_rounding else None

  with np.errstate(invalid='ignore', over='ignore'):
    sgn = np.sign(x)
    b = _to_bits(np.abs(x), dt)
    if stochastic_rounding:
      r = rnd.copy()
      if trunc > 16:
        r = ((r << np.uint32(1)) | np.uint32(1)) & wrap
        r = (r << np.uint32(trunc - 16 - 1)) & wrap
      b = (b + (r & trunc_mask)) & wrap
    else:
      b = (b + np.uint32(1 << (trunc - 1))) & wrap
    b = b & (~trunc_mask & wrap)
    normal = np.clip(_from_bits(b, dt), min_normal, max_normal)
    # jnp.clip propagates NaN
    normal = np.where(np.isnan(_from_bits(b, dt)), np.float32(np.nan), normal) * sgn

    if cfg.has_subnormals:
      scaled = nm.cast(x * np.float32(2**nmant), dt)
      if stochastic_rounding:
        rb = (rnd << np.uint32(7)) | np.uint32(0x3F800000)
        nz = (rb.view(np.float32) - np.float32(1.5)) + np.float32(2.0**-17)
        sub = np.rint(scaled + nz) / np.float32(2**nmant)
      else:
        sub = np.rint(scaled) / np.float32(2**nmant)
      sub = nm.cast(sub.astype(np.float32), dt)
    elif stochastic_rounding:
      rb = (rnd << np.uint32(7)) | np.uint32(0x40000000)
      rnd_floats = rb.view(np.float32) - np.float32(3.0 - 2.0**-16)
      sub = np.where(x > rnd_floats, np.float32(1.0), np.float32(-1.0))
    else:
      sub = _from_bits((_to_bits(x, dt) & sign_mask) | min_normal_repr, dt)
    out = np.where(np.abs(x) < min_normal, sub, normal)
    if nexp == 0 and cfg.has_subnormals:
      out = np.clip(out, -max_subnormal, max_subnormal)
  return out.astype(np.float32)


RADIX4_VALUES = np.array([0.0] + [4.0**e for e in range(-3, 4)] + [-(4.0**e) for e in range(-3, 4)], np.float32)


def _radix4_args(x, key, stochastic_rounding, test_noise_axis, coeff):
  """The float32 argument whose floor(log4) picks the bucket (fp_numerics.py:679-700)."""
  x = np.asarray(x, np.float32)
  f32 = np.float32
  with np.errstate(divide='ignore', invalid='ignore', over='ignore'):
    if not stochastic_rounding:
      return np.abs(f32(coeff) * x)
    abs_x = np.abs(x)
    lower_ebit = np.floor(np.log(abs_x) / np.log(f32(4)))
    lower = np.power(f32(4), lower_ebit, dtype=np.float32)
    higher = np.power(f32(4), lower_ebit + f32(1), dtype=np.float32)
    bucket_size = higher - lower
    if test_noise_axis is not None:
      assert x.shape[test_noise_axis] == 2**16, 'Input repetition should be consistent with effective noise bits.'
    rnd = _noise_bits(x.shape, key, test_noise_axis)
    noise = ((rnd.astype(np.uint32) << np.uint32(7)) | np.uint32(0x3F800000)).view(np.float32) - f32(1.0)
    return abs_x + noise * bucket_size


def radix4_log_is_safe(x, key=None, stochastic_rounding=False, test_noise_axis=None, coeff=1.6):
  """False where the argument of the logarithm (of either logarithm, with stochastic rounding) lies within four
  float32 ulps of one of the powers of 4 at which the result changes (4^-4 .. 4^3), i.e. where
  floor(log(z)/log(4)) hangs on the last bit of log()."""
  def clear(z):
    z = np.asarray(z, np.float32).astype(np.float64)
    ok = np.ones(z.shape, bool)
    for k in range(-4, 4):
      p = 4.0**k
      ok &= ~(np.abs(z - p) <= 4 * float(np.spacing(np.float32(p))))
    return ok
  ok = clear(_radix4_args(x, key, stochastic_rounding, test_noise_axis, coeff))
  if stochastic_rounding:
    ok &= clear(np.abs(np.asarray(x, np.float32)))
  return ok


def radix4_round(x, dt, key=None, stochastic_rounding=False, test_noise_axis=None, coeff=1.6):
  """radix4_round (fp_numerics.py:661-706): to the nearest of {0, +-4^-3 .. +-4^3}; bf16 in and out."""
  assert dt == 'bf16', f'Unsupported dtype for sthochastic rounding: {dt}.'
  x = np.asarray(x, np.float32)
  f32 = np.float32
  z = _radix4_args(x, key, stochastic_rounding, test_noise_axis, coeff)
  with np.errstate(divide='ignore', invalid='ignore', over='ignore'):
    ebit = np.floor(np.log(z) / np.log(f32(4)))
    subnormal = np.zeros_like(x)
    overflow = np.sign(x) * f32(64)
    radix4 = np.sign(x) * np.power(f32(4), ebit, dtype=np.float32)
    ret = np.where(ebit < -3, subnormal, np.where(ebit >= 3, overflow, radix4))
  return nm.cast(ret.astype(np.float32), 'bf16')


def fp_values(cfg: FpNumericsConfig):
  """Every value the format holds, by bit pattern (sign, exponent, mantissa): the definition
  of the format, independent of the rounding code (restates the enumeration the reference's
  test builds, fp_numerics_test.py:71-113)."""
  bits = 1 + cfg.nexp + cfg.nmant
  vals = []
  for m in range(2**bits):
    s = -1.0 if (m >> (cfg.nexp + cfg.nmant)) else 1.0
    e = (m >> cfg.nmant) & ((1 << cfg.nexp) - 1)
    man = m & ((1 << cfg.nmant) - 1)
    if cfg.has_subnormals and e == 0:
      vals.append(s * 2.0**cfg.minexp * (man / 2**cfg.nmant))
    else:
      ee = e - 1 if cfg.has_subnormals else e
      vals.append(s * 2.0**(ee + cfg.minexp) * (1 + man / 2**cfg.nmant))
  return np.array(vals, np.float32)


def fp_vjp_fwd(x, dt, cfg: FpNumericsConfig, key: Optional[np.ndarray] = None, stochastic_rounding=False):
  """FpNumerics.vjp_fwd (fp_numerics.py:632-640): the input is cast to bf16 first; bf16 out."""
  del dt
  return radix2_round(nm.cast(np.asarray(x, np.float32), 'bf16'), 'bf16', cfg, key, stochastic_rounding)

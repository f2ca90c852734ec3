"""Low-precision float formats in numpy (test infrastructure).

bf16 and fp8 values are carried as float32 arrays whose values are exactly
representable in the narrow format; `to_*` rounds (round-to-nearest-even, the
rounding `astype` performs in the reference: numerics/fp8_numerics.py:136-137,
aqt_tensor.py:179).
"""
import numpy as np

F32 = 'f32'
BF16 = 'bf16'


def to_bf16(x):
  """float32 -> nearest bf16 (ties to even), returned as float32."""
  x = np.ascontiguousarray(x, dtype=np.float32)
  u = x.view(np.uint32)
  with np.errstate(over='ignore'):
    r = (u + (((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF))) & np.uint32(0xFFFF0000)
  r = np.where(np.isnan(x), u | np.uint32(0x00400000), r).astype(np.uint32)
  return r.view(np.float32)


def bf16_bits(x):
  """uint16 bit pattern of bf16-representable float32 values."""
  return (np.ascontiguousarray(x, np.float32).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def from_bf16_bits(b):
  return (np.asarray(b, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def cast(x, dtype):
  x = np.asarray(x, np.float32)
  return to_bf16(x) if dtype == BF16 else x


def promote(a, b):
  return F32 if F32 in (a, b) else BF16


def _round_to_format(x, exp_bits, man_bits, max_finite):
  """RTNE of float32 `x` to a small float format with subnormals, no inf saturation.

  Values whose rounding exceeds max_finite become NaN (e4m3fn) / inf (e5m2) in
  real hardware; the reference clips to +-max before casting
  (numerics/fp8_numerics.py:119-120), so callers never reach that range; here
  they are returned as +-inf to make a violation visible.
  """
  x = np.asarray(x, np.float64)
  bias = (1 << (exp_bits - 1)) - 1
  min_normal_exp = 1 - bias
  ax = np.abs(x)
  with np.errstate(divide='ignore', invalid='ignore'):
    e = np.floor(np.log2(np.where(ax > 0, ax, 1.0)))
  e = np.maximum(e, min_normal_exp)
  ulp = np.exp2(e - man_bits)
  q = np.rint(ax / ulp) * ulp  # np.rint is round-half-even; ax/ulp is exact
  out = np.where(q > max_finite, np.inf, q)
  out = np.copysign(out, x)
  out = np.where(np.isnan(x), np.nan, out)
  return out.astype(np.float32)


E4M3_MAX = 448.0
E5M2_MAX = 57344.0


def to_e4m3fn(x):
  return _round_to_format(x, 4, 3, E4M3_MAX)


def to_e5m2(x):
  return _round_to_format(x, 5, 2, E5M2_MAX)


def e4m3fn_bits(x):
  """uint8 encoding of e4m3fn-representable values."""
  return _encode(x, 4, 3)


def e5m2_bits(x):
  return _encode(x, 5, 2)


def _encode(x, exp_bits, man_bits):
  x = np.asarray(x, np.float64)
  bias = (1 << (exp_bits - 1)) - 1
  sign = (np.signbit(x)).astype(np.uint8) << np.uint8(7)
  ax = np.abs(x)
  with np.errstate(divide='ignore'):
    e = np.floor(np.log2(np.where(ax > 0, ax, 1.0)))
  sub = (ax < 2.0 ** (1 - bias))
  e_field = np.where(sub, 0, e + bias).astype(np.int64)
  m = np.where(sub, ax / 2.0 ** (1 - bias - man_bits),
               (ax / np.exp2(e) - 1.0) * (1 << man_bits))
  m = np.rint(m).astype(np.int64)
  return (sign | ((e_field << man_bits) | m).astype(np.uint8)).astype(np.uint8)


def int32_to_float(acc, dtype):
  """int32 accumulator -> dequant dtype (aqt_tensor.py:179 `qvalue.astype`).

  XLA lowers integer->bf16 converts as int->f32 (RTNE) followed by f32->bf16
  (RTNE); that two-step rounding is restated here.  For |acc| < 2**24 it is
  identical to a single rounding.
  """
  f = np.asarray(acc).astype(np.float32)
  return to_bf16(f) if dtype == BF16 else f

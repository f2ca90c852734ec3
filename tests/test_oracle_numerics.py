"""Pins of the oracle's number formats and element numerics."""
import numpy as np
import pytest
import torch

from oracle import aqt_ref as R
from oracle import numerics as nm

# Input rows of numerics/fp8_numerics_test.py:50-65 in the reference.
FP8_X = np.array(
    [[0, 1, -1, 0.1234567, 100, 0.5, 0.00000000001, 0.01],
     [-2.9098532, -0.8508397, -0.14903745, -3.572757, 0.63277215, 0.7478278, 1.3707844, 1.3319879]],
    dtype=np.float32)


def test_fp8_e5m2_reference_golden():
  # numerics/fp8_numerics_test.py:69-78
  want = np.array([[0, 1, -1, 0.125, 96, 0.5, 0, 10 / 1024],
                   [-3, -0.875, -0.15625, -3.5, 0.625, 0.75, 1.25, 1.25]], np.float32)
  np.testing.assert_array_equal(nm.to_e5m2(FP8_X), want)


def test_fp8_e4m3_reference_golden():
  # numerics/fp8_numerics_test.py:101-110
  want = np.array([[0, 1, -1, 0.125, 96, 0.5, 0, 10 / 1024],
                   [-3, -0.875, -0.15625, -3.5, 0.625, 0.75, 1.375, 1.375]], np.float32)
  np.testing.assert_array_equal(nm.to_e4m3fn(FP8_X), want)


def test_fp8_113_114_round_to_112():
  # numerics/fp8_numerics_test.py:232-242
  x = np.array([113.0, 114.0], np.float32)
  np.testing.assert_array_equal(nm.to_e4m3fn(x), [112.0, 112.0])
  np.testing.assert_array_equal(nm.to_e5m2(x), [112.0, 112.0])


@pytest.mark.parametrize('fn,tdt,enc,bound', [
    (nm.to_e4m3fn, torch.float8_e4m3fn, nm.e4m3fn_bits, 448.0),
    (nm.to_e5m2, torch.float8_e5m2, nm.e5m2_bits, 57344.0),
])
def test_fp8_against_library_cast(fn, tdt, enc, bound):
  rng = np.random.default_rng(0)
  x = np.concatenate([
      rng.standard_normal(200000).astype(np.float32) * np.float32(50),
      np.exp2(rng.uniform(-24, 9, 100000)).astype(np.float32),
      np.array([0.0, -0.0, bound, -bound], np.float32)])
  x = np.clip(x, -bound, bound)
  t = torch.from_numpy(x).to(tdt)
  np.testing.assert_array_equal(fn(x), t.float().numpy())
  np.testing.assert_array_equal(enc(fn(x)), t.view(torch.uint8).numpy())


def test_bf16_against_library_cast():
  rng = np.random.default_rng(1)
  x = np.concatenate([rng.standard_normal(300000).astype(np.float32) * np.float32(1e3),
                      np.exp2(rng.uniform(-60, 60, 100000)).astype(np.float32)])
  np.testing.assert_array_equal(nm.to_bf16(x), torch.from_numpy(x).to(torch.bfloat16).float().numpy())
  # exhaustive ties: every bf16 midpoint rounds to even
  b = np.arange(0x3F80, 0x4000, dtype=np.uint32)
  mid = ((b << np.uint32(16)) | np.uint32(0x8000)).view(np.float32)
  got = nm.bf16_bits(nm.to_bf16(mid))
  np.testing.assert_array_equal(got & 1, 0)


def test_int32_to_bf16_two_step_rounding():
  # 2**24 + 2**16 + 1 lies just above the bf16 tie 2**24 + 2**16: int->f32 drops the 1 (ties to
  # even at ulp 2), f32->bf16 then sees an exact tie and goes to the even mantissa 2**24, while
  # a single rounding of the integer goes up to 2**24 + 2**17.
  v = np.array([(1 << 24) + (1 << 16) + 1], np.int32)
  two_step = nm.int32_to_float(v, 'bf16')
  assert two_step[0] == np.float32(1 << 24)
  # exact arithmetic: the distance to 2**24 exceeds half a bf16 ulp (2**16), so one rounding goes up
  assert int(v[0]) - (1 << 24) > (1 << 16)


@pytest.mark.parametrize('pz,pmv,b8,b2,b1', [
    (False, False, 128.0, 2.0, 1.0), (False, True, 127.5, 1.5, 0.5),
    (True, False, 127.5, 1.5, 0.5), (True, True, 127.0, 1.0, 0.0),
])
def test_int_quant_bound_table(pz, pmv, b8, b2, b1):
  # the table in numerics/int_numerics.py:42-49
  for bits, want in ((8, b8), (2, b2), (1, b1)):
    q = R.QuantizerCfg(bits=bits, preserve_zero=pz, preserve_max_val=pmv)
    assert R.int_quant_bound(q) == want


@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('pmv', [False, True])
def test_int_quant_range(bits, pmv):
  # numerics/int_numerics_test.py:58-115: values stay in the restricted symmetric range
  step = 0.25
  for lo, hi in ((-2, 1), (-1, 1), (-1, 2)):
    x = np.arange(lo, hi + step / 2, step, dtype=np.float32)[None]
    qt = R.quantize(x, 'f32', R.QuantizerCfg(bits=bits, preserve_max_val=pmv), [1])
    assert qt.qvalue.max() <= 2 ** (bits - 1) - 1
    assert qt.qvalue.min() >= -(2 ** (bits - 1)) + 1


def test_rtne_and_clip():
  q = R.QuantizerCfg(bits=8)
  x = np.array([[0.5, 1.5, 2.5, -0.5, -1.5, 126.5, 127.4, 300.0, -300.0]], np.float32)
  v, dt = R.int_vjp_fwd(x, 'f32', q)
  np.testing.assert_array_equal(v, [[0, 2, 2, 0, -2, 126, 127, 127, -127]])
  assert dt == 'i8'


def test_absmax_scale_closed_form():
  x = np.array([[1.0, -255.0, 3.0], [0.0, 0.0, 0.0]], np.float32)
  s, sdt = R.calibrate(x, 'f32', [1], R.QuantizerCfg(bits=8))
  np.testing.assert_array_equal(s, [[np.float32(255.0) / np.float32(127.5)], [np.float32(1.0) / np.float32(127.5)]])
  # bf16 input: the division result is rounded to bf16, also when stored as f32
  xb = nm.to_bf16(np.array([[0.3, -1.7, 2.9]], np.float32))
  sb, _ = R.calibrate(xb, 'bf16', [1], R.QuantizerCfg(bits=8, scale_dtype='f32'))
  assert sb[0, 0] == nm.to_bf16(np.float32(np.abs(xb).max()) / np.float32(127.5))


def test_fp_mantissa_round_properties():
  from oracle import prng
  x = nm.to_bf16(np.random.default_rng(0).standard_normal(4096).astype(np.float32))
  for mant in (3, 2):
    y = R.fp_mantissa_round(x, 'bf16', mant, prng.prng_key(5))
    low = nm.bf16_bits(y) & ((1 << (7 - mant)) - 1)
    np.testing.assert_array_equal(low, 0)  # low mantissa bits cleared
    assert np.all(np.abs(y) >= np.abs(nm.from_bf16_bits(nm.bf16_bits(x) & ~np.uint16((1 << (7 - mant)) - 1))))
  # unbiased within 5 standard errors (shape of numerics/fp8_numerics_test.py:184-215)
  v = np.full(200000, 1.3, np.float32)
  y = R.fp_mantissa_round(nm.to_bf16(v), 'bf16', 2, prng.prng_key(0))
  err = y - nm.to_bf16(v)
  assert abs(err.mean()) < 5 * err.std() / np.sqrt(err.size)


def test_custom1_noise_range():
  from oracle import prng
  n = R.random_centered_uniform_noise((100000,), prng.prng_key(2))
  assert n.dtype == np.float32 and n.min() >= -0.5 and n.max() <= 0.5
  assert abs(n.mean()) < 3e-3

"""Emulated small floats: the HIP kernel behind fp_numerics.fp_round against the oracle, bit for
bit, and the reference's own properties restated on the GPU path (fp_numerics_test.py)."""
import ctypes

import numpy as np
import pytest
import torch

from aqt_amd import _lib as L
from oracle import fp_ref as F
from oracle import numerics as nm
from oracle import prng
from tests import gpu_util as U


def _cfg(name):
  from aqt_amd.v2.numerics import fp_numerics
  return getattr(fp_numerics, name)


def _all_bf16(gpu):
  bits = np.arange(2**16, dtype=np.uint32)
  x = (bits << np.uint32(16)).view(np.float32)
  t = torch.from_numpy(bits.astype(np.int32)).to(gpu).to(torch.int16).view(torch.bfloat16)
  return x, t


def _eq_outside_nan(got: torch.Tensor, want: np.ndarray, x: np.ndarray):
  """Bit patterns (-0 and +0 are different results) wherever the oracle's result is a number.
  NaN inputs are included: the integer steps of fp_numerics.py:300-459 clamp a NaN pattern to
  the largest value like any other, only the float steps of the subnormal branch keep it NaN."""
  del x
  got = got.float().cpu().numpy().reshape(-1)
  want = want.reshape(-1)
  ok = ~np.isnan(want)
  np.testing.assert_array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
  assert np.isnan(got[~ok]).all()


def test_fp_round_plan_validation():
  fake = ctypes.c_void_p(0x1000)

  def err(**kw):
    p = L.FpRoundPlan()
    p.count, p.dtype, p.nexp, p.nmant, p.has_subnormals, p.mode = 16, L.BF16, 2, 1, 1, L.FP_NEAREST
    for k, v in kw.items():
      setattr(p, k, v)
    assert L.lib().aqtx_fp_round(ctypes.byref(p), fake, fake, None, None) != 0
    return L.lib().aqtx_last_error().decode()

  assert 'dtype' in err(dtype=L.I8)
  assert 'nexp' in err(nexp=8)
  assert 'nmant' in err(nmant=7)
  assert 'mode' in err(mode=5)
  assert 'noise_mod' in err(mode=L.FP_NOISE_INDEX, noise_mod=0)
  assert 'key' in err(mode=L.FP_NOISE_JAX_BITS)
  assert 'negative' in err(count=-1)
  assert L.lib().aqtx_fp_round(None, fake, fake, None, None) != 0
  p = L.FpRoundPlan()
  p.dtype, p.nexp, p.nmant = L.F32, 2, 1
  assert L.lib().aqtx_fp_round(ctypes.byref(p), None, None, None, None) == 0  # empty


@pytest.mark.gpu
@pytest.mark.parametrize('name', sorted(F.CONFIGS))
def test_every_bf16_pattern_matches_oracle(gpu, name):
  """All 2^16 bf16 inputs (infinities, container subnormals, both zeros), nearest and stochastic."""
  from aqt_amd.v2.numerics import fp_numerics
  x, t = _all_bf16(gpu)
  cfg, ocfg = _cfg(name), F.CONFIGS[name]
  got = fp_numerics.fp_round(t, cfg=cfg, key=None, stochastic_rounding=False)
  assert got.dtype == torch.bfloat16
  _eq_outside_nan(got, F.radix2_round(x, 'bf16', ocfg), x)
  for seed in (0, 42):
    key = prng.prng_key(seed)
    got = fp_numerics.fp_round(t, cfg=cfg, key=key, stochastic_rounding=True)
    _eq_outside_nan(got, F.radix2_round(x, 'bf16', ocfg, key, True), x)


@pytest.mark.gpu
@pytest.mark.parametrize('name', ['e2m1', 'e2m1_ocp', 'e3m0_ocp', 'e0m3_ocp', 'e1m0', 'e4m1_ocp', 'e5m0_ocp'])
def test_f32_slices_match_oracle(gpu, name):
  """fp_numerics_test.py:525-604's float32 slices, plus an odd length on an unaligned view."""
  from aqt_amd.v2.numerics import fp_numerics
  cfg, ocfg = _cfg(name), F.CONFIGS[name]
  vlen = 2**18
  for i in (0, 1, 100, 8191, 8192, 8193, 15900):
    bits = np.arange(vlen * i, vlen * (i + 1), dtype=np.uint32)
    x = bits.view(np.float32)
    t = torch.from_numpy(bits.view(np.int32)).to(gpu).view(torch.float32)
    _eq_outside_nan(fp_numerics.fp_round(t, cfg=cfg, key=None, stochastic_rounding=False),
                    F.radix2_round(x, 'f32', ocfg), x)
    key = prng.prng_key(12)
    _eq_outside_nan(fp_numerics.fp_round(t, cfg=cfg, key=key, stochastic_rounding=True),
                    F.radix2_round(x, 'f32', ocfg, key, True), x)
  rng = np.random.default_rng(1)
  x = (rng.standard_normal(1001) * 3).astype(np.float32)
  base = torch.from_numpy(np.concatenate([[0.0], x]).astype(np.float32)).to(gpu)
  t = base[1:]  # 4 bytes off a 16-byte boundary
  from aqt_amd import ops
  key = prng.prng_key(7)
  plan = L.FpRoundPlan()
  plan.count, plan.dtype, plan.nexp, plan.nmant, plan.has_subnormals = 1001, L.F32, ocfg.nexp, ocfg.nmant, int(ocfg.has_subnormals)
  plan.mode = L.FP_NOISE_JAX_BITS
  out = torch.empty(1002, dtype=torch.float32, device=gpu)[1:]
  k = (ctypes.c_uint32 * 2)(int(key[0]), int(key[1]))
  L.check(L.lib().aqtx_fp_round(ctypes.byref(plan), ops._ptr(t), ops._ptr(out), k, ops._stream()))
  _eq_outside_nan(out, F.radix2_round(x, 'f32', ocfg, key, True), x)


@pytest.mark.gpu
@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('nexp,nmant,sub', [(3, 0, False), (3, 0, True), (2, 1, False), (2, 1, True), (1, 2, True),
                                            (0, 3, True), (4, 1, True), (2, 3, False), (0, 5, True)])
def test_round_to_nearest_overflow_and_exact_mean(gpu, nexp, nmant, sub, dt):
  """fp_numerics_test.py:340-460 on the GPU path: interiors of the buckets round to the
  enumerated values, overflows clamp, and the 2^16 equi-spaced noise values give the input back
  as the mean (float64 accumulation)."""
  from aqt_amd.v2.numerics import fp_numerics
  cfg = fp_numerics.FpNumericsConfig(nexp=nexp, minexp=0, nmant=nmant, has_subnormals=sub, has_two_nan=False,
                                     has_naninf=False, radix=2)
  ocfg = F.FpNumericsConfig(nexp=nexp, minexp=0, nmant=nmant, has_subnormals=sub)
  centers = np.unique(F.fp_values(ocfg).astype(np.float64))
  assert centers[-1] == fp_numerics.fp_largest_representable(cfg)
  bounds = (centers[1:] + centers[:-1]) / 2
  edge = centers[-1] + (centers[-1] - bounds[-1])
  bounds = np.concatenate([[-edge], bounds, [edge]])
  lower, upper = bounds[:-1], bounds[1:]
  data = nm.cast(np.linspace(lower, upper, 129, endpoint=True, axis=0).astype(np.float32), dt)
  interior = (data > lower[None]) & (data < upper[None])
  q = fp_numerics.fp_round(U.to_dev(data, dt, gpu), cfg=cfg, key=None, stochastic_rounding=False).float().cpu().numpy()
  want = np.broadcast_to(centers[None].astype(np.float32), q.shape)
  np.testing.assert_array_equal(np.where(interior, q, 0), np.where(interior, want, 0))
  for sign in (-1.0, 1.0):
    far = nm.cast(np.linspace(sign * edge, sign * 10 * edge, 129).astype(np.float32), dt)
    far = far[np.abs(far) > edge]
    got = fp_numerics.fp_round(U.to_dev(far, dt, gpu), cfg=cfg, key=None, stochastic_rounding=False)
    assert (got.float().cpu().numpy() == sign * centers[-1]).all()
  x = nm.cast(np.linspace(centers[0], centers[-1], 129, endpoint=True).astype(np.float32), dt)
  bx = U.to_dev(x, dt, gpu)[:, None].expand(129, 2**16)
  dq = fp_numerics.fp_round(bx, cfg=cfg, key=None, stochastic_rounding=True, test_noise_axis=1)
  assert dq.dtype == U.TORCH_DT[dt]
  np.testing.assert_array_equal(dq.double().mean(dim=1).cpu().numpy(), x.astype(np.float64))
  # noise along the first axis instead
  dq0 = fp_numerics.fp_round(bx.t(), cfg=cfg, key=None, stochastic_rounding=True, test_noise_axis=0)
  assert torch.equal(dq0, dq.t())


@pytest.mark.gpu
def test_unbiased_stochastic_rounding(gpu):
  """fp_numerics_test.py:462-515 with 100000 draws per input."""
  from aqt_amd.v2.numerics import fp_numerics
  n = 100000
  for name in ('e2m1', 'e2m1_ocp', 'e3m2_ocp'):
    ocfg = F.CONFIGS[name]
    centers = np.unique(F.fp_values(ocfg).astype(np.float64))
    x = nm.cast(np.linspace(centers[0], centers[-1], 129, endpoint=True).astype(np.float32), 'bf16')
    bx = U.to_dev(x, 'bf16', gpu)[:, None].expand(129, n)
    q = fp_numerics.fp_round(bx, cfg=_cfg(name), key=prng.prng_key(42), stochastic_rounding=True).float()
    lo, hi = q.min(dim=1, keepdim=True).values, q.max(dim=1, keepdim=True).values
    assert ((q == lo) | (q == hi)).all()
    p_lo = (q == lo).double().mean(dim=1).cpu().numpy()
    lo, hi = lo[:, 0].cpu().numpy().astype(np.float64), hi[:, 0].cpu().numpy().astype(np.float64)
    size = hi - lo
    want = np.where(size == 0, 1.0, (hi - x) / np.where(size == 0, 1, size))
    assert (np.abs(p_lo - want) * np.sqrt(n) < 2.0).all()


@pytest.mark.gpu
def test_fp_numerics_class_and_quantizer(gpu):
  """FpNumerics (fp_numerics.py:618-650): bf16 out whatever the input dtype, the e1m2 / e0m3
  relation of fp_numerics_test.py:606-619 away from ties, the clipped gradient, and a
  Quantizer built on it (scale = abs-max / largest value)."""
  from aqt_amd.v2 import aqt_quantizer, calibration, utils
  from aqt_amd.v2.numerics import fp_numerics
  e1m2 = fp_numerics.FpNumerics(cfg=fp_numerics.e1m2_ocp)
  e0m3 = fp_numerics.FpNumerics(cfg=fp_numerics.e0m3_ocp)
  assert (e1m2.get_quant_bound(), e0m3.get_quant_bound(), e1m2.get_dtype()) == (1.75, 0.875, torch.bfloat16)
  ctx = utils.Context(key=None, train_step=None)
  x_np = U.rand((64, 64), 'bf16', 42)
  x_np = nm.cast(x_np / np.abs(x_np).max(), 'bf16')
  in1, in0 = nm.cast(x_np * np.float32(1.75), 'bf16'), nm.cast(x_np * np.float32(0.875), 'bf16')
  y1, _ = e1m2.vjp_fwd(U.to_dev(in1, 'bf16', gpu), ctx)
  y0, _ = e0m3.vjp_fwd(U.to_dev(in0, 'bf16', gpu), ctx)
  tie = torch.from_numpy((np.abs(in1) >= 1) & (np.abs(in0 * 8) % 1 == 0.5)).to(gpu)
  assert (y1 == y0 * 2)[~tie].all()
  np.testing.assert_array_equal(y1.float().cpu().numpy(), F.fp_vjp_fwd(in1, 'bf16', F.CONFIGS['e1m2_ocp']))
  # float32 input is cast to bf16 first
  xf = U.rand((5, 33), 'f32', 3, scale=2.0)
  yf, res = e1m2.vjp_fwd(U.to_dev(xf, 'f32', gpu), ctx)
  assert yf.dtype == torch.bfloat16
  np.testing.assert_array_equal(yf.float().cpu().numpy(), F.fp_vjp_fwd(xf, 'f32', F.CONFIGS['e1m2_ocp']))
  g = torch.ones_like(yf)
  assert e1m2.vjp_bwd(res, g)[0] is g
  clipped = fp_numerics.FpNumerics(cfg=fp_numerics.e2m1, clip_gradient=True)
  yc, resc = clipped.vjp_fwd(U.to_dev(np.float32([[0.2, 5.0, 100.0, -13.0]]), 'f32', gpu), ctx)
  assert yc.tolist() == [[1.0, 6.0, 12.0, -12.0]]
  assert clipped.vjp_bwd(resc, torch.ones_like(yc))[0].tolist() == [[1.0, 1.0, 1.0, 1.0]]  # res holds the rounded x

  q = aqt_quantizer.Quantizer(numerics=fp_numerics.FpNumerics(cfg=fp_numerics.e2m1_ocp), calib_shared_axes=None,
                              scale_stop_grad=True, calibration=calibration.AbsMaxCalibration, context=ctx)
  q.init_calibration()
  w_np = U.rand((16, 48), 'bf16', 9)
  qt, _ = q.quant(U.to_dev(w_np, 'bf16', gpu), calibration_axes=[1])
  assert qt.qvalue.dtype == torch.bfloat16 and tuple(qt.scale[0].shape) == (16, 1)
  scale = nm.cast(np.abs(w_np).max(axis=1, keepdims=True) / np.float32(6.0), 'bf16')
  np.testing.assert_array_equal(qt.scale[0].float().cpu().numpy(), scale)
  scaled = nm.cast(w_np * nm.cast(np.float32(1.0) / scale, 'bf16'), 'bf16')
  np.testing.assert_array_equal(qt.qvalue.float().cpu().numpy(), F.radix2_round(scaled, 'bf16', F.CONFIGS['e2m1_ocp']))
  vals = set(np.unique(np.abs(qt.qvalue.float().cpu().numpy())).tolist())
  assert vals <= {0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0}
  np.testing.assert_array_equal(qt.dequant().float().cpu().numpy(),
                                nm.cast(qt.qvalue.float().cpu().numpy() * scale, 'bf16'))


@pytest.mark.gpu
@pytest.mark.parametrize('dt,count', [('bf16', 16 * 50 + 13), ('bf16', 16 * 50 + 15), ('bf16', 16), ('bf16', 8),
                                      ('f32', 8 * 33 + 5), ('f32', 8 * 33 + 7), ('f32', 4), ('bf16', 1 << 20)])
def test_stochastic_rounding_paired_blocks_ragged_ends(gpu, dt, count):
  """Sizes at which the kernel that uses both words of a threefry block runs with a partly
  filled last vector in either half of the tensor."""
  from aqt_amd.v2.numerics import fp_numerics
  x = U.rand((count,), dt, count % 97, scale=2.0)
  key = prng.prng_key(count)
  for name in ('e2m1_ocp', 'e3m0'):
    got = fp_numerics.fp_round(U.to_dev(x, dt, gpu), cfg=_cfg(name), key=key, stochastic_rounding=True)
    _eq_outside_nan(got, F.radix2_round(x, dt, F.CONFIGS[name], key, True), x)


# ---- radix 4 (fp_numerics.py:661-706) -------------------------------------------------------------
@pytest.mark.gpu
def test_radix4_every_bf16_pattern(gpu):
  """Round to nearest on all 65536 patterns: equal to the oracle wherever the reference's logarithm
  is clear of a power of 4, and the mathematical floor(log4) where it is not (1.6 x = 4^n exactly)."""
  from aqt_amd.v2.numerics import fp_numerics
  x, t = _all_bf16(gpu)
  got = fp_numerics.fp_round(t, cfg=fp_numerics.RADIX4, key=None, stochastic_rounding=False)
  g = got.float().cpu().numpy()
  want = F.radix4_round(x, 'bf16')
  safe = F.radix4_log_is_safe(x) & ~np.isnan(x)
  assert safe.sum() > 65536 - 254 - 20
  np.testing.assert_array_equal(g[safe].view(np.uint32), want[safe].view(np.uint32))
  assert np.isnan(g[np.isnan(x)]).all()
  edge = ~safe & ~np.isnan(x)
  y = np.abs(np.float32(1.6) * x[edge]).astype(np.float64)
  exact = np.sign(x[edge]) * 4.0**np.floor(np.log2(y) / 2)
  exact = np.where(np.abs(exact) < 4.0**-3, 0.0, np.where(np.abs(exact) >= 64, np.sign(x[edge]) * 64, exact))
  np.testing.assert_array_equal(g[edge], exact.astype(np.float32))
  assert set(np.unique(np.abs(g[~np.isnan(g)]))) == set(np.abs(F.RADIX4_VALUES))


@pytest.mark.gpu
def test_radix4_stochastic_rounding(gpu):
  """The 2^16 equi-spaced noise values (test_noise_axis) and jax.random.bits noise against the oracle,
  and the exact mean."""
  from aqt_amd.v2.numerics import fp_numerics
  xs = nm.cast(np.array([0.0, 0.004, 0.02, 0.05, 0.3, 0.9, 1.7, 3.1, 5.0, 12.0, 17.0, 50.0, 300.0, -2.5, -40.0], np.float32), 'bf16')
  x = np.broadcast_to(xs[:, None], (xs.size, 2**16)).copy()
  t = U.to_dev(x, 'bf16', gpu)
  got = fp_numerics.fp_round(t, cfg=fp_numerics.RADIX4, key=None, stochastic_rounding=True, test_noise_axis=1)
  g = got.float().cpu().numpy()
  want = F.radix4_round(x, 'bf16', stochastic_rounding=True, test_noise_axis=1)
  safe = F.radix4_log_is_safe(x, stochastic_rounding=True, test_noise_axis=1)
  assert safe.mean() > 0.99
  np.testing.assert_array_equal(g[safe], want[safe])
  inside = (np.abs(xs) >= 4.0**-3) & (np.abs(xs) < 64)
  width = 3 * 4.0**np.floor(np.log2(np.abs(xs[inside].astype(np.float64))) / 2)
  assert np.all(np.abs(g[inside].astype(np.float64).mean(axis=1) - xs[inside]) <= 2.0**-15 * width)
  key = np.array([7, 11], np.uint32)
  rng = np.random.default_rng(5)
  x = nm.cast((rng.standard_normal((257, 1000)) * np.exp(rng.uniform(-5, 5, (257, 1000)))).astype(np.float32), 'bf16')
  got = fp_numerics.fp_round(U.to_dev(x, 'bf16', gpu), cfg=fp_numerics.RADIX4, key=key, stochastic_rounding=True)
  want = F.radix4_round(x, 'bf16', key=key, stochastic_rounding=True)
  safe = F.radix4_log_is_safe(x, key=key, stochastic_rounding=True)
  assert safe.mean() > 0.99
  np.testing.assert_array_equal(got.float().cpu().numpy()[safe], want[safe])


@pytest.mark.gpu
def test_radix4_takes_bf16_only(gpu):
  from aqt_amd.v2.numerics import fp_numerics
  with pytest.raises(AssertionError, match='Unsupported dtype'):
    fp_numerics.fp_round(torch.zeros(8, device=gpu), cfg=fp_numerics.RADIX4, key=None, stochastic_rounding=False)
  p = L.FpRoundPlan()
  p.count, p.dtype, p.radix, p.mode = 16, L.F32, 4, L.FP_NEAREST
  fake = ctypes.c_void_p(0x1000)
  assert L.lib().aqtx_fp_round(ctypes.byref(p), fake, fake, None, None) != 0
  assert 'bf16' in L.lib().aqtx_last_error().decode()

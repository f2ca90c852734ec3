"""Pins of the oracle's dot_general orchestration (known answers and exact equivalences)."""
import numpy as np
import pytest

from oracle import aqt_ref as R
from oracle import numerics as nm
from oracle import prng

MATMUL = (((1,), (0,)), ((), ()))


def test_readme_int8_matmul_golden():
  """README.md:385-388: the worked int8 example (scale = 127/absmax, clip +-127)."""
  np.random.seed(0)
  a = np.random.normal(size=(3, 4)).astype(np.float32)
  np.random.seed(0)
  w = np.random.normal(size=(4, 5)).astype(np.float32)
  a_s = np.float32(127) / np.max(np.abs(a), axis=1, keepdims=True)
  w_s = np.float32(127) / np.max(np.abs(w), axis=0, keepdims=True)
  qa = np.clip(np.rint(a * a_s), -127, 127).astype(np.int8)
  qw = np.clip(np.rint(w * w_s), -127, 127).astype(np.int8)
  acc = R.lax_dot_general(qa, qw, MATMUL, np.int32)
  got = acc.astype(np.float32) / (a_s * w_s)
  want = np.array([[3.5998788, 5.8562713, 1.9385538, 4.7426414, 1.9792401],
                   [4.321886, 0.99681264, 2.737299, 4.3591022, 3.6352503],
                   [-0.07714217, 2.7415617, -0.35343346, 0.20568734, -1.1974115]], np.float32)
  np.testing.assert_allclose(got, want, rtol=2e-6)
  fl = np.array([[3.6095254, 5.8575077, 1.9510972, 4.732388, 1.9792626],
                 [4.335892, 0.9743651, 2.7298734, 4.3540883, 3.637487],
                 [-0.07735002, 2.7310796, -0.3519049, 0.19912864, -1.2023292]], np.float32)
  np.testing.assert_allclose(a @ w, fl, rtol=2e-6)


@pytest.mark.parametrize('shard_count,expected', [(2, 1281280.0), (1, 1280000.0)])
def test_local_aqt_known_answer(shard_count, expected):
  """aqt_dot_general_test.py:1079-1113."""
  cfg = R.fully_quantized(8, 8, use_stochastic_rounding=False)
  cfg.drhs.local_aqt_shard_count = shard_count
  for q in (cfg.fwd.lhs, cfg.fwd.rhs, cfg.drhs.lhs, cfg.drhs.rhs):
    q.preserve_max_val = True
  lhs = np.array([1270.0, 10.0, 1270000.0, 10000.0], np.float32)
  rhs = np.array([1.0], np.float32)
  dn = (((), ()), ((), ()))
  f = R.dg_fwd(lhs, rhs, 'f32', dn, cfg)
  _, drhs = R.dg_bwd(np.ones_like(f.out), 'f32', dn, f, cfg)
  assert drhs.shape == (1,) and drhs[0] == expected


def test_per_tensor_scale_is_one():
  """aqt_dot_general_test.py:1115-1144: bits=4, max |x| = 7.5 -> scale exactly 1."""
  x = np.array([[1, 2, 3, 4], [5, 6, 7, 7.5], [3, 5, 1, -1]], np.float32)
  qt = R.quantize(x, 'f32', R.QuantizerCfg(bits=4, calib_shared_axes='per_tensor'), None)
  assert qt.scale[0].shape == (1, 1) and qt.scale[0][0, 0] == 1.0


def test_per_subchannel_shapes():
  """aqt_dot_general_test.py:1146-1167 (tiled shape (4,4,2,2), scale (1,4,2,1))."""
  x = np.arange(64, dtype=np.float32).reshape(4, 4, 2, 2)
  qt = R.quantize(x, 'f32', R.QuantizerCfg(bits=4, scale_dtype='f32'), [0, 3])
  assert qt.qvalue.shape == (4, 4, 2, 2) and qt.scale[0].shape == (1, 4, 2, 1)
  assert R.dequant(qt).shape == (4, 4, 2, 2)


def _rand(shape, seed, scale=1.0):
  return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(np.float32)


@pytest.mark.parametrize('dn,ls,rs', [
    (MATMUL, (5, 7), (7, 3)),
    ((((2,), (1,)), ((0,), (0,))), (2, 5, 7), (2, 7, 3)),
    ((((2,), (0,)), ((), ())), (2, 3, 8), (8, 4, 5)),
    ((((0,), (0,)), ((), ())), (7, 5), (7, 3)),
])
def test_unquantized_equals_float_dot_and_its_gradients(dn, ls, rs):
  """aqt_dot_general_test.py:705-715: no numerics -> lax.dot_general and autodiff gradients."""
  cfg = R.dot_general_make(None, None, None)
  lhs, rhs = _rand(ls, 1), _rand(rs, 2)
  f = R.dg_fwd(lhs, rhs, 'f32', dn, cfg)
  (lca, rca), (lba, rba) = dn
  want = R.lax_dot_general(lhs, rhs, dn, np.float32)
  np.testing.assert_allclose(f.out, want, rtol=1e-5, atol=1e-5)
  g = _rand(f.out.shape, 3)
  dl, dr = R.dg_bwd(g, 'f32', dn, f, cfg)
  # numerical gradient of sum(out * g) by central differences in float64
  def loss(l, r):
    return float(np.sum(R.lax_dot_general(l, r, dn, np.float64) * g))
  for arr, grad, which in ((lhs, dl, 0), (rhs, dr, 1)):
    assert grad.shape == arr.shape
    idx = tuple(np.random.default_rng(4).integers(0, s) for s in arr.shape)
    pert = arr.astype(np.float64).copy()
    pert[idx] += 1e-3
    hi = loss(pert, rhs.astype(np.float64)) if which == 0 else loss(lhs.astype(np.float64), pert)
    pert[idx] -= 2e-3
    lo = loss(pert, rhs.astype(np.float64)) if which == 0 else loss(lhs.astype(np.float64), pert)
    np.testing.assert_allclose(grad[idx], (hi - lo) / 2e-3, rtol=1e-3, atol=1e-3)


def _po2(cfg):
  for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
    raw.lhs.po2_scale = raw.rhs.po2_scale = True


@pytest.mark.parametrize('seed', range(4))
def test_int_path_equals_fake_quant_with_po2_scales(seed):
  """aqt_dot_general_test.py:615-715: with power-of-two scales the int8/int32 path
  (DequantMode.OUTPUT) and the fake-quant path (THIS_INPUT, float dot) agree exactly."""
  lhs, rhs, g = _rand((10, 20), seed), _rand((20, 6), seed + 10), _rand((10, 6), seed + 20)
  a = R.fully_quantized(8, 8, use_stochastic_rounding=False)
  _po2(a)
  b = R.fully_quantized(8, 8, use_stochastic_rounding=False)
  _po2(b)
  for raw in (b.fwd, b.dlhs, b.drhs):
    raw.lhs_dequant_mode = raw.rhs_dequant_mode = 'this_input'
    raw.lhs.keep_float = raw.rhs.keep_float = True
    raw.acc = None
  fa = R.dg_fwd(lhs, rhs, 'f32', MATMUL, a)
  fb = R.dg_fwd(lhs, rhs, 'f32', MATMUL, b)
  np.testing.assert_array_equal(fa.out, fb.out)
  # use_fwd_quant needs integer residuals; compare the bwd with it disabled on both
  a.dlhs.rhs_use_fwd_quant = a.drhs.rhs_use_fwd_quant = False
  b.dlhs.rhs_use_fwd_quant = b.drhs.rhs_use_fwd_quant = False
  for x, y in zip(R.dg_bwd(g, 'f32', MATMUL, fa, a), R.dg_bwd(g, 'f32', MATMUL, fb, b)):
    np.testing.assert_array_equal(x, y)


def test_use_fwd_quant_is_irrelevant_without_rounding():
  """aqt_dot_general_test.py (use_fwd_quant True == False when rounding is disabled)."""
  lhs, rhs, g = _rand((6, 8), 1), _rand((8, 4), 2), _rand((6, 4), 3)
  outs = []
  for ufq in (True, False):
    cfg = R.fully_quantized(8, 8, use_fwd_quant=ufq, use_stochastic_rounding=False)
    _po2(cfg)
    for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
      for q in (raw.lhs, raw.rhs):
        q.round = False
        q.keep_float = True
      raw.acc = None
    f = R.dg_fwd(lhs, rhs, 'f32', MATMUL, cfg)
    outs.append((f.out,) + R.dg_bwd(g, 'f32', MATMUL, f, cfg))
  for x, y in zip(*outs):
    np.testing.assert_allclose(x, y, rtol=1e-6, atol=1e-7)


def test_tiled_equals_untiled_on_ones():
  """tiled_dot_general_test.py:191-224: all-ones operands, any tile size."""
  lhs, rhs = np.ones((6, 32), np.float32), np.ones((32, 5), np.float32)
  cfg = R.dot_general_make(None, None, None)  # the reference injects plain lax.dot_general
  for ts in (4, 8, 16, 32):
    got, _ = R.tiled_dg_fwd(lhs, rhs, 'f32', ts, cfg)
    np.testing.assert_array_equal(got, lhs @ rhs)
  # int8 per-tile scales: every 1.0 becomes 127 * (1/127.5), so the result is 32 * (127/127.5)**2
  q = R.dot_general_make(8, 8, None)
  got, res = R.tiled_dg_fwd(lhs, rhs, 'f32', 8, q)
  assert res.lhs_res.qx.scale[0].shape == (6, 4, 1) and res.rhs_res.qx.scale[0].shape == (4, 1, 5)
  np.testing.assert_allclose(got, 32.0 * (127.0 / 127.5) ** 2, rtol=1e-6)


def test_scale_transposes_round_trip_shapes():
  """transpose_test.py:40-178 shapes: keepdims scales re-laid out for the output."""
  dn = (((2,), (1,)), ((0,), (0,)))
  ls, rs = (3, 4, 5), (3, 5, 6)
  sl = np.arange(12, dtype=np.float32).reshape(3, 4, 1)
  sr = np.arange(18, dtype=np.float32).reshape(3, 1, 6)
  assert R.lhs_scale_transpose_to_output(sl, dn, ls, rs).shape == (3, 4, 1)
  assert R.rhs_scale_transpose_to_output(sr, dn, ls, rs).shape == (3, 1, 6)
  assert R.rhs_scale_transpose_for_lhs_input(sr.reshape(3, 1, 6), (((2,), (2,)), ((0,), (0,))), (3, 4, 6)).shape == (3, 1, 6)


def test_sr_noise_depends_on_key_and_is_centered():
  x = nm.to_bf16(_rand((64, 256), 0))
  outs = []
  for seed in (1, 2):
    q = R.QuantizerCfg(bits=8, noise='jax.uniform', key=prng.prng_key(seed))
    outs.append(R.quantize(x, 'bf16', q, [1]).qvalue.astype(np.int32))
  rtn = R.quantize(x, 'bf16', R.QuantizerCfg(bits=8), [1]).qvalue.astype(np.int32)
  assert (outs[0] != outs[1]).any()
  assert np.abs(outs[0] - rtn).max() <= 1
  assert abs((outs[0] - rtn).mean()) < 0.02


def _po2_data(shape, seed):
  rng = np.random.default_rng(seed)
  return np.exp2(np.floor(rng.uniform(-3.0, 3.0, shape) + 3.0)).astype(np.float32)


def _mode_cfg(lmode, rmode, lcal='ca', rcal='ca', disable_rounding=False):
  """The reference test helper `_modify_dg` (aqt_dot_general_test.py:229-309) on the oracle's
  config: po2 scales everywhere, the modes on all three contractions, sides in THIS_INPUT
  mode held in float, no use_fwd_quant."""
  cfg = R.fully_quantized(8, 8, use_fwd_quant=False, use_stochastic_rounding=False)
  _po2(cfg)
  for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
    raw.lhs_dequant_mode, raw.rhs_dequant_mode = lmode, rmode
    raw.lhs_calibration_mode, raw.rhs_calibration_mode = lcal, rcal
    for q, mode in ((raw.lhs, lmode), (raw.rhs, rmode)):
      if mode == 'this_input' or disable_rounding:
        q.keep_float = True
      if disable_rounding:
        q.round = False
    if 'this_input' in (lmode, rmode) or disable_rounding:
      raw.acc = None
  return cfg


MODE_CASES = [
    ('CA', dict(lmode='output', rmode='output', disable_rounding=True)),
    ('CA fake', dict(lmode='this_input', rmode='this_input', disable_rounding=True)),
    ('RA L', dict(lmode='other_input', rmode='this_input', lcal='ra', rcal='ra')),
    ('RA R', dict(lmode='this_input', rmode='other_input', lcal='ra', rcal='ra')),
    ('RA fake', dict(lmode='this_input', rmode='this_input', lcal='ra', rcal='ra')),
]


def test_equality_between_different_calibration_axes():
  """aqt_dot_general_test.py:972-1048: on power-of-two data (no quantization loss) calibrating
  over the contraction axes with output dequantisation, over the remaining axes with the
  scale moved to the other operand, and the fake-quant forms all give the float result;
  a wrong scale transpose or calibration axis breaks it."""
  lhs, rhs, g = _po2_data((10, 20), 1), _po2_data((20, 30), 2), _po2_data((10, 30), 3)
  want = (lhs @ rhs, g @ rhs.T, lhs.T @ g)
  for name, kw in MODE_CASES:
    cfg = _mode_cfg(**kw)
    f = R.dg_fwd(lhs, rhs, 'f32', MATMUL, cfg)
    got = (f.out,) + tuple(R.dg_bwd(g, 'f32', MATMUL, f, cfg))
    for x, y in zip(got, want):
      np.testing.assert_array_equal(x, y, err_msg=name)


def test_abs_mean_calibration_closed_forms():
  """calibration.py:160-193: mean over the non-zero entries, p-norm form, clipping scale."""
  x = np.array([[1.0, -2.0, 0.0, 3.0], [0.0, 0.0, 0.0, 0.0]], np.float32)
  q = R.QuantizerCfg(bits=8, abs_mean_p=1.0, clipping_scale=1.0)
  s, sdt = R.calibrate(x, 'f32', [1], q)
  np.testing.assert_array_equal(s, np.array([[2.0], [1.0]], np.float32) / np.float32(127.5))
  q = R.QuantizerCfg(bits=8, abs_mean_p=2.0, clipping_scale=3.0)
  s, _ = R.calibrate(np.array([[3.0, 4.0, 0.0]], np.float32), 'f32', [1], q)
  np.testing.assert_allclose(s, [[3.0 * np.sqrt(12.5) / 127.5]], rtol=3e-7)


def test_snr_calibration_picks_the_brute_force_best_clip():
  """calibration.py:196-399: with a single candidate 1.0 it is abs-max calibration; with an
  outlier in a 4-bit row the candidate minimising the float64 squared error wins."""
  rng = np.random.default_rng(0)
  x = rng.standard_normal((6, 1024)).astype(np.float32)
  x[::2, 7] = 12.0  # outliers in every other row
  only_one = R.QuantizerCfg(bits=4, auto_clip_search=[1.0])
  s1, _ = R.calibrate(x, 'f32', [1], only_one)
  s0, _ = R.calibrate(x, 'f32', [1], R.QuantizerCfg(bits=4))
  np.testing.assert_array_equal(s1, s0)
  cands = [1.0, 0.5, 0.25, 0.1, 0.05]
  s, _ = R.calibrate(x, 'f32', [1], R.QuantizerCfg(bits=4, auto_clip_search=cands))
  amax = np.abs(x).max(axis=1, keepdims=True).astype(np.float64)
  errs = []
  for c in cands:
    sc = amax * c / 7.5
    deq = np.clip(np.rint(x / sc), -7, 7) * sc
    errs.append(((x - deq) ** 2).sum(axis=1))
  best = np.array(cands)[np.argmin(np.stack(errs), axis=0)]
  np.testing.assert_allclose(s[:, 0], (amax[:, 0] * best / 7.5), rtol=1e-6)
  assert (best[::2] < best[1::2]).all()  # rows with the outlier clip harder

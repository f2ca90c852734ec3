"""GPU parity of the step-by-step DotGeneralRaw path (configurations without a fused kernel)
against the numpy oracle: fake quantization, scaling of the other operand, calibration over
the remaining axes, one-sided quantization, po2 / clipped / constant calibrations, numerics
without rounding or clipping, plugin hooks.

Quantized values and scales are compared bit for bit.  Outputs of *float* contractions
(fake quantization, one-sided quantization) go through the library GEMM, whose summation
order differs from numpy's: those are compared to rtol 1e-4 (f32) / 2e-2 (bf16) with an
absolute floor scaled to the output magnitude.
"""
import copy
import functools

import numpy as np
import pytest
import torch

from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import calibration
from aqt_amd.v2 import config
from aqt_amd.v2 import utils
from oracle import aqt_ref as R
from oracle import numerics as nm
from oracle import prng
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

MATMUL = (((1,), (0,)), ((), ()))
BATCHED = (((2,), (1,)), ((0,), (0,)))
MODE = {'output': aqt.DequantMode.OUTPUT, 'this_input': aqt.DequantMode.THIS_INPUT,
        'other_input': aqt.DequantMode.OTHER_INPUT}
CAL = {'ca': aqt.CalibrationMode.CONTRACTING_AXIS, 'ra': aqt.CalibrationMode.REMAINING_AXIS}


def _np(t):
  return t.detach().float().cpu().numpy()


def _close(got, want, dt):
  rtol = 1e-4 if dt == 'f32' else 2e-2
  atol = rtol * float(np.abs(want).max() + 1e-30)
  np.testing.assert_allclose(got, want, rtol=rtol, atol=atol)


@pytest.fixture
def lowered_only(monkeypatch):
  """The call has to stay on the lowered kernels: the step-by-step path raises."""
  def no_step_by_step(self, *a, **k):
    raise AssertionError('the step-by-step path was taken')
  monkeypatch.setattr(aqt.DotGeneralRaw, '_unfused_call', no_step_by_step)


def _raw_pair(lhs_bits=8, rhs_bits=8, *, lmode='output', rmode='output', lcal='ca', rcal='ca',
              keep_float=False, acc='auto', calib=None):
  """A product DotGeneralRaw and the oracle RawCfg with the same settings."""
  raw = aqt.dot_general_raw_make(lhs_bits, rhs_bits, initialize_calibration=False)
  raw.lhs.dequant_mode, raw.rhs.dequant_mode = MODE[lmode], MODE[rmode]
  raw.lhs.calibration_mode, raw.rhs.calibration_mode = CAL[lcal], CAL[rcal]
  oraw = R.RawCfg(R.QuantizerCfg(bits=lhs_bits), R.QuantizerCfg(bits=rhs_bits),
                  lhs_dequant_mode=lmode, rhs_dequant_mode=rmode,
                  lhs_calibration_mode=lcal, rhs_calibration_mode=rcal)
  if keep_float:
    for q, oq, bits in ((raw.dg_quantizer.lhs, oraw.lhs, lhs_bits), (raw.dg_quantizer.rhs, oraw.rhs, rhs_bits)):
      if bits is not None:
        q.numerics.dtype = None
        oq.keep_float = True
  if acc != 'auto':
    raw.dg_accumulator_dtype = acc
    oraw.acc = acc
  if calib:
    _set_calibration(raw, oraw, **calib)
  raw.dg_quantizer.init_calibration()
  return raw, oraw


def _run_raw(raw, oraw, lhs, rhs, dt, dn, gpu):
  out, res = raw(U.to_dev(lhs, dt, gpu), U.to_dev(rhs, dt, gpu), None, None, dn)
  want, wdt, (lres, rres), _ = R.dg_raw(lhs, dt, rhs, dt, dn, oraw)
  assert out.dtype == U.TORCH_DT[wdt]
  return out, res, want, lres, rres


def _assert_residuals_equal(res, lres, rres):
  for got, want in ((res.lhs.mt.qx, lres.qx), (res.rhs.mt.qx, rres.qx)):
    np.testing.assert_array_equal(_np(got.qvalue), np.asarray(want.qvalue, np.float32))
    assert len(got.scale) == len(want.scale)
    for gs, ws in zip(got.scale, want.scale):
      assert tuple(gs.shape) == ws.shape
      np.testing.assert_array_equal(_np(gs), ws)


@pytest.mark.parametrize('dt', ['f32', 'bf16'])
@pytest.mark.parametrize('name,kw', [
    ('fake_ca', dict(lmode='this_input', rmode='this_input')),
    ('fake_ca_float_held', dict(lmode='this_input', rmode='this_input', keep_float=True)),
    ('ra_lhs_scales_rhs', dict(lmode='other_input', rmode='this_input', lcal='ra', rcal='ra')),
    ('ra_rhs_scales_lhs', dict(lmode='this_input', rmode='other_input', lcal='ra', rcal='ra')),
    ('fake_ra', dict(lmode='this_input', rmode='this_input', lcal='ra', rcal='ra')),
    ('fake_lhs_only', dict(lmode='this_input', rmode='output')),
])
@pytest.mark.parametrize('dn,ls,rs', [(MATMUL, (48, 96), (96, 40)), (BATCHED, (3, 20, 64), (3, 64, 24))])
def test_dequant_and_calibration_modes(gpu, name, kw, dt, dn, ls, rs, lowered_only):
  """aqt_dot_general_test.py:761-903 walks these combinations; here each one is checked
  against the oracle.  Float-held operands make the contraction a float one.  All of them run on the
  lowered path: quantize kernels, one scale-and-cast pass per operand, the library's float product."""
  raw, oraw = _raw_pair(acc=None, **kw)
  lhs, rhs = U.rand(ls, dt, 1, outliers=True), U.rand(rs, dt, 2, 0.05)
  out, res, want, lres, rres = _run_raw(raw, oraw, lhs, rhs, dt, dn, gpu)
  _assert_residuals_equal(res, lres, rres)
  _close(_np(out), want, dt)


@pytest.mark.parametrize('dt', ['f32', 'bf16'])
@pytest.mark.parametrize('lhs_bits,rhs_bits', [(None, 8), (8, None), (None, 4)])
def test_one_sided_quantization(gpu, lhs_bits, rhs_bits, dt, lowered_only):
  """Weight-only / activation-only: the int8 side is promoted to the float dtype for the
  contraction, its scale multiplies the output."""
  raw, oraw = _raw_pair(lhs_bits, rhs_bits)
  assert raw.dg_accumulator_dtype is None
  lhs, rhs = U.rand((40, 128), dt, 3, outliers=True), U.rand((128, 56), dt, 4, 0.05)
  out, res, want, lres, rres = _run_raw(raw, oraw, lhs, rhs, dt, MATMUL, gpu)
  _assert_residuals_equal(res, lres, rres)
  _close(_np(out), want, dt)


def test_weight_only_serving_keeps_the_promoted_weight(gpu, monkeypatch):
  """With WEIGHT_ONLY_FLOAT_COPY on, a frozen int8 weight next to a float lhs of more than 64 rows (fewer go to
  the weight-only kernel) is promoted to the float dtype once, not on every call; a change of the weight in place
  is noticed (version counter); while gradients are recorded no copy is kept."""
  from aqt_amd.v2 import aqt_dot_general as adg
  monkeypatch.setattr(adg, 'WEIGHT_ONLY_FLOAT_COPY', True)
  dt = 'bf16'
  cfg = config.set_context(aqt.dot_general_make(None, 8), None, None)
  x1, x2 = U.to_dev(U.rand((72, 1024), dt, 1), dt, gpu), U.to_dev(U.rand((72, 1024), dt, 2), dt, gpu)
  w = U.to_dev(U.rand((1024, 1024), dt, 3, 0.05), dt, gpu)
  _, (_, wq) = cfg.dg_core(x1, w, None, None, MATMUL)
  assert wq.qvalue.dtype == torch.int8

  def serve(x):
    with torch.no_grad():
      return cfg.dg_core(x, torch.zeros_like(w), None, wq, MATMUL)[0]

  adg._PROMOTED_RHS.clear()
  cfg.dg_core(x1, torch.zeros_like(w), None, wq, MATMUL)
  assert not adg._PROMOTED_RHS  # gradients were being recorded
  a1, a2 = serve(x1), serve(x2)
  assert list(adg._PROMOTED_RHS) == [id(wq.qvalue)]
  kept = adg._PROMOTED_RHS[id(wq.qvalue)][1]
  b1 = serve(x1)
  assert adg._PROMOTED_RHS[id(wq.qvalue)][1] is kept and torch.equal(a1, b1) and not torch.equal(a1, a2)
  want = (x1.float() @ (wq.qvalue.float() * wq.scale[0].float())).to(torch.bfloat16)
  np.testing.assert_allclose(a1.float().cpu().numpy(), want.float().cpu().numpy(), rtol=2e-2, atol=2e-2)
  wq.qvalue.neg_()   # in place: the kept copy is stale
  c1 = serve(x1)
  assert adg._PROMOTED_RHS[id(wq.qvalue)][1] is not kept
  assert torch.equal(c1, -a1)


def _set_calibration(raw, oraw, **kw):
  for q, oq in ((raw.dg_quantizer.lhs, oraw.lhs), (raw.dg_quantizer.rhs, oraw.rhs)):
    if 'const_bound' in kw:
      q.calibration = functools.partial(calibration.ConstantCalibration, bound=kw['const_bound'])
      oq.const_bound = kw['const_bound']
    else:
      q.calibration = functools.partial(q.calibration, **kw)
      for k, v in kw.items():
        setattr(oq, k, v)


@pytest.mark.parametrize('dt', ['f32', 'bf16'])
@pytest.mark.parametrize('kw', [dict(po2_scale=True), dict(clipping_scale=0.3),
                                dict(po2_scale=True, clipping_scale=0.5), dict(const_bound=2.0)])
def test_calibration_variants_int8_path(gpu, kw, dt):
  """po2 / clipped abs-max and constant bounds: the scales come from elementwise steps after
  the abs-max kernel, the contraction is the int8 MFMA one: everything is bit-exact."""
  raw, oraw = _raw_pair(calib=kw)
  lhs, rhs = U.rand((64, 160), dt, 5, outliers=True), U.rand((160, 72), dt, 6, 0.05)
  out, res, want, lres, rres = _run_raw(raw, oraw, lhs, rhs, dt, MATMUL, gpu)
  _assert_residuals_equal(res, lres, rres)
  np.testing.assert_array_equal(_np(out), want)


@pytest.mark.parametrize('dt', ['f32', 'bf16'])
@pytest.mark.parametrize('kw', [dict(round=False), dict(clip=False, round=False),
                                dict(preserve_zero=False), dict(preserve_max_val=True)])
def test_numerics_variants_float_held(gpu, kw, dt, lowered_only):
  """IntSymmetric settings whose results are not integers (int_numerics.py:81-111), values held in
  the input dtype, fake-quant dequantisation."""
  raw, oraw = _raw_pair(lmode='this_input', rmode='this_input', keep_float=True, acc=None)
  for q, oq in ((raw.dg_quantizer.lhs, oraw.lhs), (raw.dg_quantizer.rhs, oraw.rhs)):
    for k, v in kw.items():
      setattr(q.numerics, k, v)
      setattr(oq, k, v)
  lhs, rhs = U.rand((32, 64), dt, 7), U.rand((64, 48), dt, 8, 0.05)
  out, res, want, lres, rres = _run_raw(raw, oraw, lhs, rhs, dt, MATMUL, gpu)
  _assert_residuals_equal(res, lres, rres)
  _close(_np(out), want, dt)


def test_int_path_equals_fake_quant_with_po2_scales(gpu):
  """aqt_dot_general_test.py:557-715: with power-of-two scales the int8 contraction with
  output dequantisation and the fake-quant float contraction are the same numbers."""
  dt = 'f32'
  lhs, rhs = U.rand((32, 64), dt, 9, outliers=True), U.rand((64, 48), dt, 10, 0.05)
  outs = []
  for mode, acc in (('output', 'auto'), ('this_input', None)):
    raw, oraw = _raw_pair(lmode=mode, rmode=mode, acc=acc, calib=dict(po2_scale=True))
    out, _ = raw(U.to_dev(lhs, dt, gpu), U.to_dev(rhs, dt, gpu), None, None, MATMUL)
    outs.append(_np(out))
  # int8 products summed in f32 are exact below 2^24; po2 scales only shift exponents
  np.testing.assert_array_equal(outs[0], outs[1])


def test_fake_quant_fwd_and_bwd(gpu):
  """DotGeneral with a fake-quant forward: the backward contractions still take the fused
  kernels; use_fwd_quant is off as the forward qvalues are not what the contraction saw."""
  dt = 'bf16'
  lhs, rhs, g = U.rand((64, 128), dt, 1), U.rand((128, 32), dt, 2, 0.02), U.rand((64, 32), dt, 3, 1e-3)
  cfg = config.fully_quantized(use_fwd_quant=False, use_stochastic_rounding=True)
  config.set_fwd_dequant_mode(cfg, lhs_dequant_mode=aqt.DequantMode.THIS_INPUT,
                              rhs_dequant_mode=aqt.DequantMode.THIS_INPUT)
  cfg.fwd.dg_accumulator_dtype = None
  ocfg = R.fully_quantized(use_fwd_quant=False, use_stochastic_rounding=True)
  ocfg.fwd.lhs_dequant_mode = ocfg.fwd.rhs_dequant_mode = 'this_input'
  ocfg.fwd.acc = None
  key = prng.prng_key(11)
  cfg = config.set_context(cfg, key, None)
  ocfg = R.set_context(ocfg, key)
  L = U.to_dev(lhs, dt, gpu).requires_grad_(True)
  Rr = U.to_dev(rhs, dt, gpu).requires_grad_(True)
  out = cfg(L, Rr, MATMUL)
  out.backward(U.to_dev(g, dt, gpu))
  f = R.dg_fwd(lhs, rhs, dt, MATMUL, ocfg)
  dl, dr = R.dg_bwd(g, dt, MATMUL, f, ocfg)
  _close(_np(out), f.out, dt)
  np.testing.assert_array_equal(_np(L.grad), dl)
  np.testing.assert_array_equal(_np(Rr.grad), dr)


def test_custom_dot_general_hook(gpu):
  """DotGeneralRaw.dot_general is a plugin point (aqt_dot_general.py:749): a user function
  receives the quantized operands and the accumulator dtype."""
  seen = []

  def hook(lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None):
    seen.append((lhs.dtype, rhs.dtype, preferred_element_type))
    return aqt.lax_dot_general(lhs, rhs, dimension_numbers, precision, preferred_element_type)

  dt = 'bf16'
  raw, oraw = _raw_pair()
  raw.dot_general = hook
  lhs, rhs = U.rand((48, 96), dt, 1, outliers=True), U.rand((96, 40), dt, 2, 0.05)
  out, res, want, lres, rres = _run_raw(raw, oraw, lhs, rhs, dt, MATMUL, gpu)
  assert seen == [(torch.int8, torch.int8, torch.int32)]
  _assert_residuals_equal(res, lres, rres)
  np.testing.assert_array_equal(_np(out), want)


def test_custom_dg_quantizer(gpu):
  """A DotGeneralQuantizer of the user's own (aqt_dot_general.py:331-422): here one that
  halves every calibrated scale's bound by delegating and editing the scale."""

  class Halving(aqt.DefaultDotGeneralQuantizer):
    calls = 0

    def calibrate(self, lhs, rhs, dimension_numbers, lhs_mode, rhs_mode):
      Halving.calls += 1
      (lhs, lqt), (rhs, rqt) = super().calibrate(lhs, rhs, dimension_numbers, lhs_mode, rhs_mode)
      lqt.scale = [s * 0.5 for s in lqt.scale]
      return (lhs, lqt), (rhs, rqt)

  dt = 'f32'
  raw, oraw = _raw_pair()
  d = raw.dg_quantizer
  raw.dg_quantizer = Halving(lhs=d.lhs, rhs=d.rhs, lhs_mid=d.lhs_mid, rhs_mid=d.rhs_mid)
  oraw.lhs.clipping_scale = 0.5  # the same scale: abs_max * 0.5 / 127 (exact halving in f32)
  lhs, rhs = U.rand((48, 96), dt, 1), U.rand((96, 40), dt, 2, 0.05)
  out, res, want, lres, rres = _run_raw(raw, oraw, lhs, rhs, dt, MATMUL, gpu)
  assert Halving.calls == 1
  # abs_max * 0.5 / 127 and (abs_max / 127) * 0.5 round alike except at subnormals
  _assert_residuals_equal(res, lres, rres)
  np.testing.assert_array_equal(_np(out), want)


@pytest.mark.parametrize('dt', ['f32', 'bf16'])
def test_clip_gradient(gpu, dt, monkeypatch):
  """IntSymmetric.clip_gradient with a clipping calibration (int_numerics.py:113-125): the
  gradient is the unclipped one times the mask of scaled inputs inside the clip bound, the scaled
  input being x * (1 / scale) in x's dtype (aqt_tensor.py:151-155).  The call stays on the fused
  quantize and contraction kernels; the mask is made in the backward pass."""
  lhs, rhs, g = U.rand((32, 64), dt, 1, outliers=True), U.rand((64, 16), dt, 2), U.rand((32, 16), dt, 3)
  cfg = config.fully_quantized(use_fwd_quant=False, use_stochastic_rounding=False)
  config.set_absmax_calib_scale(cfg, 0.25)
  assert cfg.fwd.dg_quantizer.lhs.numerics.clip_gradient and cfg.fwd.dg_quantizer.rhs.numerics.clip_gradient
  cfg = config.set_context(cfg, None, None)

  def no_step_by_step(self, *a, **k):
    raise AssertionError('the step-by-step path was taken')
  monkeypatch.setattr(aqt.DotGeneralRaw, '_unfused_call', no_step_by_step)
  Lh = U.to_dev(lhs, dt, gpu).requires_grad_(True)
  Rh = U.to_dev(rhs, dt, gpu).requires_grad_(True)
  out, (lqt, rqt) = cfg.dg_core(Lh, Rh, None, None, MATMUL)
  out.backward(U.to_dev(g, dt, gpu))
  cfg2 = copy.deepcopy(cfg)
  for q in (cfg2.fwd.dg_quantizer.lhs, cfg2.fwd.dg_quantizer.rhs):
    q.numerics.clip_gradient = False
  L2 = U.to_dev(lhs, dt, gpu).requires_grad_(True)
  R2 = U.to_dev(rhs, dt, gpu).requires_grad_(True)
  out2, _ = cfg2.dg_core(L2, R2, None, None, MATMUL)
  out2.backward(U.to_dev(g, dt, gpu))
  np.testing.assert_array_equal(_np(out), _np(out2))
  for x, qt, got, plain in ((lhs, lqt, Lh.grad, L2.grad), (rhs, rqt, Rh.grad, R2.grad)):
    inv = nm.cast(np.float32(1.0) / _np(qt.scale[0]), dt)
    scaled = nm.cast(nm.cast(x, dt) * inv, dt)
    inside = np.abs(scaled) <= 127.0
    assert (~inside).any() and inside.any()
    np.testing.assert_array_equal(_np(got), _np(plain) * inside)


def test_mid_quantization_known_answer(gpu, lowered_only):
  """The reference's own vectors (aqt_dot_general_test.py:1169-1208): binary quantization
  rounds 1, 2, 4 (and 1, 4, 16) to one magnitude; with mid scales of alpha 0.5 and
  power-of-two scales it becomes lossless."""

  def make_binary_dg(use_mid):
    mid_alpha = 0.5 if use_mid else config.SKIP
    dg = config.config_v4(fwd_bits=1, dlhs_bits=1, drhs_bits=1, fwd_mid_alpha_both=mid_alpha,
                          dlhs_mid_alpha_both=mid_alpha, drhs_mid_alpha_both=mid_alpha)
    for q in (dg.fwd.dg_quantizer.lhs, dg.fwd.dg_quantizer.rhs):
      q.numerics.preserve_max_val = True
      q.calibration = functools.partial(q.calibration, po2_scale=True)
    return config.set_context(dg, None, None)

  a = torch.tensor([[1.0, 2.0, 4.0], [1.0, 4.0, 16.0]], device=gpu)
  b = torch.tensor([[4.0, 2.0, 1.0], [16.0, 4.0, 1.0]], device=gpu)
  dn = (((1,), (1,)), ((0,), (0,)))
  ret = np.array([4.0, 16.0], np.float32) * 3.0
  np.testing.assert_array_equal(_np(aqt.lax_dot_general(a, b, dn)), ret)
  ret_no_mid = np.array([3 * 4.0 ** 2, 3 * 16.0 ** 2], np.float32)
  np.testing.assert_array_equal(_np(make_binary_dg(False)(a, b, dn)), ret_no_mid)
  np.testing.assert_array_equal(_np(make_binary_dg(True)(a, b, dn)), ret)


def test_quantizer_per_tensor_known_answer(gpu):
  """aqt_dot_general_test.py:1115-1144: the abs-max over everything is 2**(bits-1) - 0.5,
  so the single scale is exactly one."""
  from aqt_amd.v2 import aqt_quantizer
  bits = 4
  q = aqt_quantizer.quantizer_make(bits, initialize_calibration=False)
  q.calib_shared_axes = 'per_tensor'
  q.context = utils.Context(key=None, train_step=None)
  q.init_calibration()
  x = torch.tensor([[1, 2, 3, 4], [5, 6, 7, 2 ** (bits - 1) - 0.5], [3, 5, 1, -1]],
                   dtype=torch.float32, device=gpu)
  qx, _ = q.quant(x, calibration_axes=None)
  assert len(qx.scale) == 1 and tuple(qx.scale[0].shape) == (1, 1)
  assert float(qx.scale[0]) == 1.0


def test_quantizer_per_subchannel_shapes(gpu):
  """aqt_dot_general_test.py:1146-1167: an integer input, a float32 scale, axis 2 split in
  tiles of 2; quantize then dequantize through the tiling state."""
  from aqt_amd.v2 import aqt_quantizer
  from aqt_amd.v2 import tiled_dot_general
  q = aqt_quantizer.quantizer_make(4, scale_dtype=torch.float32)
  q.context = utils.Context(key=None, train_step=None)
  x = torch.arange(0, 64, device=gpu).reshape(4, 4, 4)
  ts = tiled_dot_general.generate_tiling_state(x, [tiled_dot_general.AxisTiling(axis=2, tile_size=2)])
  qx, _ = q.quant(x, calibration_axes=[0, 2], tiling_state=ts)
  assert tuple(qx.qvalue.shape) == (4, 4, 2, 2)
  assert tuple(qx.scale[0].shape) == (1, 4, 2, 1)
  assert qx.scale[0].dtype == torch.float32
  y = qx.dequant()
  assert tuple(y.shape) == (4, 4, 4)
  # int4 with per-(row, tile) scales: within half a step of the input, plus the truncation of
  # the cast back to the integer input dtype
  step = _np(qx.scale[0]).max()
  assert y.dtype == x.dtype
  assert np.abs(_np(y) - _np(x)).max() <= 0.5 * step + 1.0


def _mode_dg(lmode, rmode, lcal='ca', rcal='ca', disable_rounding=False):
  """The reference test helper `_modify_dg` (aqt_dot_general_test.py:229-309): po2 scales
  everywhere, the modes on all three contractions, sides in THIS_INPUT mode held in float."""
  dg = config.fully_quantized(use_fwd_quant=False, use_stochastic_rounding=False)
  for raw in (dg.fwd, dg.dlhs, dg.drhs):
    raw.lhs.dequant_mode, raw.rhs.dequant_mode = MODE[lmode], MODE[rmode]
    raw.lhs.calibration_mode, raw.rhs.calibration_mode = CAL[lcal], CAL[rcal]
    for q, mode in ((raw.dg_quantizer.lhs, lmode), (raw.dg_quantizer.rhs, rmode)):
      q.calibration = functools.partial(q.calibration, po2_scale=True)
      if mode == 'this_input' or disable_rounding:
        q.numerics.dtype = None
      if disable_rounding:
        q.numerics.round = False
    if 'this_input' in (lmode, rmode) or disable_rounding:
      raw.dg_accumulator_dtype = None
  return config.set_context(dg, None, None)


@pytest.mark.parametrize('name,kw', [
    ('CA', dict(lmode='output', rmode='output', disable_rounding=True)),
    ('CA int8', dict(lmode='output', rmode='output')),
    ('CA fake', dict(lmode='this_input', rmode='this_input', disable_rounding=True)),
    ('RA L', dict(lmode='other_input', rmode='this_input', lcal='ra', rcal='ra')),
    ('RA R', dict(lmode='this_input', rmode='other_input', lcal='ra', rcal='ra')),
    ('RA fake', dict(lmode='this_input', rmode='this_input', lcal='ra', rcal='ra')),
])
def test_equality_between_different_calibration_axes(gpu, name, kw):
  """aqt_dot_general_test.py:972-1048: on power-of-two data every calibration axis /
  dequantisation mode gives the float result exactly, forward and both gradients."""
  rng = np.random.default_rng(0)
  po2 = lambda shape: np.exp2(np.floor(rng.uniform(-3.0, 3.0, shape) + 3.0)).astype(np.float32)
  lhs, rhs, g = po2((10, 20)), po2((20, 30)), po2((10, 30))
  dg = _mode_dg(**kw)
  dg.assert_config_validity()
  L = U.to_dev(lhs, 'f32', gpu).requires_grad_(True)
  Rr = U.to_dev(rhs, 'f32', gpu).requires_grad_(True)
  out = dg(L, Rr, MATMUL)
  out.backward(U.to_dev(g, 'f32', gpu))
  np.testing.assert_array_equal(_np(out), lhs @ rhs)
  np.testing.assert_array_equal(_np(L.grad), g @ rhs.T)
  np.testing.assert_array_equal(_np(Rr.grad), lhs.T @ g)


@pytest.mark.parametrize('dt', ['f32', 'bf16'])
@pytest.mark.parametrize('p,clip', [(1.0, 1.0), (1.0, 2.5), (2.0, 1.5)])
def test_abs_mean_calibration(gpu, p, clip, dt):
  """AbsMeanCalibration (calibration.py:160-193) on integer-valued data, where the sums are
  exact whatever their order; p = 2 goes through the device pow (2 ulp allowed there)."""
  from aqt_amd.v2 import aqt_quantizer
  rng = np.random.default_rng(3)
  x = rng.integers(-6, 7, (24, 96)).astype(np.float32)
  x[5] = 0.0
  q = aqt_quantizer.quantizer_make(8, initialize_calibration=False)
  q.calibration = functools.partial(calibration.AbsMeanCalibration, clipping_scale=clip, p=p)
  q.context = utils.Context(key=None, train_step=None)
  q.init_calibration()
  qx, _ = q.quant(U.to_dev(x, dt, gpu), calibration_axes=[1])
  oq = R.QuantizerCfg(bits=8, abs_mean_p=p, clipping_scale=clip)
  want = R.quantize(x, dt, oq, [1])
  if p == 1.0:
    np.testing.assert_array_equal(_np(qx.scale[0]), want.scale[0])
    np.testing.assert_array_equal(_np(qx.qvalue), np.asarray(want.qvalue, np.float32))
  else:
    np.testing.assert_allclose(_np(qx.scale[0]), want.scale[0], rtol=2.4e-7 if dt == 'f32' else 8e-3)


@pytest.mark.parametrize('dt', ['f32', 'bf16'])
@pytest.mark.parametrize('bits', [4, 8])
def test_snr_based_auto_calibration(gpu, bits, dt):
  """SnrBasedAutoCalibration (calibration.py:196-399) through config.set_auto_calib_scale:
  rows with an outlier pick a smaller clipping scale; scale and quantized weights equal the
  oracle's."""
  rng = np.random.default_rng(0)
  w = rng.standard_normal((1024, 12)).astype(np.float32)
  w[7, ::2] = 12.0 if bits == 4 else 300.0
  w = R.nm.cast(w, dt)
  lhs = U.rand((16, 1024), dt, 1)
  cands = [1.0, 0.5, 0.25, 0.1, 0.05]
  dg = config.dot_general_make(bits, bits)
  config.set_auto_calib_scale(dg, cands)
  dg = config.set_context(dg, None, None)
  out, (_, rqt) = dg.dg_core(U.to_dev(lhs, dt, gpu), U.to_dev(w, dt, gpu), None, None, MATMUL)
  oraw = R.RawCfg(R.QuantizerCfg(bits=bits), R.QuantizerCfg(bits=bits, auto_clip_search=cands))
  want, _, (_, rres), _ = R.dg_raw(lhs, dt, w, dt, MATMUL, oraw)
  np.testing.assert_array_equal(_np(rqt.scale[0]), rres.qx.scale[0])
  np.testing.assert_array_equal(_np(rqt.qvalue), np.asarray(rres.qx.qvalue, np.float32))
  np.testing.assert_array_equal(_np(out), want)
  ratio = _np(rqt.scale[0])[0] / (np.abs(w).max(axis=0) / R.quant_bound(oraw.rhs))
  if bits == 4:  # coarse steps: clipping the outlier pays
    assert (ratio[::2] < 0.75).all() and len(set(np.round(ratio, 3))) > 1


def test_qtensor_with_tiling_state(gpu):
  """aqt_tensor_test.py:122-204: a QTensor quantized through a tiling state reports the
  untiled shape, holds the tiled qvalue, dequantizes back to the untiled shape, and refuses a
  tiling state that does not match its qvalue."""
  from aqt_amd.v2 import aqt_tensor
  from aqt_amd.v2 import tiled_dot_general as T
  rng = np.random.default_rng(0)
  lhs = torch.from_numpy(rng.integers(0, 100, (30, 40, 50)).astype(np.float32)).to(gpu)
  rhs = torch.from_numpy(rng.integers(0, 100, (40, 50, 60)).astype(np.float32)).to(gpu)
  cfg = T.Cfg(
      lhs=T.TensorTiling(contraction_axes=[T.AxisTiling(axis=1, tile_size=10), T.AxisTiling(axis=2, tile_size=25)],
                         remaining_axes=[]),
      rhs=T.TensorTiling(contraction_axes=[T.AxisTiling(axis=0, tile_size=10), T.AxisTiling(axis=1, tile_size=25)],
                         remaining_axes=[]))
  lhs_ca, rhs_ca = (1, 2), (0, 1)
  xlhs, xrhs = T.generate_tiling_states_for_dot_general(cfg, lhs, rhs, ((lhs_ca, rhs_ca), ((), ())))
  qts = []
  for x, st, ca in ((lhs, xlhs, lhs_ca), (rhs, xrhs, rhs_ca)):
    _, tca = st.to_tiled_axes_transposed(ca)
    scale = torch.amax(st.apply(x), dim=list(tca), keepdim=True) / (2.0 ** 7 - 1)
    qt = aqt_tensor.QTensor(qvalue=None, scale=[scale], scale_t=None, bias=[], dequant_dtype=scale.dtype,
                            tiling_state=st)
    qt = qt.quant(x)
    assert qt.shape == tuple(x.shape) and qt.ndim == x.dim()
    assert tuple(qt.qvalue.shape) == tuple(st.tiled_shape)
    deq = qt.dequant()
    assert tuple(deq.shape) == tuple(x.shape)
    np.testing.assert_allclose(_np(deq), _np(x), rtol=1e-6)  # no rounding in QTensor.quant
    qts.append(qt)
  qlhs, qrhs = qts
  qlhs.tiling_state.tiled_shape = tuple(qrhs.qvalue.shape)
  with pytest.raises(AssertionError):
    qlhs.dequant()
  with pytest.raises(AssertionError):
    qlhs.shape  # pylint: disable=pointless-statement

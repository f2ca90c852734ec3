"""The reference's main metamorphic test, restated on this library (GPU).

aqt_dot_general_test.py:465-760 runs a list of configurations (1..8 bit, unquantized,
one-sided, local AQT, clip_gradient, bf16, a 4-D / 5-D dimension_numbers case) and for each one
checks *exact* equalities between ways of computing the same numbers once all scales are
powers of two:

  * the integer path with output dequantisation == fake quantization == the raw forward
    call == the raw fake-quant forward call;
  * mid-scale quantization, integer path == fake-quant path;
  * use_fwd_quant on == off when rounding is disabled;
  * local AQT, integer path == fake-quant path;
  * a numerics object of the user's own ("tricky": rounds, and lets gradient through only
    where x >= 0) zeroes exactly the gradients it should;
  * the unquantized config == the plain float contraction.

Exact equality holds here as it does in the reference: products and sums of small integers
are exact in float32 whatever the summation order, and power-of-two scales commute with
rounding.
"""
import copy
import functools

import numpy as np
import pytest
import torch

from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import config
from aqt_amd.v2.numerics import int_numerics
from aqt_amd.v2.numerics import no_numerics
from aqt_amd.v2.numerics import numerics

pytestmark = pytest.mark.gpu

KEY = np.array([0, 4], np.uint32)  # jax.random.PRNGKey(4)
OUTPUT, THIS_INPUT = aqt.DequantMode.OUTPUT, aqt.DequantMode.THIS_INPUT
CA = aqt.CalibrationMode.CONTRACTING_AXIS


def _apply_po2_scale(quantizer):
  if quantizer.calibration is None:
    return
  cls, keywords = quantizer.calibration, {}
  if isinstance(cls, functools.partial):
    keywords, cls = dict(cls.keywords), cls.func
  keywords.update(po2_scale=True)
  quantizer.calibration = functools.partial(cls, **keywords)


class _TrickyNumerics(numerics.AqtNumerics):
  """Rounds; zero gradient where x < 0 (aqt_dot_general_test.py:188-211)."""
  dtype = None

  def get_dtype(self):
    return self.dtype

  def get_quant_bound(self):
    return 1.0

  def vjp_fwd(self, x, context):
    del context
    return torch.round(x), (x,)

  def vjp_bwd(self, res, grad):
    (x,) = res
    return (grad * (x >= 0), None)


def _modify_dg(readonly_dg, *, lhs_dequant_mode=OUTPUT, rhs_dequant_mode=OUTPUT,
               lhs_calibration_mode=CA, rhs_calibration_mode=CA, use_fwd_quant=None,
               disable_rounding=False, fwd_lhs_tricky_clip_and_round=False, local_aqt=None,
               use_mid_quant=False, clip_gradient=False):
  """aqt_dot_general_test.py:214-309."""
  dg = copy.deepcopy(readonly_dg)
  if fwd_lhs_tricky_clip_and_round:
    dg.fwd.dg_quantizer.lhs.numerics = _TrickyNumerics()
    dg.fwd.dg_accumulator_dtype = None

  def disable_quant_types(c, on_lhs=True, on_rhs=True):
    if on_lhs:
      c.dg_quantizer.lhs.numerics.dtype = None
    if on_rhs:
      c.dg_quantizer.rhs.numerics.dtype = None
    if on_lhs or on_rhs:
      c.dg_accumulator_dtype = None

  for c in (dg.fwd, dg.dlhs, dg.drhs):
    _apply_po2_scale(c.dg_quantizer.lhs)
    _apply_po2_scale(c.dg_quantizer.rhs)
    c.lhs.dequant_mode, c.rhs.dequant_mode = lhs_dequant_mode, rhs_dequant_mode
    c.lhs.calibration_mode, c.rhs.calibration_mode = lhs_calibration_mode, rhs_calibration_mode
    disable_quant_types(c, lhs_dequant_mode == THIS_INPUT, rhs_dequant_mode == THIS_INPUT)

  if disable_rounding:
    for c in (dg.fwd, dg.dlhs, dg.drhs):
      disable_quant_types(c)
      for q in (c.dg_quantizer.lhs, c.dg_quantizer.rhs):
        if isinstance(q.numerics, int_numerics.IntSymmetric):
          q.numerics.round = False

  if use_fwd_quant is not None:
    if not isinstance(dg.fwd.dg_quantizer.lhs.numerics, no_numerics.NoNumerics):
      dg.drhs.rhs.use_fwd_quant = use_fwd_quant
    if not isinstance(dg.fwd.dg_quantizer.rhs.numerics, no_numerics.NoNumerics):
      dg.dlhs.rhs.use_fwd_quant = use_fwd_quant

  if use_mid_quant:
    config.set_use_mid_quant(dg, fwd_mid_alpha_both=1.0, dlhs_mid_alpha_both=1.0, drhs_mid_alpha_both=1.0)

  if local_aqt is not None:
    dg.dlhs.local_aqt = local_aqt
    dg.drhs.local_aqt = local_aqt

  for q in (dg.fwd.dg_quantizer.lhs, dg.fwd.dg_quantizer.rhs):
    if isinstance(q.numerics, int_numerics.IntSymmetric):
      q.numerics.clip_gradient = clip_gradient
  return dg


def _aqt_dg_full_lr_diff(lhs_dequant_mode, rhs_dequant_mode, lhs_calibration_mode=CA,
                         rhs_calibration_mode=CA, *, readonly_dg, dims, **kw):
  dg = _modify_dg(readonly_dg, lhs_dequant_mode=lhs_dequant_mode, rhs_dequant_mode=rhs_dequant_mode,
                  lhs_calibration_mode=lhs_calibration_mode, rhs_calibration_mode=rhs_calibration_mode, **kw)
  dg = config.set_context(dg, key=KEY, train_step=None)
  return lambda lhs, rhs: dg(lhs, rhs, dims)


def _aqt_dg_full(dequant_mode, calibration_mode=CA, **kw):
  return _aqt_dg_full_lr_diff(dequant_mode, dequant_mode, calibration_mode, calibration_mode, **kw)


def _aqt_dg_raw_lr_diff(lhs_dequant_mode, rhs_dequant_mode, lhs_calibration_mode=CA,
                        rhs_calibration_mode=CA, *, readonly_dg, dims):
  dg = _modify_dg(readonly_dg, lhs_dequant_mode=lhs_dequant_mode, rhs_dequant_mode=rhs_dequant_mode,
                  lhs_calibration_mode=lhs_calibration_mode, rhs_calibration_mode=rhs_calibration_mode)
  dg = config.set_context(dg, key=KEY, train_step=None)
  dg.fwd.dg_quantizer.init_calibration()
  return lambda lhs, rhs: dg.fwd(lhs, rhs, None, None, dims)[0]


def _aqt_dg_raw(dequant_mode, calibration_mode=CA, **kw):
  return _aqt_dg_raw_lr_diff(dequant_mode, dequant_mode, calibration_mode, calibration_mode, **kw)


def _eq(name, a, b, exact=True):
  """Exact equality where every contraction sums small integers (any summation order gives the
  same float); where a contraction is a float one on arbitrary data (an unquantized side),
  the library GEMM's summation order depends on the operand layout, which differs between the
  paths compared: there the bound is 4e-6 of the largest magnitude in float32 (the order
  noise of <= 30-term sums), one bf16 ulp in bfloat16.  A single flipped rounding of an 8-bit
  operand would move an output by >= 6e-5 of that magnitude."""
  assert a.shape == b.shape, (name, a.shape, b.shape)
  assert a.dtype == b.dtype, (name, a.dtype, b.dtype)
  if not a.numel():
    return
  err = (a.float() - b.float()).abs().max().item()
  if exact:
    assert err == 0.0, f'{name}: max err = {err}'
  else:
    tol = (4e-6 if a.dtype == torch.float32 else 2.0 ** -7) * a.float().abs().max().item()
    assert err <= tol, f'{name}: max err = {err} > {tol}'


def _quantized(raw):
  return not any(isinstance(q.numerics, no_numerics.NoNumerics)
                 for q in (raw.dg_quantizer.lhs, raw.dg_quantizer.rhs))


def _check_result_eq(dgs, *, lhs, rhs, gra, exact=(True, True, True)):
  """aqt_dot_general_test.py:144-183."""
  good = None
  for name, dg, options in dgs:
    test_gradient = options.get('test_gradient', True)
    lrf = dg(lhs, rhs)
    L, Rr = lhs.clone().requires_grad_(True), rhs.clone().requires_grad_(True)
    lr = dg(L, Rr)
    gl = gr = None
    if test_gradient:
      lr.backward(gra)
      gl, gr = L.grad, Rr.grad
    lr = lr.detach()
    if options.get('check_fwd_lhs_tricky_clip_and_round', False):
      assert (gl[lhs < 0] == 0.0).all()
    if good is None:
      good = (lr, gl, gr)
    _eq(f'{name}: lr vs lrf', lr, lrf.detach())
    _eq(f'{name}: lr', good[0], lr, exact[0])
    if test_gradient:
      _eq(f'{name}: gl', good[1], gl, exact[1])
      _eq(f'{name}: gr', good[2], gr, exact[2])


def _rand_unif(shape, maxval, seed, dtype, dev):
  x = np.random.default_rng(seed).uniform(-maxval, maxval, shape).astype(np.float32)
  return torch.from_numpy(x).to(dtype).to(dev)


def _fqt(s, use_fwd_quant, **kw):
  return dict(dg=lambda: config.fully_quantized(use_fwd_quant=use_fwd_quant, use_stochastic_rounding=False, **kw),
              seed=s)


_DIMS_5D = dict(dims=(((0, 2), (1, 0)), ((3, 1), (2, 4))), lhs_shape=(2, 3, 5, 4),
                rhs_shape=(5, 2, 4, 6, 3), gra_shape=(4, 3, 6))
_LOCAL2 = aqt.LocalAqt(contraction_axis_shard_count=2)

CASES = [
    dict(dg=lambda: config.config_v3(fwd_bits=3, dlhs_bits=6, drhs_bits=5, drhs_accumulator_dtype=torch.int32)),
    dict(dg=lambda: config.dot_general_make(None, None)),
    dict(dg=lambda: config.dot_general_make(1, 1)),
    dict(dg=lambda: config.dot_general_make(1, 2)),
    dict(dg=lambda: config.dot_general_make(2, 1)),
    dict(dg=lambda: config.dot_general_make(2, 2)),
    dict(dg=lambda: config.dot_general_make(8, 8)),
    dict(dg=lambda: config.dot_general_make(8, 8), clip_gradient=True),
    dict(dg=lambda: config.dot_general_make(8, 8, dlhs_local_aqt=_LOCAL2)),
    dict(dg=lambda: config.dot_general_make(8, 8, drhs_local_aqt=_LOCAL2)),
    dict(dg=lambda: config.dot_general_make(2, 2), dtype=torch.bfloat16),
    dict(dg=lambda: config.dot_general_make(8, 8), dtype=torch.bfloat16),
    dict(dg=lambda: config.dot_general_make(None, 8)),
    dict(dg=lambda: config.dot_general_make(8, None)),
    dict(_fqt(10, True), **_DIMS_5D),
    dict(_fqt(10, True, dlhs_local_aqt=_LOCAL2), **_DIMS_5D),
    dict(dg=lambda: config.dot_general_make(2, 2), **_DIMS_5D),
    *[_fqt(s, False) for s in range(3)],
    *[_fqt(s, True) for s in range(3)],
]


@pytest.mark.parametrize('case', range(len(CASES)))
def test_dot_general_calibration_with_contracting_axis(gpu, case):
  p = dict(lhs_maxval=10.0, rhs_maxval=20.0, gra_maxval=30.0, dims=(((1,), (0,)), ((), ())),
           lhs_shape=(10, 20), rhs_shape=(20, 30), gra_shape=(10, 30), seed=0, dtype=torch.float32,
           clip_gradient=False)
  p.update(CASES[case])
  readonly_dg, dims, dtype = p['dg'](), p['dims'], p['dtype']
  lhs = _rand_unif(p['lhs_shape'], p['lhs_maxval'], p['seed'], dtype, gpu)
  rhs = _rand_unif(p['rhs_shape'], p['rhs_maxval'], p['seed'] + 1, dtype, gpu)
  gra = _rand_unif(p['gra_shape'], p['gra_maxval'], p['seed'] + 2, dtype, gpu)

  full = functools.partial(_aqt_dg_full, readonly_dg=readonly_dg, dims=dims, clip_gradient=p['clip_gradient'])
  raw = functools.partial(_aqt_dg_raw, readonly_dg=readonly_dg, dims=dims)
  exact = (_quantized(readonly_dg.fwd), _quantized(readonly_dg.dlhs), _quantized(readonly_dg.drhs))
  check = functools.partial(_check_result_eq, lhs=lhs, rhs=rhs, gra=gra, exact=exact)

  check([
      ('default    ', full(OUTPUT), dict()),
      ('FQ         ', full(THIS_INPUT), dict()),
      ('raw fwd    ', raw(OUTPUT), dict(test_gradient=False)),
      ('raw fwd FQ ', raw(THIS_INPUT), dict(test_gradient=False)),
  ])
  check([
      ('midQ FQ    ', full(THIS_INPUT, use_mid_quant=True, use_fwd_quant=False), dict()),
      ('midQ       ', full(OUTPUT, use_mid_quant=True, use_fwd_quant=False), dict()),
  ])
  check([
      ('fwd_quant=F', full(OUTPUT, use_fwd_quant=False, disable_rounding=True), dict()),
      ('fwd_quant=T', full(OUTPUT, use_fwd_quant=True, disable_rounding=True), dict()),
  ])
  check([
      ('local      ', full(OUTPUT, local_aqt=_LOCAL2), dict()),
      ('local FQ   ', full(THIS_INPUT, local_aqt=_LOCAL2), dict()),
  ])
  if isinstance(readonly_dg.fwd.dg_quantizer.lhs.numerics, int_numerics.IntSymmetric):
    check([('tricky', full(OUTPUT, fwd_lhs_tricky_clip_and_round=True),
            dict(check_fwd_lhs_tricky_clip_and_round=True))])

  def unquant_aqt_dg(lhs, rhs):
    return config.default_unquantized_config()(lhs, rhs, dims)

  def lax_dg(lhs, rhs):
    return _LaxDg.apply(lhs, rhs, dims)

  _check_result_eq([('unquantized default:', unquant_aqt_dg, dict()), ('lax.dot_general:', lax_dg, dict())],
                   lhs=lhs, rhs=rhs, gra=gra)


class _LaxDg(torch.autograd.Function):
  """The plain float contraction with the gradient contractions written out, as the float
  reference of the last check."""

  @staticmethod
  def forward(ctx, lhs, rhs, dims):
    ctx.save_for_backward(lhs, rhs)
    ctx.dims = dims
    return aqt.lax_dot_general(lhs, rhs, dims)

  @staticmethod
  def backward(ctx, g):
    lhs, rhs = ctx.saved_tensors
    outs = []
    for y, y_is_lhs in ((rhs, False), (lhs, True)):
      d, out_axes = aqt._update_dimension_numbers_for_backward(ctx.dims, y_is_lhs, g.dim(), y.dim())
      outs.append(aqt.lax_dot_general(g, y, d).permute(*out_axes))
    return outs[0], outs[1], None


RA_CASES = [
    dict(dg=lambda: config.config_v3(fwd_bits=3, dlhs_bits=4, drhs_bits=5, drhs_accumulator_dtype=torch.int32)),
    dict(dg=lambda: config.dot_general_make(None, None)),
    dict(dg=lambda: config.dot_general_make(1, 1)),
    dict(dg=lambda: config.dot_general_make(1, 2)),
    dict(dg=lambda: config.dot_general_make(2, 1)),
    dict(dg=lambda: config.dot_general_make(2, 2)),
    dict(dg=lambda: config.dot_general_make(8, 8)),
    dict(dg=lambda: config.dot_general_make(8, 8), clip_gradient=True),
    dict(dg=lambda: config.dot_general_make(8, 8, dlhs_local_aqt=_LOCAL2)),
    dict(dg=lambda: config.dot_general_make(8, 8, drhs_local_aqt=_LOCAL2)),
    dict(dg=lambda: config.dot_general_make(2, 2), dtype=torch.bfloat16),
    dict(dg=lambda: config.dot_general_make(8, 8), dtype=torch.bfloat16),
    dict(dg=lambda: config.dot_general_make(None, 8)),
    dict(dg=lambda: config.dot_general_make(8, None)),
    dict(dg=lambda: config.dot_general_make(2, 2), **_DIMS_5D),
    *[_fqt(s, False) for s in range(3)],
]


@pytest.mark.parametrize('case', range(len(RA_CASES)))
def test_dot_general_calibration_with_remaining_axis(gpu, case):
  """aqt_dot_general_test.py:717-903: calibration over the remaining axes; the scale of one
  operand is applied to the other operand (OTHER_INPUT) or the operand is fake-quantized; all
  forms agree exactly, as full calls, raw forward calls and with local AQT in the backward."""
  p = dict(lhs_maxval=10.0, rhs_maxval=20.0, gra_maxval=30.0, dims=(((1,), (0,)), ((), ())),
           lhs_shape=(10, 20), rhs_shape=(20, 30), gra_shape=(10, 30), seed=0, dtype=torch.float32,
           clip_gradient=False)
  p.update(RA_CASES[case])
  readonly_dg, dims, dtype = p['dg'](), p['dims'], p['dtype']
  readonly_dg.drhs.rhs.use_fwd_quant = False
  readonly_dg.dlhs.rhs.use_fwd_quant = False
  lhs = _rand_unif(p['lhs_shape'], p['lhs_maxval'], p['seed'], dtype, gpu)
  rhs = _rand_unif(p['rhs_shape'], p['rhs_maxval'], p['seed'] + 1, dtype, gpu)
  gra = _rand_unif(p['gra_shape'], p['gra_maxval'], p['seed'] + 2, dtype, gpu)
  common = dict(readonly_dg=readonly_dg, dims=dims)
  full = functools.partial(_aqt_dg_full, clip_gradient=p['clip_gradient'], **common)
  full_lr = functools.partial(_aqt_dg_full_lr_diff, clip_gradient=p['clip_gradient'], **common)
  raw = functools.partial(_aqt_dg_raw, **common)
  raw_lr = functools.partial(_aqt_dg_raw_lr_diff, **common)
  exact = (_quantized(readonly_dg.fwd), _quantized(readonly_dg.dlhs), _quantized(readonly_dg.drhs))
  check = functools.partial(_check_result_eq, lhs=lhs, rhs=rhs, gra=gra, exact=exact)
  OTHER, RA = aqt.DequantMode.OTHER_INPUT, aqt.CalibrationMode.REMAINING_AXIS
  check([
      ('RA L       ', full_lr(OTHER, THIS_INPUT, RA, RA), dict()),
      ('RA R       ', full_lr(THIS_INPUT, OTHER, RA, RA), dict()),
      ('RA fake    ', full(THIS_INPUT, RA), dict()),
      ('RA L fwd   ', raw_lr(OTHER, THIS_INPUT, RA, RA), dict(test_gradient=False)),
      ('RA R fwd   ', raw_lr(THIS_INPUT, OTHER, RA, RA), dict(test_gradient=False)),
      ('RA fake fwd', raw(THIS_INPUT, RA), dict(test_gradient=False)),
  ])
  check([
      ('RA fake    ', full(THIS_INPUT, RA, local_aqt=_LOCAL2), dict()),
      ('RA L       ', full_lr(OTHER, THIS_INPUT, RA, RA, local_aqt=_LOCAL2), dict()),
      ('RA R       ', full_lr(THIS_INPUT, OTHER, RA, RA, local_aqt=_LOCAL2), dict()),
  ])


def test_dynamic_context(gpu):
  """aqt_dot_general_test.py:1050-1058: a rank-1 contraction, value and gradient."""
  dg = config.set_context(config.dot_general_make(), key=KEY, train_step=None)
  lhs = torch.tensor([3.0, 4.0], device=gpu, requires_grad=True)
  rhs = torch.tensor([4.0, 5.0], device=gpu, requires_grad=True)
  out = dg(lhs, rhs, (((0,), (0,)), ((), ())))
  out.backward()
  assert out.item() == 32.0
  assert lhs.grad.tolist() == [4.0, 5.0] and rhs.grad.tolist() == [3.0, 4.0]


def test_hardware_int8(gpu):
  """aqt_dot_general_test.py:1060-1077: the contraction of an 8-bit config really is
  int8 x int8 -> int32."""
  dg_raw = config.dot_general_raw_make(8, 8)
  seen = []

  def hook(lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None):
    out = aqt.lax_dot_general(lhs, rhs, dimension_numbers, precision, preferred_element_type)
    seen.append((lhs.dtype, rhs.dtype, out.dtype))
    return out

  dg_raw.dot_general = hook
  lhs = _rand_unif((10, 20), 1.0, 0, torch.float32, gpu)
  rhs = _rand_unif((20, 30), 1.0, 1, torch.float32, gpu)
  ret, _ = dg_raw(lhs, rhs, None, None, (((1,), (0,)), ((), ())))
  assert seen == [(torch.int8, torch.int8, torch.int32)] and ret.dtype == torch.float32
  assert dg_raw.dg_quantizer.lhs.numerics.get_dtype() == torch.int8
  assert dg_raw.dg_quantizer.rhs.numerics.get_dtype() == torch.int8


@pytest.mark.parametrize('shard_count,expected_product', [(2, 1281280.0), (1, 1280000.0)])
def test_local_aqt_known_answer(gpu, shard_count, expected_product):
  """aqt_dot_general_test.py:1079-1113: with two shards the small and the large half of lhs
  get their own scales in the drhs contraction, with one shard 1270 and 10 round to 0 and 0...
  the reference's expected gradients."""
  dg = config.fully_quantized(fwd_bits=8, bwd_bits=8, use_stochastic_rounding=False,
                              drhs_local_aqt=aqt.LocalAqt(contraction_axis_shard_count=shard_count))
  for q in (dg.fwd.dg_quantizer.lhs, dg.fwd.dg_quantizer.rhs, dg.drhs.dg_quantizer.lhs, dg.drhs.dg_quantizer.rhs):
    q.numerics.preserve_max_val = True
  dg = config.set_context(dg, None, None)
  lhs = torch.tensor([1270.0, 10.0, 1270000.0, 10000.0], device=gpu, requires_grad=True)
  rhs = torch.tensor([1.0], device=gpu, requires_grad=True)
  out = dg(lhs, rhs, (((), ()), ((), ())))
  out.backward(torch.ones_like(out))
  assert rhs.grad.item() == expected_product

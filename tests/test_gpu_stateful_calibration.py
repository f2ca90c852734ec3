"""Stateful calibrators (static range, weighted statistics, delayed scaling) on the GPU: the
statistics follow the closed-form sequences of the reference's update rules
(flax/aqt_flax_calibration.py:33-251, flax/delayed_scaling_calibration.py:26-124), and a
DotGeneral configured with them quantizes with the bound those statistics give."""
import functools

import numpy as np
import pytest
import torch

from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import calibration
from aqt_amd.v2 import config
from aqt_amd.v2 import utils
from aqt_amd.v2.flax import aqt_flax_calibration
from aqt_amd.v2.flax import delayed_scaling_calibration
from aqt_amd.v2.numerics import int_numerics

pytestmark = pytest.mark.gpu


def _num8():
  return int_numerics.IntSymmetric(bits=8, preserve_zero=True, preserve_max_val=False, clip=True, round=True,
                                   noise_fn=None, clip_gradient=False, dtype=torch.int8)


def _ctx(mode):
  return utils.Context(key=None, train_step=None, quant_mode=mode)


def test_mean_of_abs_max(gpu):
  st = calibration.State()
  cal = aqt_flax_calibration.MeanOfAbsMaxCalibration(quant_collection='qc', state=st)
  xs = [torch.tensor([[1.0, -4.0], [2.0, 0.5]], device=gpu) * f for f in (1.0, 3.0, 5.0)]
  # the first call only creates the statistics (Flax init); the next ones accumulate
  cal.get_bound(xs[0], [1], _ctx(utils.QuantMode.CALIBRATE))
  assert st['count'].item() == 0
  for x in xs:
    bound = cal.get_bound(x, [1], _ctx(utils.QuantMode.CALIBRATE))
  assert st['count'].item() == 3
  np.testing.assert_array_equal(bound.cpu().numpy(), np.array([[4.0 * 3], [2.0 * 3]], np.float32))
  # other modes read the statistics and leave them alone
  b2 = cal.get_bound(xs[2] * 100, [1], _ctx(utils.QuantMode.TRAIN))
  assert torch.equal(b2, bound) and st['count'].item() == 3
  # a new calibrator object given the same dict continues from it
  cal2 = aqt_flax_calibration.MeanOfAbsMaxCalibration(quant_collection='qc', state=st)
  (scale,), bias, mask = cal2.get_scale_and_bias_and_sparsity(xs[0], [1], _num8(), _ctx(utils.QuantMode.SERVE))
  np.testing.assert_array_equal(scale.cpu().numpy(), (bound / torch.tensor(127.5, device=gpu)).cpu().numpy())
  assert bias == [] and mask is None


def test_weighted_stats(gpu):
  st = calibration.State()
  cal = aqt_flax_calibration.WeightedStatsCalibration(
      quant_collection='qc', state=st, l1_dev_coeff=1.0, lp_dev_coeff=2.0, max_dev_coeff=3.0,
      const_bound_coeff=0.5, ema_update_count=4)
  x = torch.tensor([[3.0, -4.0, 0.0, 0.0]], device=gpu)
  bound = cal.get_bound(x, [1], _ctx(utils.QuantMode.TRAIN))
  rate = 0.25
  ones = (1 - rate) * 1.0 + rate * 2.0          # prior count 1, two non-zero entries
  l1 = (rate * 7.0) / ones
  lp = np.sqrt((rate * 25.0) / ones)
  mx = rate * 4.0
  np.testing.assert_allclose(bound.cpu().numpy(), [[1.0 * l1 + 2.0 * lp + 3.0 * mx + 0.5]], rtol=1e-6)
  before = {k: v.clone() for k, v in st.items()}
  cal.get_bound(x * 9, [1], _ctx(utils.QuantMode.SERVE))
  assert all(torch.equal(st[k], before[k]) for k in st)
  assert tuple(st['sum_of_ones'].shape) == (1, 1) and st['sum_of_ones'].dtype == torch.float32


def test_delayed_scaling_history_and_bound(gpu):
  st = calibration.State()
  cal = delayed_scaling_calibration.DelayedScalingCalibration(amax_history_length=3, state=st)
  xs = [torch.full((4, 5), v, device=gpu, dtype=torch.bfloat16) for v in (2.0, -8.0, 4.0, 1.0, 0.5)]
  bounds = [cal.get_bound(x, None, _ctx(utils.QuantMode.TRAIN)).reshape(()).item() for x in xs]
  # the bound of a step is the largest abs-max of the (up to three) previous steps; before any
  # history it is the initial 0 (amax <= 0 keeps the previous bound)
  assert bounds == [0.0, 2.0, 8.0, 8.0, 8.0]
  assert st['amax_history'].tolist() == [0.5, 4.0, 1.0] or sorted(st['amax_history'].tolist()) == [0.5, 1.0, 4.0]
  b_serve = cal.get_bound(xs[0] * 100, None, None)  # no context: SERVE, nothing is written
  assert b_serve.reshape(()).item() == 4.0 and sorted(st['amax_history'].tolist()) == [0.5, 1.0, 4.0]
  # a zero or non-finite history keeps the previous bound
  st2 = calibration.State(amax_history=torch.zeros(3, device=gpu), bound=torch.tensor([7.0], device=gpu))
  cal2 = delayed_scaling_calibration.DelayedScalingCalibration(amax_history_length=3, state=st2)
  assert cal2.get_bound(xs[0], None, _ctx(utils.QuantMode.TRAIN)).reshape(()).item() == 7.0


def test_dot_general_with_delayed_scaling(gpu):
  """fp8-style per-tensor delayed scaling through the DotGeneral API: the second step
  quantizes with the abs-max of the first step's operands."""
  states = {}

  def make():
    dg = config.dot_general_make(8, 8)
    for name, q in (('lhs', dg.fwd.dg_quantizer.lhs), ('rhs', dg.fwd.dg_quantizer.rhs)):
      q.calibration = functools.partial(delayed_scaling_calibration.DelayedScalingCalibration,
                                        amax_history_length=4, state=states.setdefault(name, calibration.State()))
      q.calib_shared_axes = 'per_tensor'
    return config.set_context(dg, None, None)

  rng = np.random.default_rng(0)
  a1 = torch.from_numpy(rng.standard_normal((16, 64)).astype(np.float32)).to(gpu)
  b1 = torch.from_numpy(rng.standard_normal((64, 24)).astype(np.float32)).to(gpu)
  make().dg_core(a1, b1, None, None, (((1,), (0,)), ((), ())))  # step 1: bound 0 -> scale 0, fills the history
  a2, b2 = a1 * 0.5, b1 * 0.25
  out, (lqt, rqt) = make().dg_core(a2, b2, None, None, (((1,), (0,)), ((), ())))
  q = torch.tensor(127.5, device=gpu)
  assert lqt.scale[0].reshape(()).item() == (a1.abs().max() / q).item()
  assert rqt.scale[0].reshape(()).item() == (b1.abs().max() / q).item()
  ref = a2 @ b2
  # 7 and 6 effective bits (the operands are half and a quarter of the bounds)
  assert (out - ref).abs().max().item() <= 0.05 * ref.abs().max().item()


class _CountingAbsMax(calibration.AbsMaxCalibration):
  """Abs-max calibration that counts its calls and has no fused kernel (a stand-in for any
  stateful calibrator: every call is a state update)."""
  calls = 0

  def kernel_supported(self):
    return False

  def get_scale_and_bias_and_sparsity(self, x, shared_axes, numerics_, context=None):
    type(self).calls += 1
    return super().get_scale_and_bias_and_sparsity(x, shared_axes, numerics_, context)


def test_fallback_after_a_fused_attempt_calibrates_once(gpu):
  """The lhs calibrates step by step inside the fused attempt; the rhs (numerics without the clip)
  then turns the call over to the step-by-step path, which must take the lhs scale over
  instead of calibrating a second time (the reference calibrates once per call)."""
  dg = aqt.dot_general_raw_make(8, 8)
  dg.dg_quantizer.lhs.calibration = _CountingAbsMax
  dg.dg_quantizer.rhs.numerics.clip = False  # no fused form: found out after the lhs is done
  dg.dg_quantizer.lhs._calibrator = None
  dg.dg_quantizer.rhs._calibrator = None
  dg.dg_quantizer.init_calibration()
  lhs = torch.randn(32, 64, device=gpu)
  rhs = torch.randn(64, 48, device=gpu)
  _CountingAbsMax.calls = 0
  out, res = dg(lhs, rhs, None, None, (((1,), (0,)), ((), ())))
  torch.cuda.synchronize()
  assert _CountingAbsMax.calls == 1
  assert out.shape == (32, 48) and torch.isfinite(out).all()
  # and the scale the step-by-step path used is the one that calibration returned
  want = lhs.abs().amax(dim=1, keepdim=True) / torch.tensor(127.5, device=gpu)  # a tensor divisor rounds correctly
  torch.testing.assert_close(res.lhs.mt.qx.scale[0], want, rtol=0, atol=0)

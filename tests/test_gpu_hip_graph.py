"""GPU: serving calls recorded into a HIP graph give the eager call's bits on every replay.

Each graph is replayed several times on fresh inputs, with eager calls of the same layer (and
synchronisations) between the replays, and every replay is compared with the eager result.
"""
import pytest
import torch

from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import config
from aqt_amd.v2 import hip_graph
from aqt_amd.v2 import tiled_dot_general
from aqt_amd.v2 import utils
from aqt_amd.v2.flax import aqt_flax
from tests import gpu_util as U

pytestmark = pytest.mark.gpu
QM, FM = utils.QuantMode, aqt_flax.FreezerMode
MATMUL = (((1,), (0,)), ((), ()))


def _rngs():
  return {'params': utils.prng_key(0)}


def _serving_layer(cfg, x, w, tiling=None):
  mk = lambda mode: aqt_flax.AqtDotGeneral(
      cfg, rhs_quant_mode=mode, tiling_cfg=tiling, lhs_freeze_mode=FM.CALIBRATION,
      rhs_freeze_mode=FM.CALIBRATION_AND_VALUE, use_legacy_freezer=False, rngs=_rngs())
  with torch.no_grad():
    conv = mk(QM.CONVERT)
    conv(x, w, MATMUL, None)
    serve = mk(QM.SERVE)
    serve.load_variables(conv.variables())
  return serve


def _check_replays(graphed, eager, make_input, n=5):
  for i in range(n):
    x = make_input(100 + i)
    got = graphed(x).clone()
    torch.cuda.synchronize()
    with torch.no_grad():
      want = eager(x)
      eager(make_input(500 + i))  # eager work of the same kernels between replays
    torch.cuda.synchronize()
    assert got.dtype == want.dtype and got.shape == want.shape
    assert torch.equal(got, want), f'replay {i} differs from the eager call'


@pytest.mark.parametrize('m,k', [(1, 1024), (8, 1024), (64, 1024), (512, 1024), (96, 4096)])
def test_int8_serving_layer_replays(gpu, m, k):
  """Frozen int8 weight: the small-batch decode kernels (m <= 64) and the dense GEMM (m = 512; m = 96 with
  k = 4096: few output tiles and a long k, contracted in slices of k through a scratch array)."""
  dt = 'bf16'
  n = 1536
  w = U.to_dev(U.rand((k, n), dt, 2, 0.02), dt, gpu)
  mk = lambda seed: U.to_dev(U.rand((m, k), dt, seed, outliers=True), dt, gpu)
  serve = _serving_layer(config.fully_quantized(use_stochastic_rounding=False), mk(1), w)
  call = lambda x: serve(x, w, MATMUL, None)
  graphed = hip_graph.GraphedCall(call, mk(1))
  _check_replays(graphed, call, mk)


@pytest.mark.parametrize('rhs_bits', [8, 4])
def test_tiled_serving_layer_replays(gpu, rhs_bits):
  """Subchannel scales (contraction axis in 4 tiles): the grouped-scale kernel, int4 weight packed."""
  dt = 'bf16'
  m, k, n, tiles = 16, 1024, 384, 4
  w = U.to_dev(U.rand((k, n), dt, 2, 0.02), dt, gpu)
  mk = lambda seed: U.to_dev(U.rand((m, k), dt, seed, outliers=True), dt, gpu)
  tiling = tiled_dot_general.Cfg(
      lhs=tiled_dot_general.TensorTiling(
          contraction_axes=[tiled_dot_general.AxisTiling(axis=1, tile_count=tiles, tile_size=None)], remaining_axes=[]),
      rhs=tiled_dot_general.TensorTiling(
          contraction_axes=[tiled_dot_general.AxisTiling(axis=0, tile_count=tiles, tile_size=None)], remaining_axes=[]))
  serve = _serving_layer(aqt.dot_general_make(8, rhs_bits), mk(1), w, tiling)
  call = lambda x: serve(x, w, MATMUL, None)
  graphed = hip_graph.GraphedCall(call, mk(1))
  _check_replays(graphed, call, mk)


def test_both_operands_quantized_per_call_replays(gpu):
  """No frozen state: both operands calibrated and quantized inside the recorded call."""
  dt = 'bf16'
  m, k, n = 256, 512, 384
  mk = lambda seed: U.to_dev(U.rand((m, k), dt, seed, outliers=True), dt, gpu)
  w = U.to_dev(U.rand((k, n), dt, 2, 0.02), dt, gpu)
  dg = config.config_v4()
  call = lambda x: dg(x, w, MATMUL)
  graphed = hip_graph.GraphedCall(call, mk(1))
  _check_replays(graphed, call, mk)


def test_quantized_convolution_replays(gpu):
  """conv_general_dilated: per-batch-element abs-max through the kept-zero workspace (owned by the
  graph), window gather, contraction with both scales in the epilogue."""
  from aqt_amd.v2 import aqt_conv_general
  dt = 'bf16'
  mk = lambda seed: U.to_dev(U.rand((4, 14, 14, 128), dt, seed, outliers=True), dt, gpu)
  kernel = U.to_dev(U.rand((3, 3, 128, 64), dt, 2, 0.05), dt, gpu)
  conv = aqt_conv_general.make_conv_general_dilated(aqt_conv_general.conv_general_dilated_make(2, 8, 8))
  dn = aqt_conv_general.flax_conv_dimension_numbers((4, 14, 14, 128))
  call = lambda x: conv(x, kernel, (1, 1), 'SAME', dimension_numbers=dn)
  graphed = hip_graph.GraphedCall(call, mk(1))
  _check_replays(graphed, call, mk)
  # a second graph recorded while the first is alive, replayed alternately
  other = hip_graph.GraphedCall(call, mk(2))
  for i in range(3):
    xa, xb = mk(40 + i), mk(60 + i)
    ya = graphed(xa).clone()
    yb = other(xb).clone()
    with torch.no_grad():
      assert torch.equal(ya, call(xa)) and torch.equal(yb, call(xb))


def test_per_tensor_scales_replay(gpu):
  """Whole-tensor abs-max (atomics into the kept-zero workspace) inside a recording."""
  dt = 'bf16'
  mk = lambda seed: U.to_dev(U.rand((512, 1024), dt, seed, outliers=True), dt, gpu)
  w = U.to_dev(U.rand((1024, 256), dt, 2, 0.02), dt, gpu)
  dg = config.config_v4()
  for raw in (dg.fwd,):
    raw.dg_quantizer.lhs.calib_shared_axes = 'per_tensor'
    raw.dg_quantizer.rhs.calib_shared_axes = 'per_tensor'
  call = lambda x: dg(x, w, MATMUL)
  graphed = hip_graph.GraphedCall(call, mk(1))
  _check_replays(graphed, call, mk)


def test_static_argument_is_read_in_place(gpu):
  dt = 'bf16'
  x = U.to_dev(U.rand((64, 256), dt, 1), dt, gpu)
  w = U.to_dev(U.rand((256, 128), dt, 2, 0.02), dt, gpu)
  dg = config.config_v4()
  graphed = hip_graph.GraphedCall(lambda a, b: dg(a, b, MATMUL), x, w, static_argnums=(1,))
  assert graphed.inputs[1] is w and graphed.inputs[0] is not x
  w2 = U.to_dev(U.rand((256, 128), dt, 3, 0.02), dt, gpu)
  w.copy_(w2)
  got = graphed(x, w).clone()
  with torch.no_grad():
    assert torch.equal(got, dg(x, w2, MATMUL))


def test_argument_checks(gpu):
  x = torch.zeros(8, 256, device=gpu, dtype=torch.bfloat16)
  w = torch.ones(256, 128, device=gpu, dtype=torch.bfloat16)
  dg = config.config_v4()
  graphed = hip_graph.GraphedCall(lambda a: dg(a, w, MATMUL), x)
  with pytest.raises(ValueError, match='recorded as'):
    graphed(torch.zeros(4, 256, device=gpu, dtype=torch.bfloat16))
  with pytest.raises(ValueError, match='recorded as'):
    graphed(x.float())
  with pytest.raises(ValueError, match='arguments'):
    graphed(x, x)
  with pytest.raises(ValueError, match='GPU'):
    hip_graph.GraphedCall(lambda a: a, torch.zeros(4))


def test_training_step_with_a_key_on_the_device_replays(gpu):
  """Forward + backward with stochastic rounding, the PRNG key in a device tensor: the key fan-out of
  set_context runs as a kernel and the quantizers read their keys from device memory, so a recorded step
  draws the noise of whatever key the tensor holds at replay time.  Every replay equals the eager step with
  the same key given as host data."""
  import numpy as np
  dt = 'bf16'
  base = config.fully_quantized(fwd_bits=8, bwd_bits=8)
  x_np, w_np = U.rand((256, 512), dt, 1, outliers=True), U.rand((512, 384), dt, 2, 0.02)
  g = U.to_dev(U.rand((256, 384), dt, 3, 1e-3), dt, gpu)

  def eager(key):
    x = U.to_dev(x_np, dt, gpu).requires_grad_(True)
    w = U.to_dev(w_np, dt, gpu).requires_grad_(True)
    y = config.set_context(base, key, None)(x, w, MATMUL)
    y.backward(g)
    return y.detach(), x.grad, w.grad

  def on_device(key):
    return torch.from_numpy(np.asarray(key, dtype=np.uint32).view(np.int32).copy()).to(gpu)

  k1, k2, k3 = utils.prng_key(11), utils.prng_key(12), utils.prng_key(13)
  want1 = eager(k1)
  got1 = eager(on_device(k1))
  assert all(torch.equal(a, b) for a, b in zip(got1, want1)), 'device key differs from the host key (eager)'
  assert not torch.equal(want1[1], eager(k2)[1]), 'the gradient does not depend on the key'

  key_dev = on_device(k1)
  x = U.to_dev(x_np, dt, gpu).requires_grad_(True)
  w = U.to_dev(w_np, dt, gpu).requires_grad_(True)

  def step():
    x.grad = w.grad = None
    y = config.set_context(base, key_dev, None)(x, w, MATMUL)
    y.backward(g)
    return y, x.grad, w.grad

  graphed = hip_graph.GraphedStep(step)
  for key in (k2, k3, k1, k2):
    key_dev.copy_(on_device(key))
    got = [t.detach().clone() for t in graphed.replay()]
    torch.cuda.synchronize()
    want = eager(key)   # eager work of the same kernels between the replays
    torch.cuda.synchronize()
    for name, a, b in zip(('out', 'dlhs', 'drhs'), got, want):
      assert torch.equal(a, b), f'{name} of the replay differs from the eager step'

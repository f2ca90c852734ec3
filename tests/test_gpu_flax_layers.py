"""GPU: AqtDotGeneral / AqtEinsum modules over the HIP kernels (flows of aqt/jax/v2/flax/aqt_flax_test.py)."""
import numpy as np
import pytest
import torch

from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import config
from aqt_amd.v2 import tiled_dot_general
from aqt_amd.v2 import utils
from aqt_amd.v2.flax import aqt_flax
from oracle import aqt_ref as R
from oracle import prng
from tests import gpu_util as U

pytestmark = pytest.mark.gpu
QM, FM = utils.QuantMode, aqt_flax.FreezerMode
MATMUL = (((1,), (0,)), ((), ()))


def _rngs():
  return {'params': utils.prng_key(0)}


def test_aqt_einsum_external_qtensors(gpu):
  """aqt_flax_test.py:81-158: QTensor operands computed outside give the same result."""
  lhs = torch.rand(3, 4, 5, 6, device=gpu)
  rhs = torch.rand(2, 5, 6, device=gpu)
  eqn = 'ijkh,mkh->ijm'

  def run(lhs_ext, rhs_ext, cfg_fn):
    cfg = cfg_fn()
    lhs_in, rhs_in = lhs, rhs
    if lhs_ext or rhs_ext:
      dgq = cfg_fn().fwd.dg_quantizer
      dgq.init_calibration()
      dn = (((2, 3), (1, 2)), ((), ()))
      (lq, _), (rq, _) = dgq((lhs, dn[0][0]), (rhs, dn[0][1]))
      if lhs_ext:
        lhs_in = lq
      if rhs_ext:
        rhs_in = rq
    einsum = aqt_flax.AqtEinsum(cfg=cfg, lhs_freeze_mode=FM.NONE, rhs_freeze_mode=FM.CALIBRATION_AND_VALUE,
                                rngs=_rngs())
    return einsum(eqn, lhs_in, rhs_in)

  out_float = run(False, False, lambda: None)
  out_int8 = run(False, False, config.config_v4)
  assert torch.equal(out_int8, run(True, False, config.config_v4)), 'lhs external qt failed'
  assert torch.equal(out_int8, run(False, True, config.config_v4)), 'rhs external qt failed'
  assert torch.equal(out_int8, run(True, True, config.config_v4)), 'both external qt failed'
  assert torch.mean((out_int8 - out_float) ** 2) > 0, 'Einsum is not quantized.'
  assert torch.allclose(out_int8, out_float, rtol=0.05, atol=0.05)


@pytest.mark.parametrize('legacy', [True, False])
def test_convert_then_serve(gpu, legacy):
  """TRAIN -> CONVERT (weights frozen into the 'aqt' collection) -> SERVE reads them back:
  the three outputs agree, and serving ignores the float weight it is handed."""
  dt = 'bf16'
  x, w = U.to_dev(U.rand((8, 256), dt, 1), dt, gpu), U.to_dev(U.rand((256, 128), dt, 2, 0.02), dt, gpu)
  cfg = config.fully_quantized(use_stochastic_rounding=False)
  mk = lambda mode: aqt_flax.AqtDotGeneral(cfg, rhs_quant_mode=mode, rhs_freeze_mode=FM.CALIBRATION_AND_VALUE,
                                           use_legacy_freezer=legacy, rngs=_rngs())
  out_train = mk(QM.TRAIN)(x, w, MATMUL, None)
  conv = mk(QM.CONVERT)
  out_conv = conv(x, w, MATMUL, None)
  variables = conv.variables()
  assert set(variables) == {'aqt'} and set(variables['aqt']) == {'qrhs'}
  if legacy:
    assert set(variables['aqt']['qrhs']) == {'value', 'scale'}
    assert tuple(variables['aqt']['qrhs']['value'].shape) == (256, 128)
    assert tuple(variables['aqt']['qrhs']['scale'].shape) == (1, 128)
  else:
    frozen = variables['aqt']['qrhs']['frozen']
    assert tuple(frozen.qvalue.shape) == (256, 128) and tuple(frozen.scale[0].shape) == (1, 128)
  serve = mk(QM.SERVE)
  serve.load_variables(variables)
  out_serve = serve(x, torch.zeros_like(w), MATMUL, None)
  assert torch.equal(out_train, out_conv) and torch.equal(out_train, out_serve)
  f = R.dg_fwd(U.rand((8, 256), dt, 1), U.rand((256, 128), dt, 2, 0.02), dt, MATMUL, R.fully_quantized())
  np.testing.assert_array_equal(out_serve.float().cpu().numpy(), f.out)


def test_freezer_none_with_convert_raises(gpu):
  x, w = torch.randn(4, 32, device=gpu), torch.randn(32, 8, device=gpu)
  dg = aqt_flax.AqtDotGeneral(config.fully_quantized(), rhs_quant_mode=QM.CONVERT, rngs=_rngs())
  with pytest.raises(ValueError, match='Freezer mode NONE'):
    dg(x, w, MATMUL, None)


def test_einsum_swap_moves_the_side_settings(gpu):
  """'bc,ab->ac' reaches dot_general as (rhs, lhs); the frozen weight is einsum's lhs (the model's
  weight in test_einsum_grad_leak, aqt_flax_test.py:160-198) and must land in 'qlhs'."""
  dt = 'bf16'
  wgt, x = U.to_dev(U.rand((64, 48), dt, 1, 0.05), dt, gpu), U.to_dev(U.rand((16, 64), dt, 2), dt, gpu)
  cfg = config.fully_quantized(use_stochastic_rounding=False)
  conv = aqt_flax.AqtEinsum(cfg, lhs_quant_mode=QM.CONVERT, lhs_freeze_mode=FM.CALIBRATION_AND_VALUE, rngs=_rngs())
  out = conv('bc,ab->ac', wgt, x)
  assert tuple(out.shape) == (16, 48)
  v = conv.variables()
  assert set(v['aqt']) == {'qlhs'} and tuple(v['aqt']['qlhs']['value'].shape) == (64, 48)
  ref = aqt.einsum('bc,ab->ac', wgt, x, config.set_context(cfg, utils.prng_key(0), None))
  assert torch.equal(out, ref)


def test_tiling_injection(gpu):
  """aqt_flax_test.py:381-410: tile sizes by einsum letter; the layer result equals
  tiled_dot_general around the same quantized dot_general."""
  dt = 'bf16'
  lhs, rhs = U.to_dev(U.rand((6, 4, 256), dt, 1), dt, gpu), U.to_dev(U.rand((10, 4, 256), dt, 2, 0.02), dt, gpu)
  cfg = config.fully_quantized(use_stochastic_rounding=False)
  layer = aqt_flax.AqtEinsum(cfg, tile_sizes={'d': 64}, rngs=_rngs())
  out = layer('abd,cbd->ac', lhs, rhs)
  tcfg = tiled_dot_general.Cfg.from_einsum('abd,cbd->ac', {'d': 64})
  dg = config.set_context(cfg, utils.prng_key(0), None)
  want = tiled_dot_general.tiled_dot_general(tcfg, lhs, rhs, (((1, 2), (1, 2)), ((), ())), dot_general=dg)
  assert tuple(out.shape) == (6, 10) and torch.equal(out, want)
  untiled = aqt_flax.AqtEinsum(cfg, rngs=_rngs())('abd,cbd->ac', lhs, rhs)
  assert not torch.equal(out, untiled) and torch.allclose(out.float(), untiled.float(), rtol=0.1, atol=0.05)


def test_serving_from_logical_order_checkpoint(gpu):
  """A frozen weight restored in its logical [K, N] order (as a checkpoint would hold it) serves the
  same values as the one the convert step produced, through the decode path and the GEMM path, and
  is re-laid out for the kernels once, not per call: one copy, in the serving kernels' fragment order,
  which the contraction kernels read as well."""
  from aqt_amd.v2 import aqt_dot_general as adg
  dt = 'bf16'
  w = U.to_dev(U.rand((256, 128), dt, 2, 0.02), dt, gpu)
  cfg = config.fully_quantized(use_stochastic_rounding=False)
  conv = aqt_flax.AqtDotGeneral(cfg, rhs_quant_mode=QM.CONVERT, rhs_freeze_mode=FM.CALIBRATION_AND_VALUE, rngs=_rngs())
  x8 = U.to_dev(U.rand((8, 256), dt, 1), dt, gpu)
  x100 = U.to_dev(U.rand((100, 256), dt, 3), dt, gpu)
  want8, want100 = conv(x8, w, MATMUL, None), conv(x100, w, MATMUL, None)
  v = conv.variables()
  v['aqt']['qrhs']['value'] = v['aqt']['qrhs']['value'].contiguous().clone()   # logical row-major, like a restore
  assert v['aqt']['qrhs']['value'].stride() == (128, 1)
  serve = aqt_flax.AqtDotGeneral(cfg, rhs_quant_mode=QM.SERVE, rhs_freeze_mode=FM.CALIBRATION_AND_VALUE, rngs=_rngs())
  serve.load_variables(v)
  adg._KERNEL_LAYOUT_CACHE.clear()
  for _ in range(2):
    assert torch.equal(serve(x8, torch.zeros_like(w), MATMUL, None), want8)
    assert torch.equal(serve(x100, torch.zeros_like(w), MATMUL, None), want100)
  assert len(adg._KERNEL_LAYOUT_CACHE) == 1
  (_, copies), = adg._KERNEL_LAYOUT_CACHE.values()
  assert list(copies) == [(False, True)]  # (packed int4, fragment order)
  assert copies[(False, True)].numel() == 256 * 128


@pytest.mark.parametrize('bits', [8, 4])
def test_e2e_example_head_convert_and_serve(gpu, bits):
  """The quantized layers of the reference's end-to-end example (examples/flax_e2e_model.py:79-145):
  Dense 3136 -> 256 and Dense 256 -> 10 with the contraction axis split in two tiles, then the
  einsum 'bc,ab->ac' against an identity weight with 'b' tiled by 5 and the two sides' quantizers
  swapped.  After conversion the frozen QTensors have the shapes and dtypes the reference's test
  lists (examples/flax_e2e_model_test.py:141-196), the serving model reproduces the training-mode
  logits bit for bit without the float weights, and does use the frozen values
  (examples/flax_e2e_model_test.py:250-271)."""
  import copy
  batch = 4
  torch.manual_seed(0)
  x = torch.randn(batch, 3136, device=gpu)
  w0 = torch.randn(3136, 256, device=gpu) / 56.0
  w1 = torch.randn(256, 10, device=gpu) / 16.0
  # The reference's 4-bit case asks for `fwd_accumulator_dtype=None`, with which lax.dot_general
  # returns the int4 product wrapped to int4 (its expected loss on TPU is ln 10); this build
  # contracts integers into int32 only and says so when asked otherwise, so both cases keep the
  # default int32 accumulator here.
  cfg = config.config_v4(fwd_bits=bits, drhs_bits=8, drhs_accumulator_dtype=utils.int32)
  with pytest.raises(AssertionError, match='int32 accumulator'):
    bad = config.set_context(config.config_v4(fwd_bits=bits, fwd_accumulator_dtype=None), None, None)
    bad(torch.randn(4, 32, device=gpu), torch.randn(32, 8, device=gpu), MATMUL)
  tiling = tiled_dot_general.Cfg(
      lhs=tiled_dot_general.TensorTiling(
          contraction_axes=[tiled_dot_general.AxisTiling(axis=1, tile_count=2, tile_size=None)], remaining_axes=[]),
      rhs=tiled_dot_general.TensorTiling(
          contraction_axes=[tiled_dot_general.AxisTiling(axis=0, tile_count=2, tile_size=None)], remaining_axes=[]))
  cfg_swapped = copy.deepcopy(cfg)
  cfg_swapped.fwd.dg_quantizer.swap_lhs_and_rhs()

  def build(weights_mode, act_mode):
    dense = lambda: aqt_flax.AqtDotGeneral(
        cfg, lhs_quant_mode=act_mode, rhs_quant_mode=weights_mode, tiling_cfg=tiling,
        lhs_freeze_mode=FM.CALIBRATION, rhs_freeze_mode=FM.CALIBRATION_AND_VALUE, use_legacy_freezer=False,
        rngs=_rngs())
    einsum = aqt_flax.AqtEinsum(
        cfg_swapped, lhs_quant_mode=weights_mode, rhs_quant_mode=act_mode, assert_eqn='bc,ab->ac',
        assert_lhs_shape=(10, 10), assert_rhs_shape=(None, 10), tile_sizes={'b': 5},
        lhs_freeze_mode=FM.CALIBRATION_AND_VALUE, rhs_freeze_mode=FM.CALIBRATION, use_legacy_freezer=False,
        rngs=_rngs())
    return dense(), dense(), einsum

  def forward(layers, w0_, w1_):
    d0, d1, es = layers
    h = torch.relu(d0(x, w0_, MATMUL, None))
    h = d1(h, w1_, MATMUL, None)
    return es('bc,ab->ac', torch.eye(10, device=gpu, dtype=h.dtype), h)

  logits_train = forward(build(QM.TRAIN, QM.TRAIN), w0, w1)
  conv_layers = build(QM.CONVERT, QM.TRAIN)
  logits_conv = forward(conv_layers, w0, w1)
  assert torch.equal(logits_train, logits_conv)

  want_dtype = utils.int4 if bits == 4 else utils.int8
  expected = [('qrhs', (2, 1568, 256), (2, 1, 256)), ('qrhs', (2, 128, 10), (2, 1, 10)), ('qlhs', (2, 5, 10), (2, 1, 10))]
  saved = []
  for layer, (side, qshape, sshape) in zip(conv_layers, expected):
    v = layer.variables()
    if isinstance(layer, aqt_flax.AqtEinsum):
      v = v['aqt']['AqtDotGeneral_0'] if 'AqtDotGeneral_0' in v.get('aqt', {}) else v['aqt']
    else:
      v = v['aqt']
    assert set(v) == {side}, (set(v), side)
    qt = v[side]['frozen']
    assert tuple(qt.qvalue.shape) == qshape and [tuple(s.shape) for s in qt.scale] == [sshape]
    assert qt.scale[0].dtype == torch.float32 and qt.scale_t is None and qt.bias == []
    assert qt.dequant_dtype == torch.float32
    assert (qt.container_dtype or utils.int8) is want_dtype or qt.qvalue.dtype == want_dtype
    saved.append(layer.variables())

  serve_layers = build(QM.SERVE, QM.TRAIN)
  for layer, v in zip(serve_layers, saved):
    layer.load_variables(v)
  logits_serve = forward(serve_layers, torch.zeros_like(w0), torch.zeros_like(w1))
  assert torch.equal(logits_serve, logits_train)
  # the frozen values are what serving computes from
  broken = copy.deepcopy(saved[0])
  node = broken['aqt']['qrhs']['frozen']
  node.qvalue = torch.zeros_like(node.qvalue)
  serve_layers[0].load_variables(broken)
  assert not torch.equal(forward(serve_layers, torch.zeros_like(w0), torch.zeros_like(w1)), logits_train)


@pytest.mark.parametrize('rhs_bits', [8, 4])
def test_tiled_layer_serves_frozen_weights_through_the_grouped_kernel(gpu, rhs_bits, monkeypatch):
  """A Dense-like layer with the contraction axis in tiles of 256: training-mode forward (no
  gradient asked), conversion and serving all run the grouped-scale kernel (one launch instead of
  one contraction per tile plus a sum), serving reads the frozen weight -- an int4 one packed two
  per byte -- and all three equal the oracle's tiled dot_general bit for bit."""
  from aqt_amd import ops
  dt = 'bf16'
  m, k, n, tiles = 16, 1024, 384, 4
  x_np, w_np = U.rand((m, k), dt, 1, outliers=True), U.rand((k, n), dt, 2, 0.02)
  x, w = U.to_dev(x_np, dt, gpu), U.to_dev(w_np, dt, gpu)
  cfg = aqt.dot_general_make(8, rhs_bits)
  tiling = tiled_dot_general.Cfg(
      lhs=tiled_dot_general.TensorTiling(
          contraction_axes=[tiled_dot_general.AxisTiling(axis=1, tile_count=tiles, tile_size=None)], remaining_axes=[]),
      rhs=tiled_dot_general.TensorTiling(
          contraction_axes=[tiled_dot_general.AxisTiling(axis=0, tile_count=tiles, tile_size=None)], remaining_axes=[]))
  calls = []
  real = ops.gemm_grouped
  monkeypatch.setattr(ops, 'gemm_grouped', lambda *a, **kw: (calls.append(kw.get('b_dtype')), real(*a, **kw))[1])
  mk = lambda mode: aqt_flax.AqtDotGeneral(
      cfg, rhs_quant_mode=mode, tiling_cfg=tiling, lhs_freeze_mode=FM.CALIBRATION,
      rhs_freeze_mode=FM.CALIBRATION_AND_VALUE, use_legacy_freezer=False, rngs=_rngs())
  want, _ = R.tiled_dg_fwd(x_np, w_np, dt, k // tiles, R.dot_general_make(8, rhs_bits))
  with torch.no_grad():
    out_train = mk(QM.TRAIN)(x, w, MATMUL, None)
    conv = mk(QM.CONVERT)
    out_conv = conv(x, w, MATMUL, None)
    v = conv.variables()
    frozen = v['aqt']['qrhs']['frozen']
    assert tuple(frozen.qvalue.shape) == (tiles, k // tiles, n) and frozen.qvalue.dtype == torch.int8
    assert [tuple(s.shape) for s in frozen.scale] == [(tiles, 1, n)]
    assert (frozen.container_dtype is utils.int4) == (rhs_bits == 4)
    serve = mk(QM.SERVE)
    serve.load_variables(v)
    out_serve = serve(x, torch.zeros_like(w), MATMUL, None)
    # a checkpoint restore hands the values back in their logical order
    import copy
    v2 = copy.deepcopy(v)
    node = v2['aqt']['qrhs']['frozen']
    node.qvalue = node.qvalue.contiguous().clone()
    serve2 = mk(QM.SERVE)
    serve2.load_variables(v2)
    out_serve2 = serve2(x, torch.zeros_like(w), MATMUL, None)
  from aqt_amd import _lib as L
  assert len(calls) == 4 and calls[2] == calls[3] == (L.I4P if rhs_bits == 4 else L.I8), calls
  for out in (out_train, out_conv, out_serve, out_serve2):
    np.testing.assert_array_equal(out.float().cpu().numpy(), want)
  # with a gradient asked for, the layer takes the per-tile route and gives the same forward values
  xg = x.clone().requires_grad_(True)
  out_grad = mk(QM.TRAIN)(xg, w, MATMUL, None)
  assert len(calls) == 4
  np.testing.assert_array_equal(out_grad.detach().float().cpu().numpy(), want)

"""GPU: the standalone `quant` / `dot_general` entry points (aqt/jax/v2/pallas) over the HIP kernels.

Cases of pallas/quantizer_test.py:28-127 and pallas/dot_general_test.py:32-207, plus bit-for-bit
parity with the oracle's restatement of the same chain (Quantizer.quant with float32 scales,
_qtensor_dot_general, QTensor.dequant).
"""
import dataclasses

import numpy as np
import pytest
import torch

import aqt_amd.v2.pallas as aqt_pl
from aqt_amd.v2 import aqt_tensor
from aqt_amd.v2 import utils
from oracle import aqt_ref as R
from tests import gpu_util as U

pytestmark = pytest.mark.gpu
QTensor = aqt_tensor.QTensor
DequantMode = aqt_pl.DequantMode
MATMUL = (((1,), (0,)), ((), ()))


def _uniform(shape, dt, seed, lo=-3.0, hi=3.0):
  rng = np.random.default_rng(seed)
  return R.nm.cast((rng.random(shape, dtype=np.float32) * (hi - lo) + lo).astype(np.float32), dt)


def _oracle_quant(x_np, dt, bits, axes):
  q = R.QuantizerCfg(bits=bits, scale_dtype='f32', calib_shared_axes=None if axes is not None else 'per_tensor')
  qt = R.quantize(x_np, dt, q, axes)
  return dataclasses.replace(qt, dequant_dtype='f32')


@pytest.mark.parametrize('shape,axes,dummy,scale_shape,dt', [
    ((1024, 1024), (1,), False, (1024, 1), 'f32'),
    ((1024, 1024), (0,), False, (1, 1024), 'f32'),
    ((10, 512, 1024), (1,), False, (10, 1, 1024), 'f32'),
    ((10, 512, 1024), (2,), False, (10, 512, 1), 'f32'),
    ((1024, 1024), (0,), False, (1, 1024), 'bf16'),
    ((10, 512, 1024), (1,), False, (10, 1, 1024), 'bf16'),
    ((10, 512, 1024), (2,), False, (10, 512, 1), 'bf16'),
    ((10, 512, 1024), None, False, (1, 1, 1), 'bf16'),
    ((10, 512, 1024), None, True, (1, 1, 1), 'bf16'),
    ((10, 512, 1024), (2,), True, (10, 512, 1), 'bf16'),
])
def test_quant(gpu, shape, axes, dummy, scale_shape, dt):
  """pallas/quantizer_test.py:28-127, and the values against the oracle.  With the dummy static
  bound the reference still calibrates by abs-max (its ConstantCalibration factory is stored
  after the abs-max calibrator has been built), so the expected values are the same."""
  x_np = _uniform(shape, dt, 0)
  qx = aqt_pl.quant(U.to_dev(x_np, dt, gpu), 8, axes, dummy)
  assert tuple(qx.qvalue.shape) == shape and qx.qvalue.dtype == torch.int8
  assert tuple(qx.scale[0].shape) == scale_shape
  assert qx.scale[0].dtype == torch.float32  # whatever the dtype of x
  assert qx.dequant_dtype == torch.float32
  want = _oracle_quant(x_np, dt, 8, axes)
  np.testing.assert_array_equal(qx.scale[0].cpu().numpy(), want.scale[0])
  np.testing.assert_array_equal(qx.qvalue.cpu().numpy(), want.qvalue)


@pytest.mark.parametrize('mkn', [(512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048)])
@pytest.mark.parametrize('quantize_lhs', [True, False])
@pytest.mark.parametrize('quantize_rhs', [True, False])
@pytest.mark.parametrize('quant_type', [4, 8, 'e4m3', 'e5m2'])
def test_quantized_matmul_error(gpu, mkn, quantize_lhs, quantize_rhs, quant_type):
  """pallas/dot_general_test.py:32-137 (without the Pallas blocking: whole tensors; the same data
  distribution and the same error bounds)."""
  m, k, n = mkn
  lhs = torch.from_numpy(np.random.default_rng(0).random((m, k), dtype=np.float32)).to(gpu)
  rhs = torch.from_numpy(np.random.default_rng(0).random((k, n), dtype=np.float32)).to(gpu)
  ql = aqt_pl.quant(lhs, n_bits=quant_type, calibration_axes=(1,)) if quantize_lhs else lhs
  qr = aqt_pl.quant(rhs, n_bits=quant_type, calibration_axes=(0,)) if quantize_rhs else rhs
  if isinstance(ql, QTensor):
    ql = aqt_pl.load_qtensor(ql)
  out = aqt_pl.dot_general(ql, qr, dimension_numbers=MATMUL)
  assert out.dtype == torch.float32
  ref = lhs.double() @ rhs.double()
  rel = ((out.double() - ref).abs() / ref.abs()).max().item()
  bound = 1e-6 * 10  # float32 sum of k terms against float64
  if quantize_lhs or quantize_rhs:
    bound = 1e-2 if quant_type == 8 else 0.1
  assert rel < bound, rel


@pytest.mark.parametrize('lhs_axes,rhs_axes,lhs_mode,rhs_mode', [
    ((1,), (0,), DequantMode.OUTPUT, DequantMode.OUTPUT),
    ((1,), (0,), DequantMode.THIS_INPUT, DequantMode.OUTPUT),
    ((1,), (0,), DequantMode.OUTPUT, DequantMode.THIS_INPUT),
    ((0,), None, DequantMode.OTHER_INPUT, DequantMode.OUTPUT),
    (None, (1,), DequantMode.OUTPUT, DequantMode.OTHER_INPUT),
])
def test_dequantization_location(gpu, lhs_axes, rhs_axes, lhs_mode, rhs_mode):
  """pallas/dot_general_test.py:139-203 (all-zero operands; the call passing is the test), and on
  random operands the values of each placement against the oracle."""
  for fill in ('zeros', 'random'):
    if fill == 'zeros':
      l_np, r_np = np.zeros((2048, 512), np.float32), np.zeros((512, 2048), np.float32)
    else:
      l_np, r_np = _uniform((256, 512), 'f32', 1), _uniform((512, 384), 'f32', 2)
    lhs, rhs = U.to_dev(l_np, 'f32', gpu), U.to_dev(r_np, 'f32', gpu)
    lq = aqt_pl.quant(lhs, n_bits=8, calibration_axes=lhs_axes) if lhs_axes is not None else lhs
    rq = aqt_pl.quant(rhs, n_bits=8, calibration_axes=rhs_axes) if rhs_axes is not None else rhs
    out = aqt_pl.dot_general(lq, rq, dimension_numbers=MATMUL, lhs_dequant_mode=lhs_mode, rhs_dequant_mode=rhs_mode)
    assert out.dtype == torch.float32 and tuple(out.shape) == (l_np.shape[0], r_np.shape[1])
    if fill == 'zeros':
      assert not out.any()
      continue
    plain = lambda a: R.QTensor(a, 'f32', [], None, 'f32')
    lo = _oracle_quant(l_np, 'f32', 8, lhs_axes) if lhs_axes is not None else plain(l_np)
    ro = _oracle_quant(r_np, 'f32', 8, rhs_axes) if rhs_axes is not None else plain(r_np)
    both = lhs_axes is not None and rhs_axes is not None
    if not both:  # the quantized side meets a float operand as floats (pallas/dot_general.py:89-95)
      if lhs_axes is not None:
        lo = dataclasses.replace(lo, qvalue=lo.qvalue.astype(np.float32), qdtype='f32')
      if rhs_axes is not None:
        ro = dataclasses.replace(ro, qvalue=ro.qvalue.astype(np.float32), qdtype='f32')
    names = {DequantMode.OUTPUT: 'output', DequantMode.THIS_INPUT: 'this_input', DequantMode.OTHER_INPUT: 'other_input'}
    output_only = lhs_mode == DequantMode.OUTPUT and rhs_mode == DequantMode.OUTPUT
    raw = R.RawCfg(lhs=R.QuantizerCfg(bits=8 if lhs_axes is not None else None),
                   rhs=R.QuantizerCfg(bits=8 if rhs_axes is not None else None),
                   lhs_dequant_mode=names[lhs_mode], rhs_dequant_mode=names[rhs_mode],
                   acc='auto' if output_only else None)
    want = R.dequant(R.qtensor_dot_general(lo, ro, MATMUL, raw, 'f32'))
    got = out.cpu().numpy()
    if both and output_only:
      np.testing.assert_array_equal(got, want)  # integer accumulators: bit for bit
    else:
      # float contraction: the summation order is the library's; float32 tolerance over k = 512
      np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-4)


@pytest.mark.parametrize('bits', [8, 4, 'e4m3'])
@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('m,lhs_axes', [(96, (1,)), (8, (1,)), (96, None)])
def test_dot_general_of_two_qtensors_matches_the_oracle(gpu, bits, dt, m, lhs_axes):
  """quant -> dot_general with both operands quantized: the fused contraction + dequantisation
  against the oracle's quant / _qtensor_dot_general / dequant, integers bit for bit (per-row and
  per-tensor lhs scales, a decode-sized lhs)."""
  k, n = 1024, 320
  l_np, r_np = U.rand((m, k), dt, 3, outliers=True), U.rand((k, n), dt, 4, 0.02)
  lq = aqt_pl.quant(U.to_dev(l_np, dt, gpu), bits, lhs_axes)
  rq = aqt_pl.quant(U.to_dev(r_np, dt, gpu), bits, (0,))
  if bits == 4:
    assert lq.container_dtype is utils.int4 and rq.qvalue.dtype == torch.int8
  out = aqt_pl.dot_general(lq, rq, MATMUL)
  assert out.dtype == torch.float32
  lo, ro = _oracle_quant(l_np, dt, bits, lhs_axes), _oracle_quant(r_np, dt, bits, (0,))
  for got_qt, want_qt in ((lq, lo), (rq, ro)):  # quantized values and scales: bit for bit, fp8 too
    np.testing.assert_array_equal(got_qt.qvalue.float().cpu().numpy(), np.asarray(want_qt.qvalue, np.float32))
    np.testing.assert_array_equal(got_qt.scale[0].cpu().numpy(), want_qt.scale[0])
  raw = R.RawCfg(lhs=R.QuantizerCfg(bits=bits), rhs=R.QuantizerCfg(bits=bits))
  want = R.dequant(R.qtensor_dot_general(lo, ro, MATMUL, raw, 'f32'))
  if isinstance(bits, int):
    np.testing.assert_array_equal(out.cpu().numpy(), want)
  else:
    # fp8 products accumulate in float32 in the matrix core's order and alignment (the oracle sums
    # exactly and rounds once: summation order is parity unpinned); measured gap 3e-5 relative
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=2e-4, atol=2e-4 * np.abs(want).max())
  # preferred_element_type picks the result dtype
  out_bf = aqt_pl.dot_general(lq, rq, MATMUL, preferred_element_type=torch.bfloat16)
  assert out_bf.dtype == torch.bfloat16
  if isinstance(bits, int):
    # QTensor.dequant rounds the accumulator to bf16 before the float32 scales multiply it
    want_bf = R.dequant(R.qtensor_dot_general(lo, ro, MATMUL, raw, 'bf16'))
    np.testing.assert_array_equal(out_bf.float().cpu().numpy(), want_bf)
  # the given QTensors are not modified
  assert lq.qvalue.dtype in (torch.int8, torch.float8_e4m3fn)


def test_two_qtensors_take_the_fused_contraction(gpu, monkeypatch):
  """Both operands quantized, output dequantisation: one contraction launch with both scale
  vectors in its epilogue, no separate dequantize step."""
  from aqt_amd import ops
  calls = []
  real = ops.gemm
  monkeypatch.setattr(ops, 'gemm', lambda *a, **kw: (calls.append(kw), real(*a, **kw))[1])
  lq = aqt_pl.quant(torch.randn(128, 256, device=gpu), 8, (1,))
  rq = aqt_pl.quant(torch.randn(256, 64, device=gpu), 8, (0,))
  aqt_pl.dot_general(lq, rq, MATMUL)
  assert len(calls) == 1 and calls[0]['row_scale'] is not None and calls[0]['col_scale'] is not None
  assert calls[0]['out_dtype'] == torch.float32


def test_pallas_call_is_not_offered():
  with pytest.raises(NotImplementedError, match='no Pallas'):
    aqt_pl.pallas_call(lambda: None)

"""aqtx_scale_cast (the pass that makes the operands of a float contraction and scales its result) against
the oracle's QTensor.dequant and the reference's OTHER_INPUT product, bit for bit.

QTensor.dequant: the value is cast to the dequant dtype, then multiplied scale by scale, each product in the
promoted dtype of its factors, then cast once more (aqt_tensor.py:179-199).  OTHER_INPUT: the operand, already
in its own dtype, times the scale cast to that dtype (aqt_dot_general.py:887-903)."""
import numpy as np
import pytest
import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from oracle import aqt_ref as R
from oracle import numerics as nm
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

TORCH_DT = {'f32': torch.float32, 'bf16': torch.bfloat16}


def _input(kind, shape, seed):
  """(device tensor builder, float32 values, oracle qdtype, kernel dtype)."""
  rng = np.random.default_rng(seed)
  if kind == 'i8':
    q = rng.integers(-127, 128, shape).astype(np.int8)
    return (lambda dev: torch.from_numpy(q).to(dev)), q.astype(np.float32), 'i8', L.I8
  if kind in ('e4m3', 'e5m2'):
    b = rng.integers(0, 256, shape).astype(np.uint8)
    if kind == 'e4m3':
      b = np.where((b & 0x7F) == 0x7F, np.uint8(0x3C), b)  # no NaN patterns
    else:
      b = np.where((b & 0x7C) == 0x7C, np.uint8(0x3C), b)  # no inf / NaN patterns
    return (lambda dev: torch.from_numpy(b).to(dev)), U.fp8_bytes_to_float(b, kind), kind, L.E4M3 if kind == 'e4m3' else L.E5M2
  x = nm.cast(rng.standard_normal(shape).astype(np.float32) * np.float32(3.0), kind)
  return (lambda dev: U.to_dev(x, kind, dev)), x, kind, None


def _factor(rng, n, dt):
  return nm.cast((rng.random(n).astype(np.float32) * np.float32(0.02) + np.float32(1e-3)), dt)


def _want(x, out_dt, factors, shape):
  b, r, c = shape
  v, vdt = nm.cast(x, out_dt), out_dt
  for f, axis, fdt, recast in factors:
    if recast:
      v, vdt = nm.cast(v, out_dt), out_dt
    fb = np.broadcast_to(f.reshape(-1, r if axis == L.FACTOR_ROWS else c), (b, r if axis == L.FACTOR_ROWS else c))
    fb = fb[:, :, None] if axis == L.FACTOR_ROWS else fb[:, None, :]
    vdt = nm.promote(vdt, fdt)
    v = nm.cast(v * fb, vdt)
  return nm.cast(v, out_dt)


FACTORS = {
    'none': [],
    'rows_f32': [('rows', 'f32', False, True)],
    'rows_bf16': [('rows', 'bf16', False, True)],
    'cols_bf16_shared': [('cols', 'bf16', False, False)],
    'rows_then_cols_recast': [('rows', 'bf16', False, True), ('cols', 'same', True, True)],
    'rows_f32_then_cols_recast': [('rows', 'f32', False, True), ('cols', 'same', True, False)],
    'rows_and_cols': [('rows', 'bf16', False, True), ('cols', 'f32', False, True)],
}


@pytest.mark.parametrize('shape', [(1, 48, 96), (3, 20, 64), (2, 7, 40), (1, 1, 16), (2, 33, 1)])
@pytest.mark.parametrize('fname', list(FACTORS))
@pytest.mark.parametrize('out_dt', ['bf16', 'f32'])
@pytest.mark.parametrize('kind', ['i8', 'e4m3', 'e5m2', 'bf16', 'f32'])
def test_scale_cast_matches_the_elementwise_steps(gpu, kind, out_dt, fname, shape):
  b, r, c = shape
  make, x, _, kdt = _input(kind, shape, 1)
  rng = np.random.default_rng(2)
  factors, dev_factors = [], []
  for axis_name, fdt, recast, per_batch in FACTORS[fname]:
    axis = L.FACTOR_ROWS if axis_name == 'rows' else L.FACTOR_COLS
    fdt = out_dt if fdt == 'same' else fdt
    n = (r if axis == L.FACTOR_ROWS else c) * (b if per_batch else 1)
    f = _factor(rng, n, fdt)
    factors.append((f, axis, fdt, recast))
    dev_factors.append((torch.from_numpy(f).to(gpu), axis, TORCH_DT[fdt], recast))
  got = ops.scale_cast(make(gpu), dev_factors, out_dtype=TORCH_DT[out_dt], in_dtype=kdt)
  assert got.dtype == TORCH_DT[out_dt] and tuple(got.shape) == shape
  np.testing.assert_array_equal(got.float().cpu().numpy(), _want(x, out_dt, factors, shape))


@pytest.mark.parametrize('dd,sdts', [('bf16', ['bf16']), ('bf16', ['f32']), ('f32', ['f32']), ('bf16', ['bf16', 'f32']),
                                     ('bf16', ['f32', 'bf16'])])
@pytest.mark.parametrize('kind', ['i8', 'e4m3'])
def test_scale_cast_is_qtensor_dequant(gpu, kind, dd, sdts):
  """One and two scales (a per-row one, then a per-column one) through the oracle's QTensor.dequant."""
  shape = (2, 24, 80)
  b, r, c = shape
  make, x, qdtype, kdt = _input(kind, shape, 3)
  rng = np.random.default_rng(4)
  scales, dev = [], []
  for i, sdt in enumerate(sdts):
    n, axis = (r, L.FACTOR_ROWS) if i == 0 else (c, L.FACTOR_COLS)
    f = _factor(rng, b * n, sdt)
    scales.append(f.reshape(b, n, 1) if i == 0 else f.reshape(b, 1, n))
    dev.append((torch.from_numpy(f).to(gpu), axis, TORCH_DT[sdt], False))
  qv = x.astype(np.int32) if kind == 'i8' else x
  want = R.dequant(R.QTensor(qv, qdtype, scales, None, dd, scale_dtypes=list(sdts)))
  got = ops.scale_cast(make(gpu), dev, out_dtype=TORCH_DT[dd], in_dtype=kdt)
  np.testing.assert_array_equal(got.float().cpu().numpy(), want)


def test_dequantize_entry_point_takes_the_same_kernel(gpu):
  """aqtx_dequantize with q in the order of the result (one scale per row, per column, per tensor) against
  the oracle's QTensor.dequant."""
  shape = (2, 40, 96)
  b, r, c = shape
  make, x, _, _ = _input('i8', shape, 5)
  rng = np.random.default_rng(6)
  for reduce, sshape in ((L.REDUCE_COLS, (b, r, 1)), (L.REDUCE_ROWS, (b, 1, c)), (L.REDUCE_ALL, (b, 1, 1)),
                         (L.REDUCE_ALL_BATCH, (1, 1, 1))):
    for dd, sdt in (('bf16', 'bf16'), ('bf16', 'f32'), ('f32', 'f32')):
      f = _factor(rng, int(np.prod(sshape)), sdt)
      want = R.dequant(R.QTensor(x.astype(np.int32), 'i8', [f.reshape(sshape)], sdt, dd))
      got = ops.dequantize(make(gpu), torch.from_numpy(f).to(gpu), reduce=reduce, q_dtype=L.I8, out_dtype=TORCH_DT[dd],
                           scale_dtype=TORCH_DT[sdt])
      np.testing.assert_array_equal(got.float().cpu().numpy(), want)


@pytest.mark.parametrize('shape', [(2, 24, 80), (1, 7, 40)])
@pytest.mark.parametrize('axis', ['rows', 'cols'])
@pytest.mark.parametrize('dt,sdt', [('bf16', 'bf16'), ('bf16', 'f32'), ('f32', 'f32'), ('f32', 'bf16')])
@pytest.mark.parametrize('kw', [dict(round=False), dict(clip=False), dict(clip=False, round=False),
                                dict(preserve_zero=False), dict(bits=1, preserve_zero=False),
                                dict(preserve_zero=False, round=False), dict()])
def test_reciprocal_factor_and_finish_are_quant_and_int_numerics(gpu, kw, dt, sdt, axis, shape):
  """QTensor.quant (multiply by the reciprocal scale, 1 where it is infinite) followed by IntSymmetric.vjp_fwd
  without noise and with the values kept in the float dtype, against the oracle's two functions: settings whose
  results are not integers included.  One scale per row or per column; a zero and a tiny scale reach the
  infinite-reciprocal rule."""
  b, r, c = shape
  q = R.QuantizerCfg(**{'bits': 8, 'keep_float': True, **kw})
  rng = np.random.default_rng(7)
  x = nm.cast(rng.standard_normal(shape).astype(np.float32) * np.float32(40.0), dt)
  n = r if axis == 'rows' else c
  s = _factor(rng, b * n, sdt) * np.float32(20.0)
  s[0], s[1] = np.float32(0.0), nm.cast(np.full(1, 1e-39, np.float32), sdt)[0]
  sc = s.reshape(b, n, 1) if axis == 'rows' else s.reshape(b, 1, n)
  with np.errstate(over='ignore', divide='ignore'):
    v, vdt = R.qtensor_quant(x, dt, [sc], sdt)
  want, wdt = R.int_vjp_fwd(v, vdt, q)
  assert wdt == vdt
  got = ops.scale_cast(U.to_dev(x, dt, gpu), [(torch.from_numpy(s).to(gpu), L.FACTOR_ROWS if axis == 'rows' else L.FACTOR_COLS,
                                               TORCH_DT[sdt], False, True)],
                       out_dtype=TORCH_DT[vdt], finish_clip=R.int_clip_bound(q) if q.clip else None,
                       finish_round=0 if not q.round else 1 if q.preserve_zero else 2)
  np.testing.assert_array_equal(got.float().cpu().numpy(), want)

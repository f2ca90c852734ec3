"""GPU parity: aqtx_quantize / aqtx_random_bits against the numpy oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from oracle import aqt_ref as R
from oracle import numerics as nm
from oracle import prng
from tests import gpu_util as U

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('partitionable', [False, True])
@pytest.mark.parametrize('width', [16, 32])
@pytest.mark.parametrize('n', [1, 2, 7, 4096, 100003])
def test_random_bits(gpu, n, width, partitionable):
  key = prng.prng_key(42)
  got = ops.random_bits(key, n, width, partitionable, device=gpu).cpu().numpy()
  got = got.view(np.uint16 if width == 16 else np.uint32)
  want = prng.random_bits(key, (n,), width, partitionable)
  np.testing.assert_array_equal(got, want)


def test_prng_split_host():
  for part in (False, True):
    for num in (1, 2, 3, 5):
      np.testing.assert_array_equal(ops.prng_split(prng.prng_key(7), num, part),
                                    prng.split(prng.prng_key(7), num, part))


def _oracle_quant(x, dt, q, axes, prescale=None, ps_axis=None):
  if prescale is not None:
    shape = [1] * x.ndim
    shape[ps_axis] = x.shape[ps_axis]
    x = nm.cast(x * nm.cast(prescale.reshape(shape), dt), dt)
  return R.quantize(x, dt, q, axes)


def _check(qt, q_got, s_got, cfg, transpose=False):
  want_q = qt.qvalue
  if cfg.is_fp8():
    got = U.fp8_bytes_to_float(q_got, cfg.bits)
  else:
    got = q_got.astype(np.float32)
    want_q = want_q.astype(np.float32)
  if transpose:
    got = np.swapaxes(got, -1, -2)
  np.testing.assert_array_equal(s_got.reshape(-1), qt.scale[0].reshape(-1))
  np.testing.assert_array_equal(got, want_q)


ROW_CASES = [
    # (rows, cols, group)
    (4, 64, 0), (33, 128, 0), (5, 512, 0), (3, 2048, 0), (7, 4096, 0), (2, 8192, 0),
    (2, 14336, 0), (3, 100, 0), (2, 20000, 0), (6, 1024, 128), (3, 96, 32),
    # few long rows: taken as one scale per batch entry of [batch * rows][cols / c][c]
    (3, 32768, 0), (5, 16448, 0), (2, 401408, 0), (1, 16384, 0),
]


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('rows,cols,group', ROW_CASES)
def test_rows_int8_rtn(gpu, rows, cols, group, dt):
  x = U.rand((2, rows, cols), dt, seed=rows * 131 + cols, outliers=True)
  x[0, 0, :] = 0.0  # an all-zero row: abs-max 0 -> scale 1/127.5 path (calibration.py:148)
  q = R.QuantizerCfg(bits=8)
  if group:
    xv = x.reshape(2, rows, cols // group, group)
    qt = R.quantize(xv, dt, q, [3])
  else:
    qt = R.quantize(x, dt, q, [2])
  qb, cb = U.bounds(q)
  qg, sg = ops.quantize(U.to_dev(x, dt, gpu), reduce=L.REDUCE_COLS, out_dtype=L.I8,
                        quant_bound=qb, clip_bound=cb, group=group)
  got = qg.cpu().numpy()
  if group:
    got = got.reshape(2, rows, cols // group, group)
  _check(qt, got, sg.cpu().numpy(), q)


@pytest.mark.parametrize('bits,noise,scale_dtype', [
    (8, 'jax.uniform', None), (8, 'custom-1', None), (4, None, None), (4, 'jax.uniform', 'f32'),
    ('e4m3', None, None), ('e5m2', None, None), ('e4m3', 'sr', None), ('e5m2', 'sr', None),
    ('e5m2', 'sr', 'f32'), (8, None, 'f32'),
])
@pytest.mark.parametrize('partitionable', [False, True])
@pytest.mark.parametrize('dt', ['bf16', 'f32'])
def test_rows_numerics(gpu, bits, noise, scale_dtype, partitionable, dt, monkeypatch):
  monkeypatch.setattr(R, 'PARTITIONABLE', partitionable)
  rows, cols = 9, 1000 if noise else 256
  x = U.rand((1, rows, cols), dt, seed=5, scale=0.02)
  key = prng.prng_key(1234)
  q = R.QuantizerCfg(bits=bits, scale_dtype=scale_dtype, key=key)
  knoise = L.NOISE_NONE
  if noise == 'sr':
    q.fp8_sr = True
    knoise = L.NOISE_FP8_MANTISSA
  elif noise:
    q.noise = noise
    knoise = U.NOISE[noise]
  qt = R.quantize(x, dt, q, [2])
  qb, cb = U.bounds(q)
  qg, sg = ops.quantize(U.to_dev(x, dt, gpu), reduce=L.REDUCE_COLS, out_dtype=U.OUT_DT[bits],
                        quant_bound=qb, clip_bound=cb, noise=knoise, key=key,
                        partitionable=partitionable,
                        scale_dtype=U.TORCH_DT[scale_dtype] if scale_dtype else None)
  _check(qt, qg.cpu().numpy(), sg.cpu().numpy(), q)


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('rows,cols,group,transpose', [
    (128, 64, 0, True), (300, 200, 0, True), (256, 520, 0, False), (77, 13, 0, True),
    (77, 13, 0, False), (512, 256, 128, True), (256, 64, 32, False), (1024, 1024, 0, True),
])
def test_cols_int8(gpu, rows, cols, group, transpose, dt):
  x = U.rand((2, rows, cols), dt, seed=rows + cols, outliers=True)
  x[:, :, 1] = 0.0
  key = prng.prng_key(99)
  q = R.QuantizerCfg(bits=8, noise='jax.uniform', key=key)
  if group:
    qt = R.quantize(x.reshape(2, rows // group, group, cols), dt, q, [2])
    want_q = qt.qvalue.reshape(2, rows, cols)
    # noise index is the row-major index of the [2, rows/group, group, cols] tensor = same memory order
  else:
    qt = R.quantize(x, dt, q, [1])
    want_q = qt.qvalue
  qb, cb = U.bounds(q)
  qg, sg = ops.quantize(U.to_dev(x, dt, gpu), reduce=L.REDUCE_ROWS, out_dtype=L.I8,
                        quant_bound=qb, clip_bound=cb, group=group, transpose_out=transpose,
                        noise=L.NOISE_JAX_UNIFORM, key=key)
  got = qg.cpu().numpy()
  if transpose:
    got = np.swapaxes(got, 1, 2)
  np.testing.assert_array_equal(sg.cpu().numpy().reshape(-1), qt.scale[0].reshape(-1))
  np.testing.assert_array_equal(got, want_q)


@pytest.mark.parametrize('bits', [8, 'e4m3', 'e5m2'])
@pytest.mark.parametrize('dt', ['bf16', 'f32'])
def test_per_tensor(gpu, bits, dt):
  x = U.rand((3, 130, 72), dt, seed=3)
  q = R.QuantizerCfg(bits=bits, calib_shared_axes=None)
  qb, cb = U.bounds(q)
  qg, sg = ops.quantize(U.to_dev(x, dt, gpu), reduce=L.REDUCE_ALL, out_dtype=U.OUT_DT[bits],
                        quant_bound=qb, clip_bound=cb)
  qt = R.quantize(x, dt, q, [1, 2])  # one scale per batch entry
  _check(qt, qg.cpu().numpy(), sg.cpu().numpy(), q)


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
def test_prescale_and_requant(gpu, dt):
  """The two bwd-side uses: g * other-side scale, and re-quantizing int8 residuals."""
  m, n = 96, 256
  g = U.rand((1, m, n), dt, seed=11, scale=1e-3)
  col_ps = nm.cast(np.abs(U.rand((n,), 'f32', 12, 6e-4)) + np.float32(1e-5), dt)
  row_ps = nm.cast(np.abs(U.rand((m,), 'f32', 13, 0.03)) + np.float32(1e-3), dt)
  key = prng.prng_key(5)
  q = R.QuantizerCfg(bits=8, noise='jax.uniform', key=key)
  qb, cb = U.bounds(q)
  gd = U.to_dev(g, dt, gpu)
  # dlhs: per-column prescale, row-wise scales
  qt = _oracle_quant(g, dt, q, [2], col_ps, 2)
  qg, sg = ops.quantize(gd, reduce=L.REDUCE_COLS, out_dtype=L.I8, quant_bound=qb, clip_bound=cb,
                        noise=L.NOISE_JAX_UNIFORM, key=key,
                        prescale=torch.from_numpy(col_ps).to(gpu), prescale_mode=L.PRESCALE_PER_COL)
  _check(qt, qg.cpu().numpy(), sg.cpu().numpy(), q)
  # drhs: per-row prescale, column-wise scales, transposed write
  qt = _oracle_quant(g, dt, q, [1], row_ps, 1)
  qg, sg = ops.quantize(gd, reduce=L.REDUCE_ROWS, out_dtype=L.I8, quant_bound=qb, clip_bound=cb,
                        noise=L.NOISE_JAX_UNIFORM, key=key, transpose_out=True,
                        prescale=torch.from_numpy(row_ps).to(gpu), prescale_mode=L.PRESCALE_PER_ROW)
  _check(qt, qg.cpu().numpy(), sg.cpu().numpy(), q, transpose=True)
  # residual re-quantization: int8 input in a [n, k] buffer standing for a logical [k, n] tensor
  k = 128
  w_q = np.random.default_rng(3).integers(-127, 128, size=(k, n)).astype(np.int8)  # logical [k, n]
  qt = R.quantize(w_q.astype(np.float32)[None], dt, q, [2])  # per-k scale over n
  mem = torch.from_numpy(np.ascontiguousarray(w_q.T)[None]).to(gpu)  # memory [1, n, k]
  qg, sg = ops.quantize(mem, reduce=L.REDUCE_ROWS, out_dtype=L.I8, quant_bound=qb, clip_bound=cb,
                        compute_dtype=U.TORCH_DT[dt], noise=L.NOISE_JAX_UNIFORM, key=key,
                        transpose_out=True, noise_strides=(k * n, 1, n), noise_total=k * n)
  np.testing.assert_array_equal(sg.cpu().numpy().reshape(-1), qt.scale[0].reshape(-1))
  np.testing.assert_array_equal(qg.cpu().numpy(), qt.qvalue)  # transposed write -> [1, k, n]


@pytest.mark.parametrize('kind', ['e4m3', 'e5m2'])
def test_fp8_cast_exhaustive(gpu, kind):
  """Every finite bf16 value through clip + fp8 cast (scale fixed to 1)."""
  bits = np.arange(65536, dtype=np.uint32)
  x = (bits << np.uint32(16)).astype(np.uint32).view(np.float32).copy()
  x[~np.isfinite(x)] = 0.0
  x = x.reshape(1, 64, 1024)
  q = R.QuantizerCfg(bits=kind)
  b = np.float32(R.quant_bound(q))
  want = (nm.to_e4m3fn if kind == 'e4m3' else nm.to_e5m2)(np.clip(x, -b, b))
  ones = torch.ones((1, 64, 1), dtype=torch.float32, device=gpu)
  qg, _ = ops.quantize(U.to_dev(x, 'bf16', gpu), reduce=L.REDUCE_COLS, out_dtype=U.OUT_DT[kind],
                       quant_bound=float(b), clip_bound=float(b), scale=ones)
  got = U.fp8_bytes_to_float(qg.cpu().numpy(), kind)
  np.testing.assert_array_equal(got, want)
  # signed zero / sign of tiny values must survive as well
  np.testing.assert_array_equal(np.signbit(got), np.signbit(want))


def test_workspace_kept_across_calls(gpu):
  """The abs-max workspace is shared by successive calls and handed back zeroed: calls with
  many, few, and again many scales, column-wise and per tensor, give what a first call gives."""
  from aqt_amd import _lib as L
  rng = np.random.default_rng(5)
  xs = [torch.from_numpy(rng.standard_normal(s).astype(np.float32)).to(torch.bfloat16).to(gpu)
        for s in ((1, 96, 4096), (1, 64, 24), (2, 40, 1000), (1, 128, 8192))]
  kw = dict(out_dtype=L.I8, quant_bound=127.5, clip_bound=127.0)
  first = {}
  for rnd in range(3):
    for i, x in enumerate(xs):
      for reduce in (L.REDUCE_ROWS, L.REDUCE_ALL_BATCH):
        q, s = ops.quantize(x, reduce=reduce, **kw)
        if rnd == 0:
          amax = x.float().abs().amax(dim=1) if reduce == L.REDUCE_ROWS else x.float().abs().amax().reshape(1)
          want = (amax / 127.5).to(torch.bfloat16).float()
          assert torch.equal(s.reshape(-1), want.reshape(-1))
          first[(i, reduce)] = (q.clone(), s.clone())
        else:
          assert torch.equal(q, first[(i, reduce)][0]) and torch.equal(s, first[(i, reduce)][1])


@pytest.mark.parametrize('noise', ['jax.uniform', 'custom-1'])
@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('batch,rows,cols', [(1, 4, 32768), (2, 3, 16448), (3, 1, 65536)])
def test_few_long_rows_stochastic_rounding(gpu, batch, rows, cols, noise, dt):
  """The few-long-rows form with noise: the counters of [batch, rows, cols] carry over to the
  per-batch-entry form, and a scale handed in is used the same way."""
  x = U.rand((batch, rows, cols), dt, seed=cols + rows, scale=0.3)
  key = prng.prng_key(77)
  q = R.QuantizerCfg(bits=8, key=key, noise=noise)
  qt = R.quantize(x, dt, q, [2])
  qb, cb = U.bounds(q)
  qg, sg = ops.quantize(U.to_dev(x, dt, gpu), reduce=L.REDUCE_COLS, out_dtype=L.I8, quant_bound=qb, clip_bound=cb,
                        noise=U.NOISE[noise], key=key)
  _check(qt, qg.cpu().numpy(), sg.cpu().numpy(), q)
  qg2, _ = ops.quantize(U.to_dev(x, dt, gpu), reduce=L.REDUCE_COLS, out_dtype=L.I8, quant_bound=qb, clip_bound=cb,
                        noise=U.NOISE[noise], key=key, scale=sg.clone())
  assert torch.equal(qg, qg2)


@pytest.mark.parametrize('reduce,transpose,shape', [
    (L.REDUCE_COLS, False, (1, 64, 1024)),   # rows kernel, rows paired over one threefry block
    (L.REDUCE_COLS, False, (2, 9, 1000)),    # rows kernel, plain
    (L.REDUCE_COLS, False, (1, 5, 1001)),    # generic rows kernel
    (L.REDUCE_ROWS, True, (1, 256, 192)),    # tile kernel, transposed write
    (L.REDUCE_ALL, False, (2, 130, 70)),     # tile kernel, one scale per batch entry
])
@pytest.mark.parametrize('noise,out', [(L.NOISE_JAX_UNIFORM, L.I8), (L.NOISE_FP8_MANTISSA, L.E5M2)])
def test_key_in_device_memory_equals_key_in_the_plan(gpu, reduce, transpose, shape, noise, out):
  """plan.key_device: the kernels read the two key words from device memory (the form a traced
  jax key arrives in under XLA); same bits as the key given by value."""
  x = U.to_dev(U.rand(shape, 'bf16', seed=7, scale=0.5), 'bf16', gpu)
  key = prng.prng_key(4321)
  qb, cb = (127.5, 127.0) if out == L.I8 else (57344.0, 57344.0)
  kw = dict(reduce=reduce, out_dtype=out, quant_bound=qb, clip_bound=cb, noise=noise, transpose_out=transpose)
  q0, s0 = ops.quantize(x, key=key, **kw)
  kd = torch.tensor([int(key[0]), int(key[1])], dtype=torch.int64).to(torch.int32).to(gpu) if max(key) < 2**31 else \
      torch.from_numpy(np.asarray(key, dtype=np.uint32).view(np.int32).copy()).to(gpu)
  q1, s1 = ops.quantize(x, key_device=kd, **kw)
  assert torch.equal(q0, q1) and torch.equal(s0, s1)
  # and a different key gives different bits (the device key is really what is read)
  kd2 = kd.clone()
  kd2[1] += 1
  q2, _ = ops.quantize(x, key_device=kd2, **kw)
  assert not torch.equal(q0, q2)


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('reduce,shape', [
    (L.REDUCE_COLS, (2, 9, 1024)), (L.REDUCE_COLS, (1, 3, 1001)), (L.REDUCE_ROWS, (1, 200, 96)),
    (L.REDUCE_ALL, (3, 40, 64)),
])
def test_nan_reaches_the_scale(gpu, dt, reduce, shape):
  """jnp.max(jnp.abs(x)) propagates a NaN into the scale (calibration.py:126-157), which is how a
  diverged step shows up in the outputs; the kernels' abs-max does the same, and the scales of
  segments without a NaN are untouched."""
  x = U.rand(shape, dt, seed=11)
  x[0, 1, 5] = np.nan
  q = R.QuantizerCfg(bits=8)
  axes = {L.REDUCE_COLS: [2], L.REDUCE_ROWS: [1], L.REDUCE_ALL: [1, 2]}[reduce]
  with np.errstate(invalid='ignore'):
    want = R.quantize(x, dt, q, axes).scale[0].reshape(-1)
  _, sg = ops.quantize(U.to_dev(x, dt, gpu), reduce=reduce, out_dtype=L.I8, quant_bound=127.5, clip_bound=127.0)
  got = sg.cpu().numpy().reshape(-1)
  assert np.isnan(want).sum() == 1
  np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
  np.testing.assert_array_equal(got[~np.isnan(want)], want[~np.isnan(want)])


def test_nan_row_gives_nan_outputs(gpu):
  """End to end: one NaN activation makes exactly that token's outputs NaN (its scale is NaN), in
  the training-shape path and in the serving kernels."""
  from aqt_amd.v2 import aqt_dot_general as aqt
  from aqt_amd.v2 import config
  lhs = torch.randn(48, 256, device=gpu).to(torch.bfloat16)
  rhs = (torch.randn(256, 64, device=gpu) * 0.05).to(torch.bfloat16)
  lhs[7, 100] = float('nan')
  cfg = config.set_context(config.fully_quantized(fwd_bits=8, bwd_bits=8, use_stochastic_rounding=False), None, None)
  out, _ = cfg.dg_core(lhs, rhs, None, None, (((1,), (0,)), ((), ())))
  bad = torch.isnan(out).any(dim=1).cpu().numpy()
  assert bad[7] and bad.sum() == 1 and bool(torch.isnan(out[7]).all())
  wq = torch.randint(-127, 128, (64, 256), dtype=torch.int8, device=gpu)
  ws = torch.rand(64, device=gpu) * 1e-3
  for m in (2, 48):
    o, xs = ops.decode(lhs[6:6 + m].contiguous(), wq, ws, quant_bound=127.5, clip_bound=127.0)
    assert bool(torch.isnan(xs[1])) and bool(torch.isnan(o[1]).all()) and not bool(torch.isnan(o[0]).any())

"""The benchmark configuration at its full size (bf16 [8192, 4096] x [4096, 14336], forward and
backward, int8): the product runs the whole problem, the oracle restates slices of it.

What makes slices exact: the forward quantizes the lhs per row and the rhs per column, so
out[rows] needs lhs[rows] and the whole rhs only; dlhs[rows] needs g[rows] (quantized per row
over N) and the whole rhs residual; drhs[:, cols] needs g[:, cols] (quantized per column over M)
and the whole lhs residual.  Stochastic-rounding noise is drawn for the whole gradient tensor;
the oracle reads it at the positions of the slice (QuantizerCfg.noise_window).
"""
import copy

import numpy as np
import pytest
import torch

from oracle import aqt_ref as R
from oracle import numerics as nm
from oracle import prng
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

M, K, N = 8192, 4096, 14336
MATMUL = (((1,), (0,)), ((), ()))
# tile and half-tensor boundaries (the noise counters pair element i with i + M*N/2) and a random spread
ROWS = np.unique(np.concatenate([[0, 1, 127, 128, 255, 256, 2047, 4095, 4096, 4097, 8190, 8191],
                                 np.random.default_rng(1).integers(0, M, 12)]))
COLS = np.unique(np.concatenate([[0, 1, 63, 64, 255, 256, 7167, 7168, 14334, 14335],
                                 np.random.default_rng(2).integers(0, N, 14)]))


def make_problem():
  rng = np.random.default_rng(2024)

  def normal_bf16(shape, scale):
    x = rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)
    return (x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)  # truncated: representable in bf16

  lhs, rhs, g = normal_bf16((M, K), 1.0), normal_bf16((K, N), 0.02), normal_bf16((M, N), 1e-3)
  # outliers so that the abs-max is not the same everywhere
  lhs[ROWS[:3], 5] = nm.cast(lhs[ROWS[:3], 5] * np.float32(30), 'bf16')
  g[7, COLS[:3]] = nm.cast(g[7, COLS[:3]] * np.float32(50), 'bf16')
  return lhs, rhs, g


@pytest.fixture(scope='module')
def problem():
  return make_problem()


def _product(problem, gpu, sr, key):
  from aqt_amd.v2 import config
  lhs, rhs, g = problem
  L = U.to_dev(lhs, 'bf16', gpu).requires_grad_(True)
  Rr = U.to_dev(rhs, 'bf16', gpu).requires_grad_(True)
  cfg = config.fully_quantized(fwd_bits=8, bwd_bits=8, use_stochastic_rounding=sr)
  cfg = config.set_context(cfg, key, None)
  out = cfg(L, Rr, MATMUL)
  out.backward(U.to_dev(g, 'bf16', gpu))
  torch.cuda.synchronize()
  return out.detach(), L.grad, Rr.grad


def _one_side(g, fwd, ocfg, lhs_side, with_abs_dot=False):
  """One of the two backward contractions of dg_core_vjp_bwd (aqt_dot_general.py:1178-1221).
  with_abs_dot: also the dequantized sum of |products| of every output element."""
  y_res, raw = (fwd.lhs_res, ocfg.drhs) if lhs_side else (fwd.rhs_res, ocfg.dlhs)
  dims, out_axes = R.bwd_dimension_numbers(MATMUL, lhs_side, g.ndim, y_res.x.ndim)
  out, _, (g_res, y_res2), _ = R.dg_raw(g, 'bf16', y_res, None, dims, raw)
  out = np.transpose(out, out_axes)
  if not with_abs_dot:
    return out
  gq, yq = np.abs(g_res.qx.qvalue.astype(np.float64)), np.abs(y_res2.qx.qvalue.astype(np.float64))
  scales = float(np.asarray(g_res.qx.scale[0]).reshape(-1)[0]) * float(np.asarray(y_res2.qx.scale[0]).reshape(-1)[0])
  # dlhs contracts g[m, n] with y[k, n] over n -> [m, k]; drhs g[m, n] with y[m, k] over m -> [n, k] -> [k, n]
  abs_dot = (yq.T @ gq) if lhs_side else (gq @ yq.T)
  return out, abs_dot * scales


def _check(problem, gpu, sr):
  lhs, rhs, g = problem
  key = prng.prng_key(99)
  out, dlhs, drhs = _product(problem, gpu, sr, key)
  assert out.shape == (M, N) and dlhs.shape == (M, K) and drhs.shape == (K, N)
  ocfg = R.set_context(R.fully_quantized(8, 8, use_stochastic_rounding=sr), key if sr else None)

  # rows: forward and dlhs
  rcfg = copy.deepcopy(ocfg)
  if sr:
    rcfg.dlhs.lhs.noise_window = ((M, N), (ROWS, np.arange(N)))
  f_r = R.dg_fwd(lhs[ROWS], rhs, 'bf16', MATMUL, rcfg)
  rows_t = torch.from_numpy(ROWS).to(gpu)
  np.testing.assert_array_equal(out[rows_t].float().cpu().numpy(), f_r.out)
  np.testing.assert_array_equal(dlhs[rows_t].float().cpu().numpy(), _one_side(g[ROWS], f_r, rcfg, False))
  del f_r

  # columns: forward and drhs
  ccfg = copy.deepcopy(ocfg)
  if sr:
    ccfg.drhs.lhs.noise_window = ((M, N), (np.arange(M), COLS))
  f_c = R.dg_fwd(lhs, rhs[:, COLS], 'bf16', MATMUL, ccfg)
  cols_t = torch.from_numpy(COLS).to(gpu)
  np.testing.assert_array_equal(out[:, cols_t].float().cpu().numpy(), f_c.out)
  np.testing.assert_array_equal(drhs[:, cols_t].float().cpu().numpy(), _one_side(g[:, COLS], f_c, ccfg, True))

  # whole-tensor sanity that no slice can give: finite everywhere, and the quantized product
  # stays within the quantization error of the float one (checksums over all rows and columns; a
  # misplaced tile or a wrong scale would show as an error of order one)
  for t in (out, dlhs, drhs):
    assert torch.isfinite(t).all()
  L, Rr, G = (U.to_dev(x, 'bf16', gpu).float() for x in (lhs, rhs, g))
  ones_n = torch.ones(N, device=gpu)
  want_rowsum = L @ (Rr @ ones_n)
  got_rowsum = out.float() @ ones_n
  rel = (got_rowsum - want_rowsum).norm() / want_rowsum.norm()
  assert rel < 0.06, rel
  want_dl = G @ (Rr.t() @ torch.ones(K, device=gpu))
  rel = (dlhs.float() @ torch.ones(K, device=gpu) - want_dl).norm() / want_dl.norm()
  assert rel < 0.06, rel
  want_dr = (L.t() @ G) @ ones_n
  rel = (drhs.float() @ ones_n - want_dr).norm() / want_dr.norm()
  assert rel < 0.06, rel


def test_full_size_round_to_nearest(problem, gpu):
  _check(problem, gpu, sr=False)


def test_full_size_stochastic_rounding(problem, gpu):
  _check(problem, gpu, sr=True)


def _normal_bf16(rng, shape, scale):
  x = rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)
  return (x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)


def test_full_size_int4_weight_tiled(gpu):
  """int4 weights [8192, 28672] in groups of 128 along the contraction axis, int8 activations
  [2048, 8192], forward: lhs scales are per (row, tile), rhs scales per (tile, column), so
  out[rows, cols] needs those rows and columns only."""
  from aqt_amd.v2 import aqt_dot_general as aqt
  from aqt_amd.v2 import config
  from aqt_amd.v2 import tiled_dot_general as T
  m, k, n, ts = 2048, 8192, 28672, 128
  rng = np.random.default_rng(5)
  lhs, rhs = _normal_bf16(rng, (m, k), 1.0), _normal_bf16(rng, (k, n), 0.015)
  rows = np.unique(np.concatenate([[0, 1, 127, 128, 2047], rng.integers(0, m, 8)]))
  cols = np.unique(np.concatenate([[0, 1, 255, 256, 14335, 14336, 28671], rng.integers(0, n, 10)]))
  dg = config.set_context(aqt.dot_general_make(8, 4), None, None)
  tcfg = T.Cfg(lhs=T.TensorTiling([T.AxisTiling(axis=1, tile_size=ts)], []),
               rhs=T.TensorTiling([T.AxisTiling(axis=0, tile_size=ts)], []))
  with torch.no_grad():
    out = T.tiled_dot_general(tcfg, U.to_dev(lhs, 'bf16', gpu), U.to_dev(rhs, 'bf16', gpu), MATMUL, dot_general=dg)
  assert tuple(out.shape) == (m, n) and out.dtype == torch.bfloat16 and torch.isfinite(out).all()
  want, _ = R.tiled_dg_fwd(lhs[rows], np.ascontiguousarray(rhs[:, cols]), 'bf16', ts, R.dot_general_make(8, 4))
  got = out[torch.from_numpy(rows).to(gpu)][:, torch.from_numpy(cols).to(gpu)]
  np.testing.assert_array_equal(got.float().cpu().numpy(), want)


@pytest.mark.parametrize('accumulate', ['fast', 'f32'])
def test_full_size_fp8_einsum(gpu, accumulate, monkeypatch, record_property):
  """'bsd,dhk->bshk' with batch 8, sequence 4096, d 4096, 32 heads of 128: e4m3 forward, e5m2
  gradients with mantissa stochastic rounding, per-tensor scales.  With one scale per tensor the
  quantization is elementwise, so any block of the three results can be restated from the
  matching blocks of the operands, provided each block holds its tensor's largest element (the
  blocks are chosen that way).  The oracle rounds the exact sum once to float32.
  Tolerance, element by element, of the sum: 'fast' (the fp8 matrix instruction, which cuts every product off
  2^-13 below the largest of its group of 8): 2^-10 of the dequantized sum of |products| of that element;
  'f32' (through bf16): the float32 summation bound, k 2^-24 of that sum; plus, both, 2^-7 of the value
  (the three bf16 roundings of the dequantisation, here and in the oracle).  Besides the bound the test
  states how many sampled outputs equal the oracle's bits and how many lie within one bf16 ulp of them, and
  holds the measured shares as floors."""
  from aqt_amd import _lib as L
  from aqt_amd import ops
  from aqt_amd.v2 import aqt_dot_general as aqt
  from aqt_amd.v2 import config
  monkeypatch.setattr(ops, 'FP8_ACCUMULATE', L.ACC_F32 if accumulate == 'f32' else L.ACC_FAST)
  b, s, d, h, kh = 8, 4096, 4096, 32, 128
  bs, hk = b * s, h * kh
  rng = np.random.default_rng(6)
  lhs2, rhs2, g2 = _normal_bf16(rng, (bs, d), 1.0), _normal_bf16(rng, (d, hk), 0.02), _normal_bf16(rng, (bs, hk), 1e-3)
  rl, cl = np.unravel_index(np.abs(lhs2).argmax(), lhs2.shape)
  rr, cr = np.unravel_index(np.abs(rhs2).argmax(), rhs2.shape)
  rg, cg = np.unravel_index(np.abs(g2).argmax(), g2.shape)
  rows = np.unique(np.concatenate([[rl, rg, 0, bs - 1, bs // 2], rng.integers(0, bs, 43)]))
  dsel = np.unique(np.concatenate([[cl, rr, 0, d - 1], rng.integers(0, d, 44)]))
  cols = np.unique(np.concatenate([[cr, cg, 0, hk - 1, hk // 2], rng.integers(0, hk, 43)]))

  key = prng.prng_key(17)
  cfg = config.config_v4(fwd_bits='e4m3', dlhs_bits='e5m2', drhs_bits='e5m2')
  ocfg = R.config_v4('e4m3', 'e5m2', 'e5m2')
  for raw, oraw in ((cfg.fwd, ocfg.fwd), (cfg.dlhs, ocfg.dlhs), (cfg.drhs, ocfg.drhs)):
    raw.dg_quantizer.lhs.calib_shared_axes = raw.dg_quantizer.rhs.calib_shared_axes = 'per_tensor'
    oraw.lhs.calib_shared_axes = oraw.rhs.calib_shared_axes = 'per_tensor'
  cfg = config.set_context(cfg, key, None)
  ocfg = R.set_context(ocfg, key)
  x = U.to_dev(lhs2, 'bf16', gpu).reshape(b, s, d).requires_grad_(True)
  w = U.to_dev(rhs2, 'bf16', gpu).reshape(d, h, kh).requires_grad_(True)
  out = aqt.einsum('bsd,dhk->bshk', x, w, cfg)
  out.backward(U.to_dev(g2, 'bf16', gpu).reshape(b, s, h, kh))
  out2, dl2, dr2 = out.detach().reshape(bs, hk), x.grad.reshape(bs, d), w.grad.reshape(d, hk)
  for t in (out2, dl2, dr2):
    assert torch.isfinite(t).all()
  tr, td, tc = (torch.from_numpy(i).to(gpu) for i in (rows, dsel, cols))

  shares = {}

  def close(got, want, abs_dot, what, k):
    got = got.float().cpu().numpy().astype(np.float64)
    rel = k * 2.0 ** -24 if accumulate == 'f32' else 2.0 ** -10
    err, bound = np.abs(got - want), rel * abs_dot + 2.0 ** -7 * np.abs(want)
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert (err <= bound).all(), f'{what}: error {err[worst]} above the bound {bound[worst]} at {worst}'
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -126))) - 7)  # bf16: 8 significant bits
    shares[what] = (float((err == 0).mean()), float((err <= ulp).mean()), float((err / ulp).max()))
    for name, v in zip(('equal', 'within_1_bf16_ulp', 'max_err_in_bf16_ulps'), shares[what]):
      record_property(f'{what}_{name}_{accumulate}', v)
    # measured on about 2300 sampled elements per result: fast 0.991-0.995 equal, 0.998-0.9996 within one ulp
    # (largest 2 / 3 / 24 ulps, on sums that cancel); f32 1.0 / 1.0 / 0.9996 equal, the one other element 2 ulps off
    floor_equal, floor_ulp = (0.999, 0.999) if accumulate == 'f32' else (0.98, 0.995)
    assert shares[what][0] >= floor_equal and shares[what][1] >= floor_ulp, (what, shares[what])

  def fwd_abs_dot(f):
    lq, rq = np.abs(f.lhs_res.qx.qvalue.astype(np.float64)), np.abs(f.rhs_res.qx.qvalue.astype(np.float64))
    return (lq @ rq) * float(np.asarray(f.lhs_res.qx.scale[0]).reshape(-1)[0]) * float(
        np.asarray(f.rhs_res.qx.scale[0]).reshape(-1)[0])

  f = R.dg_fwd(lhs2[rows], np.ascontiguousarray(rhs2[:, cols]), 'bf16', MATMUL, ocfg)
  close(out2[tr][:, tc], f.out, fwd_abs_dot(f), 'out', d)
  # dlhs[rows, dsel] = g[rows, :] . rhs[dsel, :]^T
  c1 = copy.deepcopy(ocfg)
  c1.dlhs.lhs.noise_window = ((bs, hk), (rows, np.arange(hk)))
  f1 = R.dg_fwd(lhs2[np.ix_(rows, dsel)], rhs2[dsel], 'bf16', MATMUL, c1)
  close(dl2[tr][:, td], *_one_side(g2[rows], f1, c1, False, with_abs_dot=True), 'dlhs', hk)
  # drhs[dsel, cols] = lhs[:, dsel]^T . g[:, cols]
  c2 = copy.deepcopy(ocfg)
  c2.drhs.lhs.noise_window = ((bs, hk), (np.arange(bs), cols))
  f2 = R.dg_fwd(np.ascontiguousarray(lhs2[:, dsel]), rhs2[np.ix_(dsel, cols)], 'bf16', MATMUL, c2)
  close(dr2[td][:, tc], *_one_side(np.ascontiguousarray(g2[:, cols]), f2, c2, True, with_abs_dot=True), 'drhs', bs)
  print(f'fp8 einsum at full size, accumulate={accumulate}: (share equal to the oracle, share within 1 bf16 ulp, '
        f'largest error in bf16 ulps) {shares}')


@pytest.mark.parametrize('m', [1, 8, 32, 64])
@pytest.mark.parametrize('int4', [False, True])
def test_full_size_serving_weight(gpu, m, int4):
  """The serving shapes against the 4096 x 14336 weight (held [n, k]; int8, or int4 packed two
  per byte): per-token activation quantization in the call, per-output-channel weight scales,
  so the oracle restates a sample of output columns."""
  from aqt_amd import _lib as L
  from aqt_amd import ops
  n, k = 14336, 4096
  rng = np.random.default_rng(40 + m)
  x = U.rand((m, k), 'bf16', 300 + m, outliers=True)
  lim = 7 if int4 else 127
  wq = rng.integers(-lim, lim + 1, size=(n, k)).astype(np.int8)
  ws = np.abs(rng.standard_normal(n).astype(np.float32)) * np.float32(2e-4) + np.float32(1e-5)
  cols = np.unique(np.concatenate([[0, 1, 15, 16, 63, 64, n - 65, n - 64, n - 1], rng.integers(0, n, 300)]))
  xqt = R.quantize(x, 'bf16', R.QuantizerCfg(bits=8), calibration_axes=[1])
  acc = (xqt.qvalue.astype(np.float64) @ wq[cols].astype(np.float64).T).astype(np.int32)  # exact: |acc| < 2^53
  want = R.dequant(R.QTensor(acc, 'i32', [xqt.scale[0].reshape(-1, 1), ws[cols].reshape(1, -1)], None, 'bf16',
                             scale_dtypes=[xqt.scale_dtype, 'f32']))
  w_t = torch.from_numpy(wq).to(gpu)
  out, xs, xq = ops.decode(U.to_dev(x, 'bf16', gpu), ops.pack_i4(w_t) if int4 else w_t, torch.from_numpy(ws).to(gpu),
                           quant_bound=127.5, clip_bound=127.0, w_scale_dtype=torch.float32, want_xq=True,
                           w_dtype=L.I4P if int4 else L.I8)
  assert tuple(out.shape) == (m, n) and torch.isfinite(out).all()
  np.testing.assert_array_equal(xq.cpu().numpy(), xqt.qvalue.astype(np.int8))
  np.testing.assert_array_equal(xs.cpu().numpy(), xqt.scale[0].reshape(-1))
  np.testing.assert_array_equal(out[:, torch.from_numpy(cols).to(gpu)].float().cpu().numpy(), want)

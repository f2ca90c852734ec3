"""GPU parity: the aqt_amd.v2 dot_general API (fwd + bwd) against the numpy oracle."""
import numpy as np
import pytest
import torch

from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import config
from aqt_amd.v2 import utils
from oracle import aqt_ref as R
from oracle import numerics as nm
from oracle import prng
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

MATMUL = (((1,), (0,)), ((), ()))


def _np(t):
  return t.detach().float().cpu().numpy()


def _run_both(lhs, rhs, g, dt, dn, cfg, ocfg, key, gpu):
  """Runs product and oracle; returns dicts of comparable arrays."""
  cfg = config.set_context(cfg, key, None)
  ocfg = R.set_context(ocfg, key)
  L = U.to_dev(lhs, dt, gpu).requires_grad_(True)
  Rr = U.to_dev(rhs, dt, gpu).requires_grad_(True)
  out, (lqt, rqt) = cfg.dg_core(L, Rr, None, None, dn)
  out.backward(U.to_dev(g, dt, gpu))
  got = dict(out=_np(out), dlhs=_np(L.grad), drhs=_np(Rr.grad),
             lq=_np(lqt.qvalue), rq=_np(rqt.qvalue), ls=_np(lqt.scale[0]), rs=_np(rqt.scale[0]))
  f = R.dg_fwd(lhs, rhs, dt, dn, ocfg)
  dl, dr = R.dg_bwd(g, dt, dn, f, ocfg)
  want = dict(out=f.out, dlhs=dl, drhs=dr, lq=f.lhs_res.qx.qvalue.astype(np.float32),
              rq=f.rhs_res.qx.qvalue.astype(np.float32), ls=f.lhs_res.qx.scale[0],
              rs=f.rhs_res.qx.scale[0])
  return got, want


def _assert_same(got, want):
  for k in want:
    assert got[k].shape == want[k].shape, (k, got[k].shape, want[k].shape)
    np.testing.assert_array_equal(got[k], want[k], err_msg=k)


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('m,k,n', [(64, 128, 96), (256, 512, 384), (33, 80, 17), (512, 256, 2048)])
@pytest.mark.parametrize('sr', [True, False])
def test_fully_quantized_matmul(gpu, m, k, n, sr, dt):
  lhs = U.rand((m, k), dt, 1, outliers=True)
  rhs = U.rand((k, n), dt, 2, scale=0.02)
  g = U.rand((m, n), dt, 3, scale=1e-3)
  cfg = config.fully_quantized(fwd_bits=8, bwd_bits=8, use_stochastic_rounding=sr)
  ocfg = R.fully_quantized(8, 8, use_stochastic_rounding=sr)
  got, want = _run_both(lhs, rhs, g, dt, MATMUL, cfg, ocfg, prng.prng_key(42), gpu)
  _assert_same(got, want)


@pytest.mark.parametrize('partitionable', [False, True])
def test_partitionable_flag(gpu, partitionable, monkeypatch):
  monkeypatch.setattr(R, 'PARTITIONABLE', partitionable)
  monkeypatch.setattr(utils, 'threefry_partitionable', partitionable)
  lhs, rhs, g = U.rand((48, 64), 'bf16', 1), U.rand((64, 80), 'bf16', 2, 0.02), U.rand((48, 80), 'bf16', 3, 1e-3)
  got, want = _run_both(lhs, rhs, g, 'bf16', MATMUL, config.fully_quantized(), R.fully_quantized(),
                        prng.prng_key(7), gpu)
  _assert_same(got, want)


def test_use_fwd_quant_false(gpu):
  lhs, rhs, g = U.rand((64, 128), 'bf16', 1), U.rand((128, 32), 'bf16', 2, 0.02), U.rand((64, 32), 'bf16', 3, 1e-3)
  cfg = config.fully_quantized(use_fwd_quant=False)
  ocfg = R.fully_quantized(use_fwd_quant=False)
  got, want = _run_both(lhs, rhs, g, 'bf16', MATMUL, cfg, ocfg, prng.prng_key(1), gpu)
  _assert_same(got, want)


@pytest.mark.parametrize('dn,ls,rs', [
    ((((2,), (1,)), ((0,), (0,))), (3, 40, 64), (3, 64, 24)),   # batched matmul
    ((((2,), (0,)), ((), ())), (2, 16, 64), (64, 4, 8)),         # 'bsd,dhk->bshk'
    ((((1,), (1,)), ((), ())), (40, 64), (24, 64)),              # rhs already [n, k]
    ((((0,), (0,)), ((), ())), (64, 40), (64, 24)),              # lhs [k, m]
])
def test_dimension_numbers(gpu, dn, ls, rs):
  dt = 'bf16'
  lhs, rhs = U.rand(ls, dt, 1), U.rand(rs, dt, 2, 0.02)
  ocfg = R.set_context(R.fully_quantized(), prng.prng_key(3))
  f = R.dg_fwd(lhs, rhs, dt, dn, ocfg)
  g = U.rand(f.out.shape, dt, 3, 1e-3)
  got, want = _run_both(lhs, rhs, g, dt, dn, config.fully_quantized(), R.fully_quantized(),
                        prng.prng_key(3), gpu)
  _assert_same(got, want)


def test_config_v4_grad_side_sr_only(gpu):
  """config_v4: SR on the gradient only, drhs unquantized (float contraction)."""
  dt = 'bf16'
  lhs, rhs, g = U.rand((64, 128), dt, 1), U.rand((128, 32), dt, 2, 0.02), U.rand((64, 32), dt, 3, 1e-3)
  cfg = config.config_v4(fwd_bits=8, dlhs_bits=8, drhs_bits=None)
  ocfg = R.config_v4(8, 8, None)
  got, want = _run_both(lhs, rhs, g, dt, MATMUL, cfg, ocfg, prng.prng_key(9), gpu)
  drhs_got, drhs_want = got.pop('drhs'), want.pop('drhs')
  _assert_same(got, want)
  # float bf16 GEMM from the library: summation order differs, compare loosely
  np.testing.assert_allclose(drhs_got, drhs_want, rtol=2e-2, atol=2e-4)


def test_unquantized_equals_float_dot(gpu):
  lhs, rhs, g = U.rand((32, 64), 'f32', 1), U.rand((64, 16), 'f32', 2), U.rand((32, 16), 'f32', 3)
  cfg = config.set_context(config.default_unquantized_config(), None, None)
  L = U.to_dev(lhs, 'f32', gpu).requires_grad_(True)
  Rr = U.to_dev(rhs, 'f32', gpu).requires_grad_(True)
  out = cfg(L, Rr, MATMUL)
  out.backward(U.to_dev(g, 'f32', gpu))
  np.testing.assert_allclose(_np(out), lhs @ rhs, rtol=1e-5, atol=1e-5)
  np.testing.assert_allclose(_np(L.grad), g @ rhs.T, rtol=1e-5, atol=1e-5)
  np.testing.assert_allclose(_np(Rr.grad), lhs.T @ g, rtol=1e-5, atol=1e-5)


def test_serving_with_frozen_rhs(gpu):
  """rhs_qt from a first call replaces the float rhs (aqt_dot_general.py:614-671)."""
  dt = 'bf16'
  lhs, rhs = U.rand((8, 256), dt, 1), U.rand((256, 512), dt, 2, 0.02)
  cfg = config.set_context(config.fully_quantized(), prng.prng_key(0), None)
  L, Rr = U.to_dev(lhs, dt, gpu), U.to_dev(rhs, dt, gpu)
  out1, (_, rqt) = cfg.dg_core(L, Rr, None, None, MATMUL)
  out2, _ = cfg.dg_core(L, torch.zeros_like(Rr), None, rqt, MATMUL)
  np.testing.assert_array_equal(_np(out1), _np(out2))
  f = R.dg_fwd(lhs, rhs, dt, MATMUL, R.fully_quantized())
  np.testing.assert_array_equal(_np(out1), f.out)


@pytest.mark.parametrize('m', [1, 8, 33, 64, 100])
@pytest.mark.parametrize('w_sdt', ['bf16', 'f32'])
def test_serving_scale_dtypes_and_batch_sizes(gpu, m, w_sdt):
  """Frozen rhs whose scale is bf16 or f32 (jnp promotes product by product in dequant);
  m <= 64 takes the fused decode kernel, m = 100 the quantize + GEMM kernels."""
  import dataclasses
  dt = 'bf16'
  lhs, rhs = U.rand((m, 512), dt, 1, outliers=True), U.rand((512, 384), dt, 2, 0.02)
  cfg = config.set_context(config.fully_quantized(), prng.prng_key(0), None)
  L, Rr = U.to_dev(lhs, dt, gpu), U.to_dev(rhs, dt, gpu)
  _, (_, rqt) = cfg.dg_core(L, Rr, None, None, MATMUL)
  rqt = dataclasses.replace(rqt, scale=[rqt.scale[0].to(U.TORCH_DT[w_sdt])])
  out, (lqt, _) = cfg.dg_core(L, torch.zeros_like(Rr), None, rqt, MATMUL)
  # oracle: same quantizers, dequant with [lhs scale (bf16), rhs scale (w_sdt)]
  ocfg = R.fully_quantized()
  f = R.dg_fwd(lhs, rhs, dt, MATMUL, ocfg)
  lq, rq = f.lhs_res.qx, f.rhs_res.qx
  acc = (lq.qvalue.astype(np.int64) @ rq.qvalue.astype(np.int64)).astype(np.int32)
  want = R.dequant(R.QTensor(acc, 'i32', [lq.scale[0], rq.scale[0]], None, dt, scale_dtypes=['bf16', w_sdt]))
  np.testing.assert_array_equal(_np(lqt.qvalue), lq.qvalue.astype(np.float32))
  np.testing.assert_array_equal(_np(lqt.scale[0]), lq.scale[0])
  np.testing.assert_array_equal(_np(out), want)


def test_reference_assertions(gpu):
  cfg = config.fully_quantized()
  L = torch.zeros((4, 8), dtype=torch.int8, device=gpu)
  with pytest.raises(AssertionError):  # aqt_dot_general.py:984-987
    cfg(L, L.t(), MATMUL)
  a = torch.zeros((4, 8), dtype=torch.bfloat16, device=gpu)
  b = torch.zeros((8, 4), dtype=torch.float32, device=gpu)
  with pytest.raises(AssertionError):  # :1107-1109
    cfg(a, b, MATMUL)
  with pytest.raises(AssertionError):  # :1011-1013
    cfg(a, a.t(), MATMUL, precision='highest')


@pytest.mark.parametrize('fwd,bwd', [('e4m3', 'e5m2'), ('e4m3', 'e4m3')])
def test_fp8_config(gpu, fwd, bwd):
  """fp8 fwd + fp8 gradients (config_v4 with fp8 bits).  Quantized values and scales are
  bit-exact; contractions accumulate in float32 in MFMA order, so outputs are compared to
  the oracle (exact sum, one rounding) within one bf16 ulp: rtol 2**-7, plus an absolute
  term for cancelled sums."""
  dt = 'bf16'
  lhs, rhs, g = U.rand((96, 256), dt, 1, outliers=True), U.rand((256, 64), dt, 2, 0.02), U.rand((96, 64), dt, 3, 1e-3)
  cfg = config.config_v4(fwd_bits=fwd, dlhs_bits=bwd, drhs_bits=bwd)
  ocfg = R.config_v4(fwd, bwd, bwd)
  got, want = _run_both(lhs, rhs, g, dt, MATMUL, cfg, ocfg, prng.prng_key(5), gpu)
  for k in ('lq', 'rq', 'ls', 'rs'):
    np.testing.assert_array_equal(got[k], want[k], err_msg=k)
  for k in ('out', 'dlhs', 'drhs'):
    np.testing.assert_allclose(got[k], want[k], rtol=2.0 ** -7, atol=2.0 ** -9 * np.abs(want[k]).max(),
                               err_msg=k)


@pytest.mark.parametrize('sr', [False, True])
@pytest.mark.parametrize('dl,dr', [(2, 4), (1, 8), (4, None)])
def test_local_aqt_in_backward(gpu, dl, dr, sr):
  """LocalAqt (aqt_dot_general.py:259-328, 833-837): the bwd contraction axis is split in
  shards with their own scales; shard outputs are dequantized, then summed in float32."""
  dt = 'bf16'
  lhs, rhs, g = U.rand((64, 128), dt, 1, outliers=True), U.rand((128, 96), dt, 2, 0.02), U.rand((64, 96), dt, 3, 1e-3)
  mk = lambda c: None if c is None else aqt.LocalAqt(contraction_axis_shard_count=c)
  cfg = config.fully_quantized(use_stochastic_rounding=sr, dlhs_local_aqt=mk(dl), drhs_local_aqt=mk(dr))
  ocfg = R.fully_quantized(use_stochastic_rounding=sr)
  ocfg.dlhs.local_aqt_shard_count, ocfg.drhs.local_aqt_shard_count = dl, dr
  got, want = _run_both(lhs, rhs, g, dt, MATMUL, cfg, ocfg, prng.prng_key(11), gpu)
  _assert_same(got, want)


def test_local_aqt_largest_shape(gpu):
  """tile_largest_shape picks the largest contraction axis and a shard size
  (aqt_dot_general.py:279-300); on a matmul that is the same split as shard_count."""
  dt = 'bf16'
  lhs, rhs, g = U.rand((64, 128), dt, 1), U.rand((128, 96), dt, 2, 0.02), U.rand((64, 96), dt, 3, 1e-3)
  la = aqt.LocalAqt(contraction_axis_shard_size=32, tile_largest_shape=True)
  cfg = config.fully_quantized(use_stochastic_rounding=False, dlhs_local_aqt=la, drhs_local_aqt=la)
  ocfg = R.fully_quantized(use_stochastic_rounding=False)
  ocfg.dlhs.local_aqt_shard_count, ocfg.drhs.local_aqt_shard_count = 96 // 32, 64 // 32
  got, want = _run_both(lhs, rhs, g, dt, MATMUL, cfg, ocfg, prng.prng_key(11), gpu)
  _assert_same(got, want)


def test_fp8_per_tensor_einsum_projection(gpu):
  """The attention-projection config: 'bsd,dhk->bshk', per-tensor abs-max scales, e4m3 forward,
  e5m2 gradients with mantissa stochastic rounding on the gradient side.  Quantized values and
  scales bit-exact; contraction outputs within one bf16 ulp plus an absolute term (the MFMA's
  f32 summation order is not XLA's)."""
  dt = 'bf16'
  dn = (((2,), (0,)), ((), ()))
  lhs, rhs = U.rand((2, 64, 128), dt, 1, outliers=True), U.rand((128, 4, 32), dt, 2, 0.02)
  g = U.rand((2, 64, 4, 32), dt, 3, 1e-3)
  cfg = config.config_v4(fwd_bits='e4m3', dlhs_bits='e5m2', drhs_bits='e5m2')
  ocfg = R.config_v4('e4m3', 'e5m2', 'e5m2')
  for raw, oraw in ((cfg.fwd, ocfg.fwd), (cfg.dlhs, ocfg.dlhs), (cfg.drhs, ocfg.drhs)):
    raw.dg_quantizer.lhs.calib_shared_axes = raw.dg_quantizer.rhs.calib_shared_axes = 'per_tensor'
    oraw.lhs.calib_shared_axes = oraw.rhs.calib_shared_axes = 'per_tensor'
  got, want = _run_both(lhs, rhs, g, dt, dn, cfg, ocfg, prng.prng_key(21), gpu)
  for k in ('lq', 'rq', 'ls', 'rs'):
    np.testing.assert_array_equal(got[k], want[k], err_msg=k)
  for k in ('out', 'dlhs', 'drhs'):
    np.testing.assert_allclose(got[k], want[k], rtol=2.0 ** -7, atol=2.0 ** -9 * np.abs(want[k]).max(),
                               err_msg=k)


def test_mlp_block_fp32_full_size(gpu):
  """The MlpBlock config at its real size: x f32 [4096, 512], Dense 512 -> 2048, ReLU,
  Dense 2048 -> 512, fully_quantized(8, 8) with stochastic rounding in the backward pass;
  forward activations, both weight gradients and the input gradient are bit-exact."""
  dt = 'f32'
  rng = np.random.default_rng(0)
  x = U.rand((4096, 512), dt, 1)
  w1 = (rng.standard_normal((512, 2048)) / np.sqrt(512)).astype(np.float32)
  w2 = (rng.standard_normal((2048, 512)) / np.sqrt(2048)).astype(np.float32)
  g = U.rand((4096, 512), dt, 4, 1.0 / (4096 * 512))
  k1, k2 = prng.prng_key(1), prng.prng_key(2)
  # product
  X = U.to_dev(x, dt, gpu).requires_grad_(True)
  W1 = U.to_dev(w1, dt, gpu).requires_grad_(True)
  W2 = U.to_dev(w2, dt, gpu).requires_grad_(True)
  dg1 = config.set_context(config.fully_quantized(fwd_bits=8, bwd_bits=8), k1, None)
  dg2 = config.set_context(config.fully_quantized(fwd_bits=8, bwd_bits=8), k2, None)
  h = dg1(X, W1, MATMUL)
  y = dg2(torch.relu(h), W2, MATMUL)
  y.backward(U.to_dev(g, dt, gpu))
  # oracle
  o1, o2 = R.set_context(R.fully_quantized(8, 8), k1), R.set_context(R.fully_quantized(8, 8), k2)
  f1 = R.dg_fwd(x, w1, dt, MATMUL, o1)
  act = np.maximum(f1.out, np.float32(0))
  f2 = R.dg_fwd(act, w2, dt, MATMUL, o2)
  dact, dw2 = R.dg_bwd(g, dt, MATMUL, f2, o2)
  dh = np.where(f1.out > 0, dact, np.float32(0)).astype(np.float32)
  dx, dw1 = R.dg_bwd(dh, dt, MATMUL, f1, o1)
  np.testing.assert_array_equal(_np(h), f1.out)
  np.testing.assert_array_equal(_np(y), f2.out)
  np.testing.assert_array_equal(_np(W2.grad), dw2)
  np.testing.assert_array_equal(_np(W1.grad), dw1)
  np.testing.assert_array_equal(_np(X.grad), dx)


@pytest.mark.parametrize('m', [1, 16, 40, 64, 100])
@pytest.mark.parametrize('k', [512, 528])
def test_serving_int4_weights(gpu, m, k):
  """W4A8 serving: a frozen int4 rhs (held one value per byte in the QTensor).  With at most 64
  rows and k a multiple of 32 the decode kernel streams a packed copy made once; with m = 100 the
  dense kernel reads that packed copy and unpacks it in registers; k = 528 takes the
  int8-container kernels.  Same numbers either way."""
  dt = 'bf16'
  lhs, rhs = U.rand((m, k), dt, 1, outliers=True), U.rand((k, 384), dt, 2, 0.02)
  cfg = config.set_context(aqt.dot_general_make(8, 4), None, None)
  L, Rr = U.to_dev(lhs, dt, gpu), U.to_dev(rhs, dt, gpu)
  out1, (_, rqt) = cfg.dg_core(L, Rr, None, None, MATMUL)
  assert rqt.container_dtype is utils.int4
  out2, (lqt, _) = cfg.dg_core(L, torch.zeros_like(Rr), None, rqt, MATMUL)
  out3, _ = cfg.dg_core(L, torch.zeros_like(Rr), None, rqt, MATMUL)  # the cached packed copy
  f = R.dg_fwd(lhs, rhs, dt, MATMUL, R.dot_general_make(8, 4))
  np.testing.assert_array_equal(_np(out1), f.out)
  np.testing.assert_array_equal(_np(out2), f.out)
  np.testing.assert_array_equal(_np(out3), f.out)
  np.testing.assert_array_equal(_np(lqt.qvalue), f.lhs_res.qx.qvalue.astype(np.float32))

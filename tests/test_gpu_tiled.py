"""GPU parity: tiled (subchannel) dot_general through the product kernels against the oracle."""
import numpy as np
import pytest
import torch

from aqt_amd import ops
from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import config
from aqt_amd.v2 import tiled_dot_general as T
from oracle import aqt_ref as R
from oracle import numerics as nm
from tests import gpu_util as U

pytestmark = pytest.mark.gpu
MATMUL = (((1,), (0,)), ((), ()))


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('tiles,count', [(1, 64), (5, 4096), (64, 1000), (3, 1001), (7, 13)])
def test_sum_tiles(gpu, tiles, count, dt):
  x = U.rand((tiles, count), dt, 3, scale=3.0)
  want = np.zeros(count, np.float32)
  for t in range(tiles):
    want = want + x[t]
  want = nm.cast(want, dt)
  got = ops.sum_tiles(U.to_dev(x, dt, gpu))
  np.testing.assert_array_equal(got.float().cpu().numpy(), want)


def _tiling(ts):
  return T.Cfg(lhs=T.TensorTiling([T.AxisTiling(axis=1, tile_size=ts)], []),
               rhs=T.TensorTiling([T.AxisTiling(axis=0, tile_size=ts)], []))


@pytest.mark.parametrize('lhs_bits,rhs_bits', [(8, 4), (8, 8)])
@pytest.mark.parametrize('m,k,n,ts', [(48, 512, 96, 128), (33, 384, 40, 64), (256, 1024, 512, 128)])
def test_tiled_int_weights(gpu, m, k, n, ts, lhs_bits, rhs_bits):
  """int4 (or int8) weights with one scale per tile of `ts` along the contraction axis and
  per-token-per-tile int8 activations (flax/aqt_flax.py:529-561 wiring); the per-tile outputs
  are rounded to bf16 and summed in float32 in tile order."""
  dt = 'bf16'
  lhs, rhs = U.rand((m, k), dt, 1, outliers=True), U.rand((k, n), dt, 2, 0.015)
  ocfg = R.dot_general_make(lhs_bits, rhs_bits)
  want, res = R.tiled_dg_fwd(lhs, rhs, dt, ts, ocfg)
  dg = aqt.dot_general_make(lhs_bits, rhs_bits)
  dg = config.set_context(dg, None, None)
  got = T.tiled_dot_general(_tiling(ts), U.to_dev(lhs, dt, gpu), U.to_dev(rhs, dt, gpu), MATMUL,
                            dot_general=dg)
  assert got.dtype == torch.bfloat16 and tuple(got.shape) == (m, n)
  np.testing.assert_array_equal(got.float().cpu().numpy(), want)


def test_tiled_qtensors_and_scales(gpu):
  """The inner dot_general sees tile-count batch axes: one scale per (tile, row) / (tile, column)."""
  dt = 'bf16'
  m, k, n, ts = 40, 256, 24, 64
  lhs, rhs = U.rand((m, k), dt, 5), U.rand((k, n), dt, 6, 0.02)
  res = R.tiled_dg_fwd(lhs, rhs, dt, ts, R.dot_general_make(8, 4))[1]
  dg = config.set_context(aqt.dot_general_make(8, 4), None, None)
  xl, xr = T.generate_tiling_states_for_dot_general(_tiling(ts), torch.empty(m, k), torch.empty(k, n), MATMUL)
  tl, tr = xl.apply(U.to_dev(lhs, dt, gpu)), xr.apply(U.to_dev(rhs, dt, gpu))
  assert list(tl.shape) == [m, k // ts, ts] and list(tr.shape) == [k // ts, ts, n]
  _, (lqt, rqt) = dg.dg_core(tl, tr, None, None, (((2,), (1,)), ((1,), (0,))))
  np.testing.assert_array_equal(lqt.qvalue.float().cpu().numpy(), res.lhs_res.qx.qvalue.astype(np.float32))
  np.testing.assert_array_equal(rqt.qvalue.float().cpu().numpy(), res.rhs_res.qx.qvalue.astype(np.float32))
  np.testing.assert_array_equal(lqt.scale[0].float().cpu().numpy(), res.lhs_res.qx.scale[0])
  np.testing.assert_array_equal(rqt.scale[0].float().cpu().numpy(), res.rhs_res.qx.scale[0])
  assert np.abs(rqt.qvalue.float().cpu().numpy()).max() <= 7


# ---- grouped-scale contraction kernel -----------------------------------------------------------
def _grouped_ref(a, b, rs, cs, group, out, rdt, cdt):
  """Per group: QTensor.dequant of the group's int32 accumulators, rounded to `out`; float32 sum
  of the groups in order; one final cast."""
  m, k = a.shape
  n = b.shape[0]
  acc = np.zeros((m, n), np.float32)
  for g in range(k // group):
    sl = slice(g * group, (g + 1) * group)
    part = (a[:, sl].astype(np.int64) @ b[:, sl].astype(np.int64).T).astype(np.int32)
    dq = R.dequant(R.QTensor(part, 'i32', [rs[g][:, None], cs[g][None, :]], None, out, scale_dtypes=[rdt, cdt]))
    acc = acc + dq
  return nm.cast(acc, out)


@pytest.mark.parametrize('packed', [False, True])
@pytest.mark.parametrize('out,rdt,cdt', [('bf16', 'bf16', 'bf16'), ('bf16', 'bf16', 'f32'), ('f32', 'f32', 'f32')])
@pytest.mark.parametrize('m,n,k,group', [(128, 256, 256, 128), (200, 300, 512, 128), (64, 520, 1024, 256), (5, 9, 128, 128),
                                          (1, 200, 1024, 128), (16, 64, 384, 128), (17, 70, 512, 128), (40, 130, 256, 128),
                                          (64, 1000, 2048, 128), (48, 32, 8192 + 128, 128)])
def test_grouped_gemm_kernel(gpu, m, n, k, group, out, rdt, cdt, packed):
  """The tile kernels and, for at most 64 rows and groups of 128, the kernel with one wave per 16 rows of b."""
  from aqt_amd import _lib as L
  rng = np.random.default_rng(7)
  a = rng.integers(-127, 128, (m, k)).astype(np.int8)
  b = rng.integers(-7, 8, (n, k)).astype(np.int8)
  groups = k // group
  rs = nm.cast(np.abs(rng.standard_normal((groups, m)).astype(np.float32)) * np.float32(0.02) + np.float32(1e-3), rdt)
  cs = nm.cast(np.abs(rng.standard_normal((groups, n)).astype(np.float32)) * np.float32(3e-3) + np.float32(1e-4), cdt)
  want = _grouped_ref(a, b, rs, cs, group, out, rdt, cdt)
  bt = torch.from_numpy(b).to(gpu)
  if packed:
    bt = ops.pack_i4(bt)
    np.testing.assert_array_equal(bt.cpu().numpy(), (b[:, 0::2] & 0xF).astype(np.uint8) | ((b[:, 1::2] & 0xF).astype(np.uint8) << 4))
  got = ops.gemm_grouped(torch.from_numpy(a).to(gpu), bt, row_scale=torch.from_numpy(rs).to(gpu),
                         col_scale=torch.from_numpy(cs).to(gpu), group=group, out_dtype=U.TORCH_DT[out],
                         row_scale_dtype=U.TORCH_DT[rdt], col_scale_dtype=U.TORCH_DT[cdt],
                         b_dtype=L.I4P if packed else L.I4)
  np.testing.assert_array_equal(got.float().cpu().numpy(), want)
  if m <= 64 and group == 128:  # the tile kernel on the same call, and the few-rows kernel with row-major scales
    kw = dict(col_scale=torch.from_numpy(cs).to(gpu), group=group, out_dtype=U.TORCH_DT[out],
              row_scale_dtype=U.TORCH_DT[rdt], col_scale_dtype=U.TORCH_DT[cdt], b_dtype=L.I4P if packed else L.I4)
    tiled = ops.gemm_grouped(torch.from_numpy(a).to(gpu), bt, row_scale=torch.from_numpy(rs).to(gpu), tuning=128, **kw)
    assert torch.equal(tiled, got)
    by_row = ops.gemm_grouped(torch.from_numpy(a).to(gpu), bt, row_scale=torch.from_numpy(np.ascontiguousarray(rs.T)).to(gpu),
                              row_scale_by_row=True, **kw)
    assert torch.equal(by_row, got)
    if packed:
      eo = ops.gemm_grouped(torch.from_numpy(np.ascontiguousarray(_even_odd8(a))).to(gpu), bt,
                            row_scale=torch.from_numpy(rs).to(gpu), a_k_order=L.K_EVEN_ODD8, **kw)
      assert torch.equal(eo, got)


def _even_odd8(a):
  """Every aligned group of 8 along the last axis as elements 0,2,4,6,1,3,5,7."""
  g = a.reshape(a.shape[:-1] + (a.shape[-1] // 8, 8))
  return g[..., [0, 2, 4, 6, 1, 3, 5, 7]].reshape(a.shape)


@pytest.mark.parametrize('rows,cols,group', [(64, 1024, 128), (33, 256, 0), (8, 16384, 0)])
def test_quantize_even_odd_byte_order(gpu, rows, cols, group):
  """out_k_order = EVEN_ODD8 changes where the bytes of q land and nothing else."""
  from aqt_amd import _lib as L
  rng = np.random.default_rng(3)
  x = torch.from_numpy(rng.standard_normal((1, rows, cols)).astype(np.float32)).to(gpu).to(torch.bfloat16)
  kw = dict(reduce=L.REDUCE_COLS, group=group, out_dtype=L.I8, quant_bound=127.5, clip_bound=127.0)
  q0, s0 = ops.quantize(x, **kw)
  q1, s1 = ops.quantize(x, k_order=L.K_EVEN_ODD8, **kw)
  np.testing.assert_array_equal(s1.cpu().numpy(), s0.cpu().numpy())
  np.testing.assert_array_equal(q1.cpu().numpy(), _even_odd8(q0.cpu().numpy()))


def test_quantize_even_odd_byte_order_rejected_where_unsupported(gpu):
  from aqt_amd import _lib as L
  x = torch.zeros((1, 16, 64), device=gpu, dtype=torch.bfloat16)
  with pytest.raises(RuntimeError, match='EVEN_ODD8'):
    ops.quantize(x, reduce=L.REDUCE_ROWS, out_dtype=L.I8, quant_bound=127.5, clip_bound=127.0, k_order=L.K_EVEN_ODD8)
  x = torch.zeros((1, 16, 60), device=gpu, dtype=torch.bfloat16)
  with pytest.raises(RuntimeError, match='EVEN_ODD8'):
    ops.quantize(x, reduce=L.REDUCE_COLS, out_dtype=L.I8, quant_bound=127.5, clip_bound=127.0, k_order=L.K_EVEN_ODD8)


@pytest.mark.parametrize('m,n,k,group', [(128, 256, 256, 128), (200, 300, 512, 128), (64, 520, 1024, 256), (5, 9, 128, 128)])
def test_grouped_gemm_even_odd_lhs_and_row_major_scales(gpu, m, n, k, group):
  """A in even-odd byte order against a packed int4 B, row scales as [m][groups]: same result."""
  from aqt_amd import _lib as L
  rng = np.random.default_rng(11)
  a = rng.integers(-127, 128, (m, k)).astype(np.int8)
  b = rng.integers(-7, 8, (n, k)).astype(np.int8)
  groups = k // group
  rs = nm.cast(np.abs(rng.standard_normal((groups, m)).astype(np.float32)) * np.float32(0.02) + np.float32(1e-3), 'bf16')
  cs = nm.cast(np.abs(rng.standard_normal((groups, n)).astype(np.float32)) * np.float32(3e-3) + np.float32(1e-4), 'bf16')
  want = _grouped_ref(a, b, rs, cs, group, 'bf16', 'bf16', 'bf16')
  bt = ops.pack_i4(torch.from_numpy(b).to(gpu))
  got = ops.gemm_grouped(torch.from_numpy(_even_odd8(a)).to(gpu), bt,
                         row_scale=torch.from_numpy(np.ascontiguousarray(rs.T)).to(gpu),
                         col_scale=torch.from_numpy(cs).to(gpu), group=group, out_dtype=torch.bfloat16,
                         row_scale_dtype=torch.bfloat16, col_scale_dtype=torch.bfloat16, b_dtype=L.I4P,
                         a_k_order=L.K_EVEN_ODD8, row_scale_by_row=True)
  np.testing.assert_array_equal(got.float().cpu().numpy(), want)
  with pytest.raises(RuntimeError, match='a_k_order'):
    ops.gemm_grouped(torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu), row_scale=torch.from_numpy(rs).to(gpu),
                     col_scale=torch.from_numpy(cs).to(gpu), group=group, out_dtype=torch.bfloat16, b_dtype=L.I4,
                     a_k_order=L.K_EVEN_ODD8)

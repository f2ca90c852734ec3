"""GPU parity: aqtx_gemm_i8 against exact integer arithmetic and the oracle's dequant."""
import numpy as np
import pytest
import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from oracle import aqt_ref as R
from oracle import numerics as nm
from tests import gpu_util as U

pytestmark = pytest.mark.gpu


def _ints(shape, seed):
  return np.random.default_rng(seed).integers(-127, 128, size=shape).astype(np.int8)


def _ref_acc(a, b):
  return np.einsum('bmk,bnk->bmn', a.astype(np.float64), b.astype(np.float64)).astype(np.int64)


SHAPES = [
    (1, 256, 256, 128), (1, 512, 768, 384), (1, 300, 520, 144), (1, 64, 64, 16), (3, 130, 70, 48),
    (1, 17, 9, 50), (2, 5, 3, 7), (1, 1, 4096, 4096), (1, 1024, 512, 1040),
]


@pytest.mark.parametrize('batch,m,n,k', SHAPES)
def test_raw_accumulators(gpu, batch, m, n, k):
  a, b = _ints((batch, m, k), 1), _ints((batch, n, k), 2)
  c = ops.gemm(torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu), row_scale=None,
               col_scale=None, out_dtype=torch.int32)
  np.testing.assert_array_equal(c.cpu().numpy().astype(np.int64), _ref_acc(a, b))


@pytest.mark.parametrize('out', ['bf16', 'f32'])
@pytest.mark.parametrize('sdt', ['bf16', 'f32'])
@pytest.mark.parametrize('order', [L.SCALE_ROW_THEN_COL, L.SCALE_COL_THEN_ROW])
@pytest.mark.parametrize('batch,m,n,k', [(1, 256, 512, 4096), (2, 100, 72, 160), (1, 33, 20, 23)])
def test_dequant_epilogue(gpu, batch, m, n, k, order, sdt, out):
  if out == 'f32' and sdt == 'bf16':
    pytest.skip('scale dtype never narrower than the dequant dtype in the reference')
  a, b = _ints((batch, m, k), 3), _ints((batch, n, k), 4)
  rs = nm.cast(np.abs(U.rand((batch, m), 'f32', 5, 0.03)) + np.float32(1e-3), sdt)
  cs = nm.cast(np.abs(U.rand((batch, n), 'f32', 6, 6e-4)) + np.float32(1e-5), sdt)
  acc = _ref_acc(a, b).astype(np.int32)
  s1, s2 = (rs[:, :, None], cs[:, None, :])
  if order == L.SCALE_COL_THEN_ROW:
    s1, s2 = s2, s1
  want = R.dequant(R.QTensor(acc, 'i32', [s1, s2], sdt, out))
  c, acc_got = ops.gemm(torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu),
                        row_scale=torch.from_numpy(rs).to(gpu), col_scale=torch.from_numpy(cs).to(gpu),
                        out_dtype=U.TORCH_DT[out], scale_dtype=U.TORCH_DT[sdt], scale_order=order,
                        want_acc=True)
  np.testing.assert_array_equal(acc_got.cpu().numpy(), acc)
  np.testing.assert_array_equal(c.float().cpu().numpy(), want)


def test_large_accumulators_round_like_xla(gpu):
  """|acc| > 2**24: int32 -> f32 -> bf16 double rounding is part of the contract."""
  k = 4096
  a = np.full((1, 256, k), 127, np.int8)
  b = np.full((1, 256, k), 127, np.int8)
  b[0, ::2, : k // 3] = -126
  a[0, 1::3, 5:900] = 113
  acc = _ref_acc(a, b).astype(np.int32)
  assert np.abs(acc).max() > 2 ** 24
  want = nm.int32_to_float(acc, 'bf16')
  c = ops.gemm(torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu), row_scale=None,
               col_scale=None, out_dtype=torch.bfloat16)
  np.testing.assert_array_equal(c.float().cpu().numpy(), want)

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


@pytest.fixture(params=[4, 8, 16, 128, 129, 130, 131, 132, 133, 134, 0],
                ids=['waves4', 'waves8', 'persistent', 'tiles128', 'ring128', 'ring64x128', 'ring64', 'ring128x256', 'ring64pair', 'ring64x128pair', 'auto'])
def waves(request, monkeypatch):
  """Both workgroup shapes of the 256 x 256 int8 MFMA kernel, the kernel for few output tiles on each of its
  tile shapes and schedules, and the library's own choice (these shapes have few output tiles: the smaller
  tiles, with k in slices where it is long)."""
  monkeypatch.setattr(ops, 'GEMM_TUNING', request.param)
  return request.param


@pytest.fixture(params=[(8, L.ACC_FAST), (0, L.ACC_FAST), (0, L.ACC_F32)], ids=['tiles256', 'auto', 'f32sums'])
def tiles(request, monkeypatch):
  """fp8 operands: the 256 x 256 kernel, the library's own choice (the 128 x 128 kernel for these shapes), and
  the contraction through bf16 with float32-like sums (aqtx_gemm_plan.accumulate = AQTX_ACC_F32)."""
  monkeypatch.setattr(ops, 'GEMM_TUNING', request.param[0])
  monkeypatch.setattr(ops, 'FP8_ACCUMULATE', request.param[1])
  return request.param


def _ints(shape, seed):
  return np.random.default_rng(seed).integers(-127, 128, size=shape).astype(np.int8)


def _ref_acc(a, b):
  return np.einsum('bmk,bnk->bmn', a.astype(np.float64), b.astype(np.float64)).astype(np.int64)


SHAPES = [
    (1, 256, 256, 128), (1, 512, 768, 384), (1, 300, 520, 144), (1, 64, 64, 16), (3, 130, 70, 48),
    (1, 17, 9, 50), (2, 5, 3, 7), (1, 1, 4096, 4096), (1, 1024, 512, 1040),
]


@pytest.mark.parametrize('batch,m,n,k', SHAPES)
def test_raw_accumulators(gpu, waves, batch, m, n, k):
  a, b = _ints((batch, m, k), 1), _ints((batch, n, k), 2)
  c = ops.gemm(torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu), row_scale=None,
               col_scale=None, out_dtype=torch.int32)
  np.testing.assert_array_equal(c.cpu().numpy().astype(np.int64), _ref_acc(a, b))


@pytest.mark.parametrize('out', ['bf16', 'f32'])
@pytest.mark.parametrize('sdt', ['bf16', 'f32'])
@pytest.mark.parametrize('order', [L.SCALE_ROW_THEN_COL, L.SCALE_COL_THEN_ROW])
@pytest.mark.parametrize('batch,m,n,k', [(1, 256, 512, 4096), (2, 100, 72, 160), (1, 33, 20, 23)])
def test_dequant_epilogue(gpu, waves, batch, m, n, k, order, sdt, out):
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


@pytest.mark.parametrize('rdt,cdt', [('bf16', 'f32'), ('f32', 'bf16')])
@pytest.mark.parametrize('order', [L.SCALE_ROW_THEN_COL, L.SCALE_COL_THEN_ROW])
@pytest.mark.parametrize('batch,m,n,k', [(1, 256, 512, 512), (2, 100, 72, 160)])
def test_dequant_epilogue_mixed_scale_dtypes(gpu, tiles, batch, m, n, k, order, rdt, cdt):
  """A bf16 and an f32 scale: only a first product of two bf16 values is rounded to bf16."""
  a, b = _ints((batch, m, k), 3), _ints((batch, n, k), 4)
  rs = nm.cast(np.abs(U.rand((batch, m), 'f32', 5, 0.03)) + np.float32(1e-3), rdt)
  cs = nm.cast(np.abs(U.rand((batch, n), 'f32', 6, 6e-4)) + np.float32(1e-5), cdt)
  acc = _ref_acc(a, b).astype(np.int32)
  scales, sdts = [rs[:, :, None], cs[:, None, :]], [rdt, cdt]
  if order == L.SCALE_COL_THEN_ROW:
    scales, sdts = scales[::-1], sdts[::-1]
  want = R.dequant(R.QTensor(acc, 'i32', scales, None, 'bf16', scale_dtypes=sdts))
  c = ops.gemm(torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu),
               row_scale=torch.from_numpy(rs).to(gpu), col_scale=torch.from_numpy(cs).to(gpu),
               out_dtype=torch.bfloat16, row_scale_dtype=U.TORCH_DT[rdt], col_scale_dtype=U.TORCH_DT[cdt],
               scale_order=order)
  np.testing.assert_array_equal(c.float().cpu().numpy(), want)


def test_large_accumulators_round_like_xla(gpu, waves):
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


# ---- k in slices (the 128 x 128 kernel writes int32 slabs, a second kernel adds and dequantizes) ----
@pytest.mark.parametrize('slices', [2, 3, 7])
@pytest.mark.parametrize('out,sdt,order', [('bf16', 'bf16', L.SCALE_ROW_THEN_COL), ('bf16', 'f32', L.SCALE_COL_THEN_ROW),
                                           ('f32', 'f32', L.SCALE_ROW_THEN_COL), ('i32', None, None)])
@pytest.mark.parametrize('batch,m,n,k', [(1, 128, 256, 4096), (2, 100, 72, 1200), (1, 33, 21, 528), (1, 300, 130, 2064)])
def test_k_slices_give_the_same_bits(gpu, batch, m, n, k, out, sdt, order, slices):
  a, b = _ints((batch, m, k), 31), _ints((batch, n, k), 32)
  at, bt = torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu)
  acc = _ref_acc(a, b).astype(np.int32)
  if out == 'i32':
    c = ops.gemm(at, bt, row_scale=None, col_scale=None, out_dtype=torch.int32, k_split=slices)
    np.testing.assert_array_equal(c.cpu().numpy(), acc)
    return
  rs = nm.cast(np.abs(U.rand((batch, m), 'f32', 5, 0.03)) + np.float32(1e-3), sdt)
  cs = nm.cast(np.abs(U.rand((batch, n), 'f32', 6, 6e-4)) + np.float32(1e-5), sdt)
  s1, s2 = (rs[:, :, None], cs[:, None, :])
  if order == L.SCALE_COL_THEN_ROW:
    s1, s2 = s2, s1
  want = R.dequant(R.QTensor(acc, 'i32', [s1, s2], sdt, out))
  kw = dict(row_scale=torch.from_numpy(rs).to(gpu), col_scale=torch.from_numpy(cs).to(gpu),
            out_dtype=U.TORCH_DT[out], scale_dtype=U.TORCH_DT[sdt], scale_order=order)
  c, acc_got = ops.gemm(at, bt, want_acc=True, k_split=slices, **kw)
  np.testing.assert_array_equal(acc_got.cpu().numpy(), acc)
  np.testing.assert_array_equal(c.float().cpu().numpy(), want)
  assert torch.equal(c, ops.gemm(at, bt, k_split=1, **kw))


def test_k_slices_chosen_by_the_library(gpu):
  """A long k over few output tiles is cut by default; the plan's answer and the result agree with k_split = 1."""
  import ctypes
  m, n, k = 128, 512, 14336
  a, b = _ints((1, m, k), 33), _ints((1, n, k), 34)
  at, bt = torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu)
  plan = L.GemmPlan()
  plan.batch, plan.m, plan.n, plan.k, plan.lda, plan.ldb, plan.ldc = 1, m, n, k, k, k, n
  plan.a_dtype = plan.b_dtype = L.I8
  assert L.lib().aqtx_gemm_i8_k_slices(ctypes.byref(plan)) == 8
  plan.k_split = 1
  assert L.lib().aqtx_gemm_i8_k_slices(ctypes.byref(plan)) == 1
  plan.k_split, plan.m, plan.n = 0, 8192, 14336  # many tiles: never
  assert L.lib().aqtx_gemm_i8_k_slices(ctypes.byref(plan)) == 1
  rs = torch.rand(1, m, device=gpu) * 0.01 + 1e-3
  cs = torch.rand(1, n, device=gpu) * 1e-3 + 1e-5
  kw = dict(row_scale=rs, col_scale=cs, out_dtype=torch.bfloat16)
  got, want = ops.gemm(at, bt, **kw), ops.gemm(at, bt, k_split=1, **kw)
  assert torch.equal(got, want)
  np.testing.assert_array_equal(ops.gemm(at, bt, row_scale=None, col_scale=None, out_dtype=torch.int32).cpu().numpy(),
                                _ref_acc(a, b))


def test_k_slices_packed_int4_b(gpu):
  a = _ints((1, 96, 2048), 35)
  b = np.random.default_rng(36).integers(-8, 8, size=(1, 200, 2048)).astype(np.int8)
  at, bt = torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu)
  bp = ops.pack_i4(bt.reshape(200, 2048)).reshape(1, 200, 1024)
  rs = torch.rand(1, 96, device=gpu) * 0.01 + 1e-3
  cs = torch.rand(1, 200, device=gpu) * 1e-3 + 1e-5
  kw = dict(row_scale=rs, col_scale=cs, out_dtype=torch.bfloat16, want_acc=True)
  c0, acc0 = ops.gemm(at, bt, b_dtype=L.I4, k_split=1, **kw)
  for a_in, order in ((at, L.K_NATURAL), (torch.from_numpy(_even_odd8(a)).to(gpu), L.K_EVEN_ODD8)):
    c1, acc1 = ops.gemm(a_in, bp, b_dtype=L.I4P, a_k_order=order, k_split=4, **kw)
    assert torch.equal(c0, c1) and torch.equal(acc0, acc1)
  np.testing.assert_array_equal(acc0.cpu().numpy(), _ref_acc(a, b))


def test_k_slices_rejected_where_unsupported(gpu):
  a = torch.zeros((1, 64, 512), dtype=torch.int8, device=gpu)
  b = torch.zeros((1, 64, 512), dtype=torch.int8, device=gpu)
  with pytest.raises(RuntimeError, match='k_split must be in 0..64'):
    ops.gemm(a, b, row_scale=None, col_scale=None, out_dtype=torch.int32, k_split=65)
  offs = torch.tensor([0, 64], dtype=torch.int32, device=gpu)
  with pytest.raises(RuntimeError, match='k_split > 1 with ragged batches'):
    ops.gemm(a, b, row_scale=None, col_scale=None, out_dtype=torch.int32, group_offsets=offs, k_split=2)


# ---- every tile shape and schedule of the kernel for few output tiles gives the bits of the large tiles ----
@pytest.mark.parametrize('b_kind', ['rows', 'fragments', 'packed', 'packed_fragments'])
@pytest.mark.parametrize('batch,m,n,k,out,sdt', [
    (1, 200, 328, 4160, 'bf16', 'bf16'),   # ragged m and n, a k tail of 64
    (1, 130, 201, 1056, 'bf16', 'f32'),    # rows of C not 16-byte aligned: the stores straight from the accumulators
    (2, 129, 136, 384, 'f32', 'f32'),      # batches, three stages: as many as the ring has buffers
    (1, 64, 72, 128, 'bf16', 'bf16'),      # one stage
    (1, 512, 1024, 256, 'i32', None),      # raw sums, two stages
    (1, 96, 4096, 2048, 'f32', 'f32'),
])
def test_few_tiles_kernel_shapes_give_the_same_bits(gpu, monkeypatch, batch, m, n, k, out, sdt, b_kind):
  """plan->tuning 128 (128 x 128 tiles, plain schedule) and 129 .. 134 (the ring schedule on 128 x 128,
  64 x 128, 64 x 64 and 128 x 256 tiles and, with a barrier per two stages, on 64 x 64 and 64 x 128) against the 256 x 256 kernel on the same operands: integer sums, the same
  epilogue arithmetic, so bit for bit, outputs and raw accumulators, for rows and the fragment order of b,
  int8 and packed int4."""
  packed, frag = b_kind.startswith('packed'), b_kind.endswith('fragments')
  if frag and (batch > 1 or out == 'i32'):
    pytest.skip('the fragment order holds one weight, whose column count the binding reads off the column scale')
  torch.manual_seed(11)
  lo, hi = (-8, 8) if packed else (-127, 128)
  a = torch.randint(-127, 128, (batch, m, k), dtype=torch.int8, device=gpu)
  b = torch.randint(lo, hi, (batch, n, k), dtype=torch.int8, device=gpu)
  b_arg, b_dtype = b, L.I8
  if packed:
    b_arg, b_dtype = ops.pack_i4(b.reshape(batch * n, k)).reshape(batch, n, k // 2), L.I4P
  kw = dict(b_dtype=b_dtype, want_acc=True, k_split=1)
  if out == 'i32':
    kw.update(row_scale=None, col_scale=None, out_dtype=torch.int32)
  else:
    kw.update(row_scale=torch.rand(batch, m, device=gpu) + 0.5, col_scale=torch.rand(batch, n, device=gpu) * 0.01 + 1e-4,
              out_dtype=U.TORCH_DT[out], scale_dtype=U.TORCH_DT[sdt])
  monkeypatch.setattr(ops, 'GEMM_TUNING', 8)
  want, want_acc = ops.gemm(a, b_arg, **kw)
  ref = torch.einsum('bmk,bnk->bmn', a.cpu().to(torch.int64), b.cpu().to(torch.int64)).to(torch.int32)
  assert torch.equal(want_acc.cpu(), ref)
  if frag:
    b_arg, kw['b_layout'] = ops.tile_weight(b_arg[0].contiguous(), b_dtype), L.W_FRAGMENTS
  for tuning in (128, 129, 130, 131, 132, 133, 134, 0):
    monkeypatch.setattr(ops, 'GEMM_TUNING', tuning)
    got, got_acc = ops.gemm(a, b_arg, **kw)
    alone = ops.gemm(a, b_arg, **dict(kw, want_acc=False))  # without the copy of the sums the tile leaves through LDS
    bits = torch.int16 if out == 'bf16' else torch.int32
    assert torch.equal(got_acc, want_acc), tuning
    assert torch.equal(got.view(bits), want.view(bits)), tuning
    assert torch.equal(alone.view(bits), want.view(bits)), tuning
  # k in slices on request: on the plain schedule and on the ring shapes that take slices (unpacked operands)
  for tuning in (0, 128, 129, 133, 134):
    monkeypatch.setattr(ops, 'GEMM_TUNING', tuning)
    got, got_acc = ops.gemm(a, b_arg, **dict(kw, k_split=3))
    assert torch.equal(got_acc, want_acc), ('slices', tuning)
    assert torch.equal(got.view(bits), want.view(bits)), ('slices', tuning)


@pytest.mark.gpu
def test_library_choice_on_random_shapes_gives_the_bits_of_the_large_tiles(gpu, monkeypatch):
  """Forty seeded shapes with m up to 700, n up to 4500 and k up to 16500 (ragged in all three, so that the tile
  shape, the slices of k and the tails the library picks vary), b as rows and in fragment order: outputs and raw
  sums equal those of the 256 x 256 kernel bit for bit."""
  rng = np.random.default_rng(20250607)
  for case in range(40):
    m = int(rng.integers(65, 700))
    n = int(rng.choice([rng.integers(16, 600), rng.integers(600, 4500)]))
    k = int(rng.choice([rng.integers(1, 40) * 16, rng.integers(40, 520) * 32]))
    torch.manual_seed(case)
    a = torch.randint(-127, 128, (1, m, k), dtype=torch.int8, device=gpu)
    b = torch.randint(-127, 128, (1, n, k), dtype=torch.int8, device=gpu)
    kw = dict(row_scale=torch.rand(1, m, device=gpu) + 0.5, col_scale=torch.rand(1, n, device=gpu) * 0.01 + 1e-4,
              out_dtype=torch.bfloat16, want_acc=True)
    monkeypatch.setattr(ops, 'GEMM_TUNING', 8)
    want, want_acc = ops.gemm(a, b, **kw)
    monkeypatch.setattr(ops, 'GEMM_TUNING', 0)
    got, got_acc = ops.gemm(a, b, **kw)
    assert torch.equal(got_acc, want_acc) and torch.equal(got.view(torch.int16), want.view(torch.int16)), (case, m, n, k, 'rows')
    frags = ops.tile_weight(b[0].contiguous(), L.I8)
    got, got_acc = ops.gemm(a, frags, b_layout=L.W_FRAGMENTS, **kw)
    assert torch.equal(got_acc, want_acc) and torch.equal(got.view(torch.int16), want.view(torch.int16)), (case, m, n, k, 'fragments')


# ---- packed int4 B (two values per byte, unpacked in registers) ---------------------------------
def _even_odd8(a):
  g = a.reshape(a.shape[:-1] + (a.shape[-1] // 8, 8))
  return np.ascontiguousarray(g[..., [0, 2, 4, 6, 1, 3, 5, 7]].reshape(a.shape))


@pytest.mark.parametrize('k_order', [L.K_NATURAL, L.K_EVEN_ODD8])
@pytest.mark.parametrize('batch,m,n,k', [(1, 256, 256, 256), (1, 512, 768, 384), (1, 300, 520, 160), (1, 64, 64, 32),
                                           (3, 130, 70, 96), (1, 17, 9, 64), (1, 1024, 512, 1056), (1, 100, 4096, 4096)])
def test_packed_int4_b_raw_accumulators(gpu, tiles, batch, m, n, k, k_order):
  """int32 output and the copy of the accumulators: exact, whatever the byte order of A."""
  a = _ints((batch, m, k), 11)
  b = np.random.default_rng(12).integers(-8, 8, size=(batch, n, k)).astype(np.int8)
  bp = ops.pack_i4(torch.from_numpy(b).to(gpu).reshape(batch * n, k)).reshape(batch, n, k // 2)
  at = torch.from_numpy(_even_odd8(a) if k_order == L.K_EVEN_ODD8 else a).to(gpu)
  c = ops.gemm(at, bp, row_scale=None, col_scale=None, out_dtype=torch.int32, b_dtype=L.I4P, a_k_order=k_order)
  np.testing.assert_array_equal(c.cpu().numpy().astype(np.int64), _ref_acc(a, b))


@pytest.mark.parametrize('out,rdt,cdt', [('bf16', 'bf16', 'bf16'), ('bf16', 'bf16', 'f32'), ('bf16', 'f32', 'f32'), ('f32', 'f32', 'f32')])
@pytest.mark.parametrize('batch,m,n,k', [(1, 256, 512, 4096), (2, 100, 72, 160), (1, 33, 20, 32)])
def test_packed_int4_b_dequant_epilogue(gpu, tiles, batch, m, n, k, out, rdt, cdt):
  """Same bits as the same contraction with the int4 values in int8 bytes, and as the oracle's dequant."""
  a = _ints((batch, m, k), 13)
  b = np.random.default_rng(14).integers(-8, 8, size=(batch, n, k)).astype(np.int8)
  rs = nm.cast(np.abs(U.rand((batch, m), 'f32', 5, 0.03)) + np.float32(1e-3), rdt)
  cs = nm.cast(np.abs(U.rand((batch, n), 'f32', 6, 6e-4)) + np.float32(1e-5), cdt)
  acc = _ref_acc(a, b).astype(np.int32)
  want = R.dequant(R.QTensor(acc, 'i32', [rs[:, :, None], cs[:, None, :]], None, out, scale_dtypes=[rdt, cdt]))
  kw = dict(row_scale=torch.from_numpy(rs).to(gpu), col_scale=torch.from_numpy(cs).to(gpu), out_dtype=U.TORCH_DT[out],
            row_scale_dtype=U.TORCH_DT[rdt], col_scale_dtype=U.TORCH_DT[cdt], want_acc=True)
  bt = torch.from_numpy(b).to(gpu)
  bp = ops.pack_i4(bt.reshape(batch * n, k)).reshape(batch, n, k // 2)
  c0, acc0 = ops.gemm(torch.from_numpy(a).to(gpu), bt, b_dtype=L.I4, **kw)
  c1, acc1 = ops.gemm(torch.from_numpy(a).to(gpu), bp, b_dtype=L.I4P, **kw)
  c2, acc2 = ops.gemm(torch.from_numpy(_even_odd8(a)).to(gpu), bp, b_dtype=L.I4P, a_k_order=L.K_EVEN_ODD8, **kw)
  np.testing.assert_array_equal(acc1.cpu().numpy(), acc)
  np.testing.assert_array_equal(acc2.cpu().numpy(), acc)
  np.testing.assert_array_equal(c1.float().cpu().numpy(), want)
  assert torch.equal(c0, c1) and torch.equal(c1, c2)


def test_packed_int4_b_rejected_where_unsupported(gpu):
  a = torch.zeros((1, 64, 64), dtype=torch.int8, device=gpu)
  bp = torch.zeros((1, 64, 32), dtype=torch.uint8, device=gpu)
  ones = torch.ones((1, 64), device=gpu)
  with pytest.raises(RuntimeError, match='ROW_THEN_COL'):
    ops.gemm(a, bp, row_scale=ones, col_scale=ones, out_dtype=torch.bfloat16, b_dtype=L.I4P, scale_order=L.SCALE_COL_THEN_ROW)
  with pytest.raises(RuntimeError, match='a_k_order'):
    ops.gemm(a, a, row_scale=ones, col_scale=ones, out_dtype=torch.bfloat16, a_k_order=L.K_EVEN_ODD8)
  with pytest.raises(RuntimeError, match='multiple of 32'):
    ops.gemm(a[:, :, :48].contiguous(), bp[:, :, :24].contiguous(), row_scale=ones, col_scale=ones,
             out_dtype=torch.bfloat16, b_dtype=L.I4P)


# ---- fp8 ---------------------------------------------------------------------------------
_FP8_TORCH = {'e4m3': torch.float8_e4m3fn, 'e5m2': torch.float8_e5m2}
_FP8_AQTX = {'e4m3': L.E4M3, 'e5m2': L.E5M2}


def _fp8_small_ints(shape, seed, kind):
  """Bytes of small integers (exact in both fp8 formats) and their float values."""
  v = np.random.default_rng(seed).integers(-4, 5, size=shape).astype(np.float32)
  b = torch.from_numpy(v).to(_FP8_TORCH[kind]).view(torch.uint8)
  return b, v


def _fp8_random_bytes(shape, seed, kind):
  """Random finite fp8 bit patterns (|x| <= 16 so that sums stay far from overflow)."""
  rng = np.random.default_rng(seed)
  allb = np.arange(256, dtype=np.uint8)
  vals = U.fp8_bytes_to_float(allb, kind)
  ok = allb[np.isfinite(vals) & (np.abs(vals) <= 16.0)]
  b = ok[rng.integers(0, len(ok), size=shape)]
  return torch.from_numpy(b), U.fp8_bytes_to_float(b, kind)


FP8_SHAPES = [(1, 256, 256, 256), (1, 300, 520, 144), (2, 130, 70, 48), (1, 17, 9, 50), (1, 512, 256, 4096)]


@pytest.mark.parametrize('ka,kb', [('e4m3', 'e4m3'), ('e4m3', 'e5m2'), ('e5m2', 'e4m3'), ('e5m2', 'e5m2')])
@pytest.mark.parametrize('batch,m,n,k', FP8_SHAPES)
def test_fp8_exact_when_sums_are_representable(gpu, tiles, batch, m, n, k, ka, kb):
  """Small-integer operands: every partial sum is exact in float32, so any summation order
  must give the exact result; a wrong format decode or a dropped k block cannot."""
  a, av = _fp8_small_ints((batch, m, k), 11, ka)
  b, bv = _fp8_small_ints((batch, n, k), 12, kb)
  want = np.einsum('bmk,bnk->bmn', av.astype(np.float64), bv.astype(np.float64))
  c = ops.gemm(a.to(gpu), b.to(gpu), row_scale=None, col_scale=None, out_dtype=torch.float32,
               a_dtype=_FP8_AQTX[ka], b_dtype=_FP8_AQTX[kb])
  np.testing.assert_array_equal(c.cpu().numpy().astype(np.float64), want)


@pytest.mark.parametrize('ka,kb', [('e4m3', 'e4m3'), ('e4m3', 'e5m2'), ('e5m2', 'e5m2')])
@pytest.mark.parametrize('batch,m,n,k', FP8_SHAPES)
def test_fp8_random_values_within_mfma_accumulation_error(gpu, tiles, batch, m, n, k, ka, kb):
  """Tolerance of the fp8 matrix instruction (AQTX_ACC_FAST): |got - exact| <= 2**-10 * sum_k |a_k b_k|.
  Measured on gfx950 (test_fp8_accumulation_models_of_the_two_forms pins it): the products of every 8
  consecutive k are aligned to the largest of them and each is cut off 2**-13 below it, so a group loses at most
  7 * 2**-13 of its largest product; the bound is that with a factor of slack.  Through bf16 (AQTX_ACC_F32)
  the sums stay within the worst-case bound of a float32 summation of k terms, k * 2**-24 * sum_k |a_k b_k|
  (measured: at most 2 float32 ulps of the largest term per 16 k).  The exact-sum test above pins everything
  that does not depend on this hardware rounding."""
  a, av = _fp8_random_bytes((batch, m, k), 13, ka)
  b, bv = _fp8_random_bytes((batch, n, k), 14, kb)
  av, bv = av.astype(np.float64), bv.astype(np.float64)
  want = np.einsum('bmk,bnk->bmn', av, bv)
  mag = np.einsum('bmk,bnk->bmn', np.abs(av), np.abs(bv))
  c = ops.gemm(a.to(gpu), b.to(gpu), row_scale=None, col_scale=None, out_dtype=torch.float32,
               a_dtype=_FP8_AQTX[ka], b_dtype=_FP8_AQTX[kb])
  err = np.abs(c.cpu().numpy().astype(np.float64) - want)
  bound = (k * 2.0 ** -24 if tiles[1] == L.ACC_F32 else 2.0 ** -10) * mag + 1e-30
  assert (err <= bound).all(), (err / bound).max()


def test_fp8_accumulation_models_of_the_two_forms(gpu, monkeypatch):
  """What separates the two values of aqtx_gemm_plan.accumulate, on operands built for it (e4m3 powers of two).
  One product of 2**16 at k = 0 and one of 2**(16 - d) elsewhere: the fp8 matrix instruction keeps the small one
  when it lies in another group of 8 consecutive k, or at most 2**13 below the large one; through bf16 it is kept
  down to the last bit a float32 sum holds (d = 23).  With +2**16 - 2**16 in one group the fp8 form has dropped a
  product 2**14 below them before they cancel."""
  def run(pairs, accumulate):
    a = np.zeros((1, 1, 64), np.float32); b = np.zeros((1, 1, 64), np.float32)
    for kk, (x, y) in pairs.items():
      a[0, 0, kk], b[0, 0, kk] = x, y
    ab = torch.from_numpy(a).to(torch.float8_e4m3fn).view(torch.uint8).to(gpu)
    bb = torch.from_numpy(b).to(torch.float8_e4m3fn).view(torch.uint8).to(gpu)
    monkeypatch.setattr(ops, 'FP8_ACCUMULATE', accumulate)
    return float(ops.gemm(ab, bb, row_scale=None, col_scale=None, out_dtype=torch.float32, a_dtype=L.E4M3, b_dtype=L.E4M3)[0, 0, 0])
  big = (256.0, 256.0)
  small = lambda d: (2.0 ** ((16 - d) // 2), 2.0 ** ((16 - d) - (16 - d) // 2))
  for d in (4, 13):  # inside the window of the fp8 form: both exact
    for acc in (L.ACC_FAST, L.ACC_F32):
      assert run({0: big, 1: small(d)}, acc) == 2.0 ** 16 + 2.0 ** (16 - d)
  for d in (14, 18, 23):
    assert run({0: big, 1: small(d)}, L.ACC_FAST) == 2.0 ** 16                     # same group of 8: dropped
    assert run({0: big, 8: small(d)}, L.ACC_FAST) == 2.0 ** 16 + 2.0 ** (16 - d)   # another group: kept
    assert run({0: big, 1: small(d)}, L.ACC_F32) == 2.0 ** 16 + 2.0 ** (16 - d)
  assert run({0: big, 1: (-256.0, 256.0), 2: small(14)}, L.ACC_FAST) == 0.0
  assert run({0: big, 1: (-256.0, 256.0), 2: small(14)}, L.ACC_F32) == 4.0
  assert run({0: big, 1: (-256.0, 256.0), 2: small(24)}, L.ACC_F32) == 2.0 ** -8


@pytest.mark.parametrize('out,sdt', [('bf16', 'bf16'), ('bf16', 'f32'), ('f32', 'f32')])
@pytest.mark.parametrize('order', [L.SCALE_ROW_THEN_COL, L.SCALE_COL_THEN_ROW])
@pytest.mark.parametrize('batch,m,n,k', [(1, 256, 512, 1024), (2, 100, 72, 160), (1, 33, 20, 23)])
def test_fp8_dequant_epilogue(gpu, tiles, batch, m, n, k, order, sdt, out):
  """The epilogue is checked bit-exactly on the accumulators the kernel itself reports."""
  a, _ = _fp8_random_bytes((batch, m, k), 15, 'e4m3')
  b, _ = _fp8_random_bytes((batch, n, k), 16, 'e5m2')
  rs = nm.cast(np.abs(U.rand((batch, m), 'f32', 5, 0.03)) + np.float32(1e-3), sdt)
  cs = nm.cast(np.abs(U.rand((batch, n), 'f32', 6, 6e-4)) + np.float32(1e-5), sdt)
  c, acc = ops.gemm(a.to(gpu), b.to(gpu), row_scale=torch.from_numpy(rs).to(gpu),
                    col_scale=torch.from_numpy(cs).to(gpu), out_dtype=U.TORCH_DT[out],
                    scale_dtype=U.TORCH_DT[sdt], scale_order=order, a_dtype=L.E4M3, b_dtype=L.E5M2,
                    want_acc=True)
  s1, s2 = (rs[:, :, None], cs[:, None, :])
  if order == L.SCALE_COL_THEN_ROW:
    s1, s2 = s2, s1
  want = R.dequant(R.QTensor(acc.cpu().numpy(), 'f32', [s1, s2], sdt, out))
  np.testing.assert_array_equal(c.float().cpu().numpy(), want)


def test_fp8_tile_sizes_give_the_same_bits(gpu, monkeypatch):
  """Both tile sizes walk k in the same order with the same instruction: the float sums agree bit for bit."""
  a, _ = _fp8_random_bytes((1, 300, 2048), 17, 'e4m3')
  b, _ = _fp8_random_bytes((1, 520, 2048), 18, 'e5m2')
  outs = []
  monkeypatch.setattr(ops, 'FP8_ACCUMULATE', L.ACC_FAST)
  for tuning in (8, 128):
    monkeypatch.setattr(ops, 'GEMM_TUNING', tuning)
    outs.append(ops.gemm(a.to(gpu), b.to(gpu), row_scale=None, col_scale=None, out_dtype=torch.float32,
                         a_dtype=L.E4M3, b_dtype=L.E5M2))
  assert torch.equal(outs[0].view(torch.int32), outs[1].view(torch.int32))


# ---- weight-only contraction (bf16 lhs, int8 rhs widened in registers; float32 sums: tolerance, not bits) ----
@pytest.mark.gpu
@pytest.mark.parametrize('w_sdt', ['bf16', 'f32'])
@pytest.mark.parametrize('batch,m,n,k', [(1, 65, 128, 64), (1, 200, 328, 1040), (2, 129, 130, 272), (1, 1024, 512, 4096),
                                         (1, 3, 5, 16)])
def test_weight_only_gemm_within_float_summation_error(gpu, batch, m, n, k, w_sdt):
  """c = bf16(bf16(sum_k a b) * scale), float32 sums in the kernel's own order.  Tolerance, stated: against
  the exact sum (float64; a bf16 times an int8 is exact), a float32 sum in any order is off by less than
  d = k * 2^-24 * sum_k |a b|; the later steps are monotone (positive scales), so every output lies between
  those steps applied to exact - d and exact + d, and 99 % of the outputs equal them applied to the exact sum.
  A transposed operand, a dropped k chunk or a wrong scale index fails both."""
  rng = np.random.default_rng(7)
  a = nm.to_bf16(rng.standard_normal((batch, m, k), dtype=np.float32))
  b = rng.integers(-127, 128, (batch, n, k)).astype(np.int8)
  ws = nm.cast(np.abs(rng.standard_normal((batch, n)).astype(np.float32)) * np.float32(2e-3) + np.float32(1e-4), w_sdt)
  exact = np.einsum('bmk,bnk->bmn', a.astype(np.float64), b.astype(np.float64))
  slack = k * 2.0 ** -24 * np.einsum('bmk,bnk->bmn', np.abs(a).astype(np.float64), np.abs(b).astype(np.float64))

  def later_steps(total):
    prod = nm.to_bf16(total.astype(np.float32)).astype(np.float64) * ws.astype(np.float64)[:, None, :]
    return nm.to_bf16(nm.cast(prod.astype(np.float32), w_sdt)).astype(np.float64)

  want, low, high = later_steps(exact), later_steps(exact - slack), later_steps(exact + slack)
  got = ops.gemm_weight_only(torch.from_numpy(a).to(torch.bfloat16).to(gpu), torch.from_numpy(b).to(gpu),
                             torch.from_numpy(ws.astype(np.float32)).to(gpu), col_scale_dtype=U.TORCH_DT[w_sdt])
  got = got.float().cpu().numpy().astype(np.float64)
  assert ((low <= got) & (got <= high)).all(), np.argwhere((got < low) | (got > high))[:8]
  assert (got == want).mean() >= 0.99


@pytest.mark.gpu
@pytest.mark.parametrize('layout', ['rows', 'fragments'])
@pytest.mark.parametrize('w_sdt', ['bf16', 'f32'])
@pytest.mark.parametrize('m,n,k', [(300, 520, 144), (256, 256, 128), (1024, 768, 4096), (130, 72, 1040), (2304, 4100, 320)])
def test_weight_only_gemm_tile_sizes_give_the_same_bits(gpu, m, n, k, w_sdt, layout):
  """The 128 x 128 kernel, the 256 x 256 kernel with a workgroup per tile and the same walked by one workgroup
  per CU sum k in the same order with the same instruction: bit for bit the same float sums (the tolerance
  test above, which the library's own choice of kernel runs through, therefore covers all three)."""
  torch.manual_seed(11)
  a = torch.randn(1, m, k, device=gpu).to(torch.bfloat16)
  b = torch.randint(-127, 128, (1, n, k), dtype=torch.int8, device=gpu)
  cs = (torch.rand(1, n, device=gpu) * 0.01 + 1e-4).to(U.TORCH_DT[w_sdt]).float()
  kw = dict(col_scale_dtype=U.TORCH_DT[w_sdt])
  if layout == 'fragments':
    b, kw['b_layout'] = ops.tile_weight(b[0], L.I8), L.W_FRAGMENTS
  outs = [ops.gemm_weight_only(a, b, cs, tuning=t, **kw) for t in (128, 129, 130, 131, 132, 133, 134, 8, 16, 0)]
  for o in outs[1:]:
    assert torch.equal(o.view(torch.int16), outs[0].view(torch.int16))


@pytest.mark.gpu
def test_weight_only_gemm_strided_operands(gpu):
  """Rows of a and b further apart than k (views into wider tensors) and the few-rows kernel's answer:
  both kernels round alike except for summation order."""
  rng = np.random.default_rng(8)
  m, n, k = 48, 272, 528
  a_wide = torch.from_numpy(nm.to_bf16(rng.standard_normal((1, m, k + 24), dtype=np.float32))).to(torch.bfloat16).to(gpu)
  b_wide = torch.from_numpy(rng.integers(-127, 128, (1, n, k + 48)).astype(np.int8)).to(gpu)
  a, b = a_wide[:, :, 8:8 + k], b_wide[:, :, 16:16 + k]
  ws = torch.rand(1, n, device=gpu) * 0.01 + 1e-4
  got = ops.gemm_weight_only(a, b, ws)
  other = ops.decode_weight_only(a[0].contiguous(), b[0].contiguous(), ws[0].contiguous())
  ref = (a[0].float() @ b[0].float().T).to(torch.bfloat16).float() * ws[0]
  assert torch.equal(got[0], other) or (got[0] != other).float().mean() < 0.01
  torch.testing.assert_close(got[0].float(), ref, rtol=2.0 ** -7, atol=1e-6)


# ---- B in the serving kernels' fragment order: the same results as from rows ----------------------------
@pytest.mark.gpu
@pytest.mark.parametrize('packed', [False, True])
@pytest.mark.parametrize('m,n,k,k_split', [(65, 128, 64, 0), (130, 200, 1056, 0), (256, 1024, 4096, 0), (96, 136, 4096, 4),
                                           (512, 72, 2080, 1), (2048, 2048, 512, 0), (300, 4100, 320, 0),
                                           (2048, 4608, 1024, 0), (2048, 4608, 1056, 0), (2304, 4100, 320, 0),
                                           (130, 200, 1120, 0), (2048, 4608, 1120, 0), (64 + 8, 4096, 4000, 0)])
def test_fragment_ordered_b_equals_rows(gpu, m, n, k, k_split, packed):
  """aqtx_gemm_i8 with b_layout = AQTX_W_FRAGMENTS (the buffer aqtx_tile_weight writes for the serving kernels)
  against the same call on the rows: integer sums, so bit for bit, outputs and raw accumulators, with and
  without slices of k, with n and k that end inside a 16-row block / in either 64-byte step of a 128-byte
  stage; shapes with 2048 rows or more have enough output tiles for the 256 x 256 kernel."""
  if packed and k % 32 != 0:
    pytest.skip('packed int4 needs k % 32 == 0')
  torch.manual_seed(5)
  lo, hi = (-8, 8) if packed else (-127, 128)
  a = torch.randint(-127, 128, (1, m, k), dtype=torch.int8, device=gpu)
  b = torch.randint(lo, hi, (1, n, k), dtype=torch.int8, device=gpu)
  rs, cs = torch.rand(1, m, device=gpu) + 0.5, torch.rand(1, n, device=gpu) + 0.5
  b_rows, b_dtype = b, L.I8
  if packed:
    b_rows, b_dtype = ops.pack_i4(b.reshape(n, k)).reshape(1, n, k // 2), L.I4P
  frags = ops.tile_weight(b_rows[0].contiguous(), b_dtype)
  kw = dict(row_scale=rs, col_scale=cs, out_dtype=torch.bfloat16, scale_dtype=torch.float32, b_dtype=b_dtype, k_split=k_split)
  want, want_acc = ops.gemm(a, b_rows, want_acc=True, **kw)
  got, got_acc = ops.gemm(a, frags, want_acc=True, b_layout=L.W_FRAGMENTS, **kw)
  assert torch.equal(got_acc, want_acc)
  assert torch.equal(got, want)
  ref = (a[0].cpu().to(torch.int64) @ b[0].cpu().to(torch.int64).T).to(torch.int32)
  assert torch.equal(got_acc[0].cpu(), ref)


@pytest.mark.gpu
def test_weight_only_gemm_fragment_ordered_b(gpu):
  torch.manual_seed(6)
  m, n, k = 200, 328, 1040
  a = torch.randn(1, m, k, device=gpu).to(torch.bfloat16)
  b = torch.randint(-127, 128, (1, n, k), dtype=torch.int8, device=gpu)
  cs = torch.rand(1, n, device=gpu) * 0.01 + 1e-4
  want = ops.gemm_weight_only(a, b, cs)
  got = ops.gemm_weight_only(a, ops.tile_weight(b[0], L.I8), cs, b_layout=L.W_FRAGMENTS)
  assert torch.equal(got, want)  # the same products added in the same order

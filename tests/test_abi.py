"""The C-ABI library: every declared symbol is exported; argument validation needs no GPU."""
import ctypes
import os
import re

import pytest

from aqt_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
  text = open(os.path.join(ROOT, 'include', 'aqtx.h')).read()
  text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
  return sorted(set(re.findall(r'\b(aqtx_[a-z0-9_]+)\s*\(', text)))


def test_library_exports_every_declared_symbol():
  lib = L.lib()
  names = _declared_symbols()
  assert len(names) >= 10
  for name in names:
    assert hasattr(lib, name), f'{name} is declared in include/aqtx.h but not exported'
    assert name in L.SYMBOLS, f'{name} has no ctypes prototype in aqt_amd/_lib.py'
  assert lib.aqtx_version() == 1


def _err(status):
  assert status != 0
  return L.lib().aqtx_last_error().decode()


def _qplan(**kw):
  p = L.QuantPlan()
  p.in_dtype = p.compute_dtype = p.scale_dtype = L.BF16
  p.out_dtype = L.I8
  p.batch, p.rows, p.cols = 1, 4, 64
  p.reduce = L.REDUCE_COLS
  p.quant_bound, p.clip_bound = 127.5, 127.0
  p.w_dtype = L.I8
  for k, v in kw.items():
    setattr(p, k, v)
  return p


FAKE = ctypes.c_void_p(0x1000)  # never dereferenced: every call below fails validation first


@pytest.mark.parametrize('kw,needle', [
    (dict(in_dtype=L.I32), 'in_dtype'),
    (dict(compute_dtype=L.I8), 'compute_dtype'),
    (dict(in_dtype=L.F32), 'compute_dtype'),
    (dict(out_dtype=L.F32), 'out_dtype'),
    (dict(rows=-1), 'negative'),
    (dict(reduce=7), 'reduce'),
    (dict(group=48), 'does not divide'),
    (dict(transpose_out=1), 'transpose_out'),
    (dict(noise=9), 'noise'),
    (dict(noise=L.NOISE_FP8_MANTISSA), 'fp8'),
    (dict(out_dtype=L.E4M3, noise=L.NOISE_JAX_UNIFORM), 'integer'),
    (dict(noise=L.NOISE_JAX_UNIFORM, noise_total=0), 'noise_total'),
    (dict(noise=L.NOISE_JAX_UNIFORM, noise_total=1 << 33), 'noise_total'),
    (dict(prescale=5), 'prescale'),
    (dict(quant_bound=0.0), 'positive'),
])
def test_quantize_plan_validation(kw, needle):
  lib = L.lib()
  p = _qplan(**kw)
  msg = _err(lib.aqtx_quantize(ctypes.byref(p), FAKE, None, FAKE, FAKE, None, 0, None))
  assert needle in msg, msg


def test_quantize_argument_validation():
  lib = L.lib()
  assert 'NULL' in _err(lib.aqtx_quantize(None, FAKE, None, FAKE, FAKE, None, 0, None))
  p = _qplan()
  assert 'NULL' in _err(lib.aqtx_quantize(ctypes.byref(p), None, None, FAKE, FAKE, None, 0, None))
  p = _qplan(prescale=L.PRESCALE_PER_COL)
  assert 'prescale' in _err(lib.aqtx_quantize(ctypes.byref(p), FAKE, None, FAKE, FAKE, None, 0, None))
  p = _qplan(reduce=L.REDUCE_ROWS)
  assert lib.aqtx_quantize_workspace_bytes(ctypes.byref(p)) == 64 * 8
  assert 'workspace' in _err(lib.aqtx_quantize(ctypes.byref(p), FAKE, None, FAKE, FAKE, None, 0, None))
  p = _qplan()
  assert 'aligned' in _err(lib.aqtx_quantize(ctypes.byref(p), ctypes.c_void_p(0x1001), None, FAKE, FAKE, None, 0, None))
  # empty tensors are a no-op, even without a GPU
  p = _qplan(rows=0)
  assert lib.aqtx_quantize(ctypes.byref(p), None, None, None, None, None, 0, None) == 0
  assert lib.aqtx_last_error() == b''


def test_even_odd_k_order_has_a_longest_group_and_the_host_knows_it():
  """aqtx_quantize writes every 8 k in even-odd order only for segments its row kernels hold in registers; the
  tiled dot_general asks for that order up to the same length and falls back to k order beyond it."""
  from aqt_amd.v2 import aqt_dot_general
  longest = aqt_dot_general._EVEN_ODD8_MAX_GROUP
  p = _qplan(rows=2, cols=2 * (longest + 8), group=longest + 8, out_k_order=L.K_EVEN_ODD8)
  assert 'segments of at most %d' % longest in _err(L.lib().aqtx_quantize(ctypes.byref(p), FAKE, None, FAKE, FAKE, None, 0, None))


def _gplan(**kw):
  p = L.GemmPlan()
  p.batch, p.m, p.n, p.k = 1, 64, 64, 64
  p.lda = p.ldb = p.ldc = 64
  p.a_dtype = p.b_dtype = L.I8
  p.out_dtype = p.dequant_dtype = p.row_scale_dtype = p.col_scale_dtype = L.BF16
  for k, v in kw.items():
    setattr(p, k, v)
  return p


@pytest.mark.parametrize('kw,needle', [
    (dict(m=-1), 'negative'),
    (dict(a_dtype=L.F32), 'operands'),
    (dict(out_dtype=L.I8), 'out_dtype'),
    (dict(dequant_dtype=L.I8), 'dequant_dtype'),
    (dict(row_scale_dtype=L.I32), 'row_scale_dtype'),
    (dict(col_scale_dtype=L.I8), 'col_scale_dtype'),
    (dict(scale_order=3), 'scale_order'),
    (dict(lda=32), 'leading dimension'),
    (dict(out_dtype=L.F32, dequant_dtype=L.BF16), 'combination'),
    (dict(group_offsets=FAKE, k=24, lda=24, ldb=24), 'ragged batches'),
])
def test_gemm_plan_validation(kw, needle):
  p = _gplan(**kw)
  msg = _err(L.lib().aqtx_gemm_i8(ctypes.byref(p), FAKE, FAKE, None, None, FAKE, None, None))
  assert needle in msg, msg


def test_gemm_argument_validation():
  lib = L.lib()
  assert 'NULL' in _err(lib.aqtx_gemm_i8(None, FAKE, FAKE, None, None, FAKE, None, None))
  p = _gplan()
  assert 'NULL' in _err(lib.aqtx_gemm_i8(ctypes.byref(p), None, FAKE, None, None, FAKE, None, None))
  p = _gplan(out_dtype=L.I32)
  assert 'no scales' in _err(lib.aqtx_gemm_i8(ctypes.byref(p), FAKE, FAKE, FAKE, None, FAKE, None, None))
  p = _gplan(m=0)
  assert lib.aqtx_gemm_i8(ctypes.byref(p), None, None, None, None, None, None, None) == 0


def test_prng_split_host_matches_oracle():
  import numpy as np
  from aqt_amd import ops
  from oracle import prng
  for part in (False, True):
    for num in (1, 2, 3, 7):
      np.testing.assert_array_equal(ops.prng_split(prng.prng_key(7), num, part),
                                    prng.split(prng.prng_key(7), num, part))
  assert 'NULL' in _err(L.lib().aqtx_prng_split_host(None, 2, 0, None))


def test_cpu_tensors_are_rejected():
  import torch
  from aqt_amd import ops
  x = torch.zeros((1, 4, 64), dtype=torch.bfloat16)
  with pytest.raises(RuntimeError, match='no CPU fallback'):
    ops.quantize(x, reduce=L.REDUCE_COLS, out_dtype=L.I8, quant_bound=127.5, clip_bound=127.0)


def _dplan(**kw):
  p = L.DecodePlan()
  p.m, p.n, p.k = 8, 256, 512
  p.x_dtype = p.x_scale_dtype = p.out_dtype = L.BF16
  p.w_scale_dtype = L.F32
  p.quant_bound, p.clip_bound = 127.5, 127.0
  p.w_dtype = L.I8
  for k, v in kw.items():
    setattr(p, k, v)
  return p


@pytest.mark.parametrize('kw,needle', [
    (dict(m=65), 'exceeds 64'),
    (dict(k=24), 'multiple of 16'),
    (dict(k=0), 'multiple of 16'),
    (dict(n=-1), 'negative'),
    (dict(x_dtype=L.I8), 'dtypes'),
    (dict(quant_bound=0.0), 'bounds'),
    (dict(n=1 << 20, k=4096), '2 GiB'),
    (dict(w_dtype=L.E4M3), 'w_dtype'),
    (dict(w_dtype=L.I4P, k=48), 'multiple of 32'),
])
def test_decode_plan_validation(kw, needle):
  p = _dplan(**kw)
  rc = L.lib().aqtx_decode_i8(ctypes.byref(p), FAKE, FAKE, FAKE, None, FAKE, FAKE, FAKE, 1 << 30, None)
  msg = _err(rc)
  assert needle in msg, msg


def test_decode_workspace_and_null_checks():
  p = _dplan()
  need = L.lib().aqtx_decode_workspace_bytes(ctypes.byref(p))
  assert need >= 8 * 512 and need % 256 == 0
  assert L.lib().aqtx_decode_workspace_bytes(ctypes.byref(_dplan(m=65))) == 0
  assert 'NULL' in _err(L.lib().aqtx_decode_i8(ctypes.byref(p), None, FAKE, FAKE, None, FAKE, FAKE, FAKE, need, None))
  assert 'workspace' in _err(L.lib().aqtx_decode_i8(ctypes.byref(p), FAKE, FAKE, FAKE, None, FAKE, FAKE, FAKE, 16, None))
  # empty problems succeed without touching the GPU
  assert L.lib().aqtx_decode_i8(ctypes.byref(_dplan(m=0)), None, None, None, None, None, None, None, 0, None) == 0


@pytest.mark.parametrize('kw,needle', [
    (dict(m=65), 'exceeds 64'),
    (dict(k=24), 'multiple of 16'),
    (dict(w_dtype=L.I4P, k=48), 'multiple of 32'),
    (dict(x_dtype=L.F32), 'must be bf16'),
    (dict(out_dtype=L.I32), 'dtypes'),
    (dict(w_dtype=L.E5M2), 'w_dtype'),
    (dict(n=1 << 20, k=4096), '2 GiB'),
    (dict(w_layout=7), 'w_layout'),
])
def test_weight_only_decode_plan_validation(kw, needle):
  p = _dplan(**kw)
  msg = _err(L.lib().aqtx_decode_weight_only(ctypes.byref(p), FAKE, FAKE, FAKE, FAKE, None, 0, None))
  assert needle in msg, msg


def test_weight_only_decode_null_and_empty():
  assert 'NULL' in _err(L.lib().aqtx_decode_weight_only(ctypes.byref(_dplan()), None, FAKE, FAKE, FAKE, None, 0, None))
  assert 'plan is NULL' in _err(L.lib().aqtx_decode_weight_only(None, FAKE, FAKE, FAKE, FAKE, None, 0, None))
  assert L.lib().aqtx_decode_weight_only(ctypes.byref(_dplan(n=0)), None, None, None, None, None, 0, None) == 0


def test_weight_only_decode_workspace_bytes():
  """Slices of k (and so a workspace) only for more than 16 tokens against a weight of few rows and a long k."""
  need = lambda **kw: L.lib().aqtx_decode_weight_only_workspace_bytes(ctypes.byref(_dplan(**kw)))
  assert need(m=64, n=4096, k=14336) == 4 * 64 * 4096 * 4     # 64 tiles of 64 rows -> 4 slices
  assert need(m=8, n=4096, k=14336) == 0
  assert need(m=24, n=4096, k=14336) == 4 * 24 * 4096 * 4
  assert need(m=24, n=4096, k=4096) == 0 and need(m=40, n=4096, k=4096) == 4 * 40 * 4096 * 4
  assert need(m=64, n=14336, k=4096) == 0                      # 224 tiles of 64 rows fill the chip
  assert need(m=64, n=4096, k=1024) == 0                       # k too short to cut
  assert need(m=65, n=4096, k=14336) == 0                      # not a valid plan


def _woplan(**kw):
  p = L.GemmPlan()
  p.batch, p.m, p.n, p.k = 1, 256, 256, 512
  p.lda = p.ldb = 512
  p.ldc = 256
  p.a_dtype, p.b_dtype = L.BF16, L.I8
  p.out_dtype = p.dequant_dtype = p.row_scale_dtype = L.BF16
  p.col_scale_dtype = L.F32
  for k, v in kw.items():
    setattr(p, k, v)
  return p


@pytest.mark.parametrize('kw,needle', [
    (dict(a_dtype=L.I8), 'a must be bf16'),
    (dict(b_dtype=L.I4P), 'a must be bf16'),
    (dict(out_dtype=L.F32), 'must be bf16'),
    (dict(k=520, lda=520, ldb=528), 'multiple of 16'),
    (dict(lda=516), '16-byte aligned'),
    (dict(ldb=256), 'leading dimension'),
    (dict(k_split=2), 'slices'),
    (dict(m=-1), 'negative'),
])
def test_weight_only_gemm_plan_validation(kw, needle):
  msg = _err(L.lib().aqtx_gemm_weight_only(ctypes.byref(_woplan(**kw)), FAKE, FAKE, FAKE, FAKE, None))
  assert needle in msg, msg


def test_weight_only_gemm_null_and_empty():
  assert 'NULL' in _err(L.lib().aqtx_gemm_weight_only(ctypes.byref(_woplan()), None, FAKE, FAKE, FAKE, None))
  assert 'plan is NULL' in _err(L.lib().aqtx_gemm_weight_only(None, FAKE, FAKE, FAKE, FAKE, None))
  assert L.lib().aqtx_gemm_weight_only(ctypes.byref(_woplan(m=0)), None, None, None, None, None) == 0


def _ggplan(**kw):
  p = L.GroupedGemmPlan()
  p.m, p.n, p.k, p.group = 64, 128, 512, 128
  p.lda, p.ldb, p.ldc = 512, 512, 128
  p.a_dtype, p.b_dtype = L.I8, L.I4
  p.out_dtype = p.row_scale_dtype = p.col_scale_dtype = L.BF16
  for k, v in kw.items():
    setattr(p, k, v)
  return p


@pytest.mark.parametrize('kw,needle', [
    (dict(group=96), 'multiple of 128'),
    (dict(k=640, lda=640, ldb=640, group=256), 'divides k'),
    (dict(b_dtype=L.E4M3), 'b must be'),
    (dict(a_dtype=L.I4P), 'a must be'),
    (dict(out_dtype=L.I32), 'dtypes'),
    (dict(lda=256), 'leading dimension'),
    (dict(lda=520, ldb=520), '16'),
    (dict(m=-2), 'bad shape'),
])
def test_grouped_gemm_plan_validation(kw, needle):
  p = _ggplan(**kw)
  msg = _err(L.lib().aqtx_gemm_i8_grouped(ctypes.byref(p), FAKE, FAKE, FAKE, FAKE, FAKE, None))
  assert needle in msg, msg


def test_grouped_gemm_packed_leading_dimension_is_in_bytes():
  # packed int4: a row of b holds k/2 bytes, so ldb = k/2 is valid and ldb < k/2 is not
  assert 'leading dimension' in _err(L.lib().aqtx_gemm_i8_grouped(
      ctypes.byref(_ggplan(b_dtype=L.I4P, ldb=128)), FAKE, FAKE, FAKE, FAKE, FAKE, None))
  assert 'NULL' in _err(L.lib().aqtx_gemm_i8_grouped(
      ctypes.byref(_ggplan(b_dtype=L.I4P, ldb=256)), None, FAKE, FAKE, FAKE, FAKE, None))


def test_small_entry_validation():
  assert 'even' in _err(L.lib().aqtx_pack_i4(FAKE, FAKE, 7, None))
  assert L.lib().aqtx_pack_i4(None, None, 0, None) == 0
  assert 'dtype' in _err(L.lib().aqtx_sum_tiles(FAKE, FAKE, 4, 16, L.I8, None))
  assert 'NULL' in _err(L.lib().aqtx_sum_tiles(None, FAKE, 4, 16, L.BF16, None))
  assert L.lib().aqtx_sum_tiles(None, None, 4, 0, L.BF16, None) == 0


def test_im2col_validation():
  p = L.Im2colPlan()
  p.n, p.c, p.rank = 2, 16, 2
  for d in range(2):
    p.in_size[d], p.kernel[d], p.stride[d], p.dilation[d], p.pad_lo[d], p.out_size[d] = 8, 3, 1, 1, 1, 8
  assert 'NULL' in _err(L.lib().aqtx_im2col_i8(None, FAKE, FAKE, None))
  assert 'NULL' in _err(L.lib().aqtx_im2col_i8(ctypes.byref(p), None, FAKE, None))
  p.rank = 4
  assert 'rank' in _err(L.lib().aqtx_im2col_i8(ctypes.byref(p), FAKE, FAKE, None))
  p.rank = 2
  p.stride[1] = 0
  assert 'bad extent' in _err(L.lib().aqtx_im2col_i8(ctypes.byref(p), FAKE, FAKE, None))
  p.stride[1] = 1
  p.n = 0
  assert L.lib().aqtx_im2col_i8(ctypes.byref(p), None, None, None) == 0


def test_ffi_shim_binds_only_declared_entry_points():
  """csrc/aqtx_ffi.cc (compiled only where the XLA FFI headers exist) calls nothing that
  include/aqtx.h does not declare, and fills plan fields that exist."""
  import re
  here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
  src = open(os.path.join(here, 'aqt_amd', 'csrc', 'aqtx_ffi.cc')).read()
  header = open(os.path.join(here, 'include', 'aqtx.h')).read()
  called = set(re.findall(r'\b(aqtx_[a-z0-9_]+)\(', src))
  assert called and called <= set(L.SYMBOLS), called - set(L.SYMBOLS)
  for field in set(re.findall(r'\bp(?:\.|->)([a-z_0-9]+)\b', src)):
    assert re.search(r'\b%s\b' % field, header), field
  handlers = re.findall(r'XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*(\w+)', src)
  assert {'AqtxQuantize', 'AqtxGemmI8', 'AqtxGemmFp8', 'AqtxGemmI8Grouped', 'AqtxDecodeI8', 'AqtxDequantize',
          'AqtxSumTiles', 'AqtxScaleCast'} <= set(handlers)


def test_ffi_shim_is_skipped_without_xla_headers(capsys):
  from aqt_amd import build
  if build.xla_ffi_include_dir() is not None:
    pytest.skip('XLA FFI headers are present here')
  assert build.build_ffi_shim(verbose=True) is None
  assert 'not built' in capsys.readouterr().err


def _gemm_operand_requests(rows, k, ld):
  """Highest byte offset (exclusive) the MFMA contraction kernel (csrc/gemm_core.h) requests from
  an operand of `rows` rows, row stride `ld`, contraction length `k`: a model of its load
  schedule.  A workgroup tile holds 256 rows; a stage is 128 bytes of K; the prologue requests
  stages 0 and 1, every later stage two ahead.  A 16-byte request of tile row r, chunk c (c = 0,
  16, .. 112) has buffer offset r*ld + c, range-checked by the hardware against the tile's
  (rows_in_tile - 1)*ld + k bytes, plus the stage's scalar offset k0, which is NOT range-checked.
  Without a K tail (k a multiple of 256) k0 is clamped to the last stage; with one, chunks at or
  past k are masked."""
  BM, BK = 256, 128
  ktail = k % (2 * BK) != 0
  kt2 = (k + 2 * BK - 1) // (2 * BK)
  stages = [0, BK] + [s for it in range(kt2) for s in ((2 * it + 2) * BK, (2 * it + 3) * BK)]
  if not ktail:
    stages = [min(s, k - BK) for s in stages]
  highest = 0
  for tile0 in range(0, rows, BM):
    rows_in_tile = min(BM, rows - tile0)
    records = (rows_in_tile - 1) * ld + k
    for k0 in set(stages):
      for c in range(0, BK, 16):
        if ktail and k0 + c >= k:
          continue  # masked
        # the last row of the tile that passes the range check reaches furthest
        for r in range(rows_in_tile - 1, -1, -1):
          if r * ld + c + 16 <= records:
            highest = max(highest, tile0 * ld + r * ld + c + k0 + 16)
            break
  return highest


@pytest.mark.parametrize('rows,k,ld', [
    (8192, 4096, 4096), (256, 256, 256), (300, 512, 512), (17, 1024, 1040), (512, 384, 384), (256, 128, 128),
    (100, 144, 144), (64, 16, 16), (1000, 2064, 2064), (14336, 8192, 8192),
])
def test_gemm_never_requests_bytes_past_an_operand(rows, k, ld):
  """The scalar offset of a buffer load escapes the hardware range check; the kernel has to keep
  its look-ahead requests inside the operand by itself (an exactly sized allocation may end on a
  page boundary)."""
  assert _gemm_operand_requests(rows, k, ld) <= (rows - 1) * ld + k


def test_gemm_k_slices_choice_is_a_host_decision():
  """aqtx_gemm_i8_k_slices: few output tiles and a long k are cut, many tiles never; plan->k_split overrides;
  asking for slices without a workspace is an error raised before any launch."""
  lib = L.lib()

  def slices(m, n, k, **kw):
    p = _gplan(m=m, n=n, k=k, lda=k, ldb=k, ldc=n, **kw)
    return lib.aqtx_gemm_i8_k_slices(ctypes.byref(p))

  assert slices(128, 4096, 14336) == 4         # 64 tiles of 64 x 128
  assert slices(128, 4096, 14336, b_dtype=L.I4P) == 8  # packed operands: 32 tiles of 128 x 128
  assert slices(256, 4096, 14336) == 4         # 64 tiles
  assert slices(128, 4096, 8192) == 4
  assert slices(256, 4096, 8192) == 1          # 256 tiles of 64 x 64 and a k below 10240: the deep ring on all of k
  assert slices(512, 4096, 8192) == 1          # 256 tiles of 64 x 128
  assert slices(256, 4096, 8192, b_dtype=L.I4P) == 4  # packed operands go through registers: slices as before
  assert slices(128, 4096, 4096) == 1          # a k below 8192 is never cut: smaller tiles instead
  assert slices(512, 4096, 14336) == 2         # 128 tiles
  assert slices(1024, 4096, 14336) == 1        # 256 tiles: one per CU already
  assert slices(1024, 4096, 4096) == 1         # 256 tiles: one per CU already
  assert slices(8192, 14336, 4096) == 1        # the large tiles fill the chip
  assert slices(128, 4096, 14336, k_split=1) == 1
  assert slices(128, 4096, 14336, k_split=3) == 3
  assert slices(128, 4096, 512, k_split=16) == 2   # a slice holds at least 256 of k
  assert slices(128, 4096, 14336, tuning=8) == 1   # the 256 x 256 kernel was asked for
  assert slices(128, 4096, 14336, tuning=133) == 1  # a tile shape of the ring schedule was asked for
  assert slices(100, 72, 24) == 1                  # not the vector path
  p = _gplan(m=128, n=4096, k=14336, lda=14336, ldb=14336, ldc=4096, k_split=65)
  assert 'k_split must be in 0..64' in _err(lib.aqtx_gemm_i8(ctypes.byref(p), FAKE, FAKE, None, None, FAKE, None, None))
  p = _gplan(m=128, n=4096, k=14336, lda=14336, ldb=14336, ldc=4096, k_split=4)
  assert 'k_split_workspace' in _err(lib.aqtx_gemm_i8(ctypes.byref(p), FAKE, FAKE, None, None, FAKE, None, None))
  # the kernel that adds the slices up takes a row per grid row: more than 65535 rows are refused in words
  p = _gplan(m=70000, n=128, k=4096, lda=4096, ldb=4096, ldc=128, k_split=2, k_split_workspace=0x1000,
             k_split_workspace_bytes=1 << 40)
  assert 'at most 65535 rows' in _err(lib.aqtx_gemm_i8(ctypes.byref(p), FAKE, FAKE, None, None, FAKE, None, None))
  # fp8: sums through bf16 are a choice of aqtx_gemm_fp8 alone
  p = _gplan(accumulate=L.ACC_F32)
  assert 'accumulate' in _err(lib.aqtx_gemm_i8(ctypes.byref(p), FAKE, FAKE, None, None, FAKE, None, None))
  p = _gplan(accumulate=5, a_dtype=L.E4M3, b_dtype=L.E4M3)
  assert 'accumulate' in _err(lib.aqtx_gemm_fp8(ctypes.byref(p), FAKE, FAKE, None, None, FAKE, None, None))


def test_conv_validation():
  lib = L.lib()
  w = L.Im2colPlan()
  w.n, w.c, w.rank = 2, 128, 2
  for d in range(2):
    w.in_size[d], w.kernel[d], w.stride[d], w.dilation[d], w.pad_lo[d], w.out_size[d] = 8, 3, 1, 1, 1, 8
  good = dict(m=2 * 64, n=32, k=9 * 128, lda=9 * 128, ldb=9 * 128, ldc=32)
  call = lambda wp, gp, x=FAKE: lib.aqtx_conv_i8(ctypes.byref(wp), ctypes.byref(gp), x, FAKE, None, None, FAKE, None)
  assert 'm = images * positions' in _err(call(w, _gplan(**dict(good, m=100))))
  assert 'k = taps * features' in _err(call(w, _gplan(**dict(good, k=1024, lda=1024, ldb=1024))))
  assert 'no k slices' in _err(call(w, _gplan(k_split=2, **good)))
  assert 'NULL' in _err(call(w, _gplan(**good), None))
  w.c = 64
  assert 'multiple of 128' in _err(call(w, _gplan(**dict(good, k=9 * 64, lda=9 * 64, ldb=9 * 64))))
  w.c, w.rank = 128, 4
  assert 'rank' in _err(call(w, _gplan(**good)))


def test_scale_cast_rejects_bad_plans():
  plan = L.ScalePlan()
  plan.in_dtype, plan.out_dtype = L.I8, L.I8
  plan.batch, plan.rows, plan.cols = 1, 4, 16
  rc = L.lib().aqtx_scale_cast(ctypes.byref(plan), None, None, None, None, None)
  assert rc != 0 and b'out_dtype must be f32 or bf16' in L.lib().aqtx_last_error()
  plan.out_dtype, plan.factors = L.BF16, 3
  rc = L.lib().aqtx_scale_cast(ctypes.byref(plan), None, None, None, None, None)
  assert rc != 0 and b'factors must be 0, 1 or 2' in L.lib().aqtx_last_error()
  plan.factors = 1
  plan.factor_axis[0], plan.factor_dtype[0] = 5, L.F32
  rc = L.lib().aqtx_scale_cast(ctypes.byref(plan), None, None, None, None, None)
  assert rc != 0 and b'unknown factor_axis' in L.lib().aqtx_last_error()


def test_quantize_partial_maxima_plans_are_validated():
  """other_axis_absmax on a plan that cannot write it, absmax_partials on a plan that cannot take them."""
  lib = L.lib()
  p = L.QuantPlan()
  p.in_dtype = p.compute_dtype = p.scale_dtype = L.BF16
  p.out_dtype = L.I8
  p.batch, p.rows, p.cols = 1, 64, 4096
  p.reduce = L.REDUCE_COLS
  p.quant_bound, p.clip_bound = 127.5, 127.0
  assert lib.aqtx_quantize_other_axis_parts(ctypes.byref(p)) == 64
  p.rows = 5000
  assert lib.aqtx_quantize_other_axis_parts(ctypes.byref(p)) == 1792
  p.noise = L.NOISE_JAX_UNIFORM
  p.noise_total, p.noise_stride_row, p.noise_stride_col = 5000 * 4096, 4096, 1
  assert lib.aqtx_quantize_other_axis_parts(ctypes.byref(p)) == 0
  p.other_axis_absmax = 4096
  assert 'other_axis_absmax' in _err(lib.aqtx_quantize(ctypes.byref(p), FAKE, None, FAKE, FAKE, None, 0, None))
  p.other_axis_absmax = None
  p.noise = L.NOISE_NONE
  p.reduce, p.transpose_out, p.rows, p.cols = L.REDUCE_ROWS, 1, 4096, 14336
  assert lib.aqtx_quantize_other_axis_parts(ctypes.byref(p)) == 14336 // 64
  p.cols = 14336 + 8
  assert lib.aqtx_quantize_other_axis_parts(ctypes.byref(p)) == 0
  p.cols = 14336
  p.absmax_partials, p.absmax_parts = 4096, 16  # a bf16 input: the maxima describe int8 values
  ws = lib.aqtx_quantize_workspace_bytes(ctypes.byref(p))
  assert 'absmax_partials' in _err(lib.aqtx_quantize(ctypes.byref(p), FAKE, None, FAKE, FAKE, FAKE, ws, None))


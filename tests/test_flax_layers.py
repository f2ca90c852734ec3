"""Host logic of the module-level callers (aqt_amd.v2.flax): dtype promotion table, einsum
operand swap, freezer modes.  Goldens from aqt/jax/v2/flax/aqt_flax_test.py and freezer.py."""
import pytest
import torch

from aqt_amd.v2 import aqt_tensor
from aqt_amd.v2 import utils
from aqt_amd.v2.flax import aqt_flax
from aqt_amd.v2.flax import freezer as general_freezer

bf16, f32, i8, i4 = torch.bfloat16, torch.float32, torch.int8, utils.int4
e4, e5 = torch.float8_e4m3fn, torch.float8_e5m2


@pytest.mark.parametrize('lhs,rhs,want', [
    (bf16, bf16, bf16), (bf16, f32, f32), (bf16, i8, bf16), (bf16, i4, f32),
    (f32, bf16, f32), (f32, f32, f32), (f32, i8, f32), (f32, i4, f32),
    (i8, bf16, bf16), (i8, f32, f32), (i8, i8, f32), (i8, i4, f32),
    (i4, bf16, f32), (i4, f32, f32), (i4, i8, f32), (i4, i4, i4),
    (e4, e4, e4), (e4, i8, bf16), (e4, i4, f32), (e4, bf16, bf16), (e4, f32, f32),
    (e5, e5, e5), (e5, i8, bf16), (e5, i4, f32), (e5, bf16, bf16), (e5, f32, f32), (e5, e4, bf16),
])
def test_aqt_promote_dtype_table(lhs, rhs, want):
  """aqt_flax_test.py:37-79, all 27 rows."""
  assert aqt_flax.promoted_dtype(lhs, rhs) is want or aqt_flax.promoted_dtype(lhs, rhs) == want


def test_aqt_promote_dtype_on_tensors():
  l, r = aqt_flax.aqt_promote_dtype(torch.zeros(1, 1, dtype=bf16), torch.zeros(1, 1, dtype=i8))
  assert l.dtype == bf16 and r.dtype == bf16


@pytest.mark.parametrize('eqn,swap', [
    ('ijkh,mkh->ijm', False), ('bsd,dhk->bshk', False), ('bc,ab->ac', True), ('abd,cbd->ac', False),
    ('mkh,ijkh->ijm', True), ('ab,bc->ca', True), ('bij,bjk->bik', False), ('bij,bjk->bki', True),
])
def test_einsum_operand_swap(eqn, swap):
  """jnp.einsum hands (rhs, lhs) to dot_general when the result is exactly
  (batch, rhs free, lhs free); AqtEinsum swaps its per-side settings with it."""
  assert aqt_flax.einsum_swaps_operands(eqn) is swap


def test_einsum_swapped_result_equals_unswapped():
  from aqt_amd.v2 import aqt_dot_general
  l, r = torch.randn(5, 7), torch.randn(3, 5)
  got = aqt_dot_general.einsum('bc,ab->ac', l, r)
  assert torch.allclose(got, torch.einsum('bc,ab->ac', l, r), atol=1e-5)


def _qt():
  return aqt_tensor.QTensor(qvalue=torch.ones(2, 3, dtype=torch.int8), scale=[torch.full((2, 1), 0.5)],
                            scale_t=[torch.full((2, 1), 0.5)], bias=[], dequant_dtype=torch.float32)


def test_legacy_freezer_modes():
  """aqt_flax.py:149-232: get() is None except in SERVE; set() stores only in CONVERT."""
  mk = lambda mode: aqt_flax.Freezer(quant_collection='aqt', quant_mode=mode, q_shape=(2, 3), q_dtype=torch.int8,
                                     s_shape=(2, 1), name='qrhs')
  for mode in (utils.QuantMode.TRAIN, utils.QuantMode.CALIBRATE):
    f = mk(mode)
    f.set(_qt())
    assert f.get() is None and f.state() == {}
  f = mk(utils.QuantMode.CONVERT)
  f.set(_qt())
  assert f.get() is None
  st = f.state()
  assert set(st['aqt']) == {'value', 'scale'} and st['aqt']['value'].dtype == torch.int8
  g = mk(utils.QuantMode.SERVE)
  with pytest.raises(AssertionError, match='holds no converted tensor'):
    g.get()
  g.load_state(st)
  qt = g.get()
  assert qt.scale is None and len(qt.scale_t) == 1 and qt.dequant_dtype == torch.float32
  g.set(_qt().replace(qvalue=torch.zeros(2, 3, dtype=torch.int8)))   # ignored while serving
  assert g.get().qvalue.sum() == 6
  with pytest.raises(NotImplementedError, match='biases'):
    f.set(_qt().replace(bias=[torch.zeros(1)]))


def test_general_freezer_modes():
  """freezer.py:32-100: NONE ignores, WRITE stores, READ returns (set only initialises)."""
  FM = general_freezer.FreezerMode
  f = general_freezer.Freezer(collection='aqt', mode=FM.NONE)
  f.set(1)
  assert f.get() is None and f.state() == {}
  f.mode = FM.WRITE
  f.set('a')
  assert f.get() is None and f.state() == {'aqt': {'frozen': 'a'}}
  f.mode = FM.READ
  assert f.get() == 'a'
  f.set('b')
  assert f.get() == 'a'
  g = general_freezer.Freezer(collection='aqt', mode=FM.READ)
  assert g.get() is None
  g.set('init')
  assert g.get() == 'init'


def test_freeze_mode_none_rejects_convert():
  with pytest.raises(ValueError, match='Freezer mode NONE'):
    aqt_flax._apply_freeze_mode(_qt(), aqt_flax.FreezerMode.NONE, True, utils.QuantMode.CONVERT, 'rhs')
  assert aqt_flax._apply_freeze_mode(_qt(), aqt_flax.FreezerMode.CALIBRATION, True, utils.QuantMode.CONVERT,
                                     'rhs').qvalue is None


def test_unquantized_layer_is_a_float_dot_general():
  dg = aqt_flax.AqtDotGeneral(cfg=None)
  l, r = torch.randn(4, 6), torch.randn(6, 5)
  out = dg(l, r, (((1,), (0,)), ((), ())), None)
  assert torch.allclose(out, l @ r, atol=1e-5)

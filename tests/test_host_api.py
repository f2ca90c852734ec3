"""Host-side logic of the aqt_amd.v2 mirror (runs without a GPU)."""
import dataclasses

import numpy as np
import pytest
import torch

from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import aqt_quantizer
from aqt_amd.v2 import calibration
from aqt_amd.v2 import config
from aqt_amd.v2 import lowering
from aqt_amd.v2 import stochastic_rounding
from aqt_amd.v2 import transpose
from aqt_amd.v2 import utils
from aqt_amd.v2.numerics import fp8_numerics
from aqt_amd.v2.numerics import int_numerics
from aqt_amd.v2.numerics import no_numerics
from oracle import aqt_ref as R
from oracle import prng


def test_fully_quantized_defaults():
  """Structure pinned by the reference's config_test.py:56-270 (fully_quantized(8, 8))."""
  cfg = config.fully_quantized(fwd_bits=8, bwd_bits=8)
  for raw, scope in ((cfg.fwd, 'aqt_fwd'), (cfg.dlhs, 'aqt_dlhs'), (cfg.drhs, 'aqt_drhs')):
    assert raw.jax_scope_name == scope
    assert raw.dg_accumulator_dtype == utils.int32
    assert raw.local_aqt is None
    assert raw.lhs.dequant_mode == aqt.DequantMode.OUTPUT
    assert raw.lhs.calibration_mode == aqt.CalibrationMode.CONTRACTING_AXIS
    for q in (raw.dg_quantizer.lhs, raw.dg_quantizer.rhs):
      n = q.numerics
      assert isinstance(n, int_numerics.IntSymmetric)
      assert (n.bits, n.preserve_zero, n.preserve_max_val, n.clip, n.clip_gradient, n.round) == (
          8, True, False, True, False, True)
      assert n.dtype == utils.int8
      assert q.calibration is calibration.AbsMaxCalibration
      assert q.calib_shared_axes is None and q.scale_stop_grad is True and q.scale_dtype is None
      assert q._calibrator is None  # initialised lazily inside the forward pass
  assert cfg.dlhs.rhs.use_fwd_quant is True and cfg.drhs.rhs.use_fwd_quant is True
  assert cfg.fwd.rhs.use_fwd_quant is False
  # stochastic rounding on both sides of both backward dots, none in the forward
  assert cfg.fwd.dg_quantizer.lhs.numerics.noise_fn is None
  for raw in (cfg.dlhs, cfg.drhs):
    for q in (raw.dg_quantizer.lhs, raw.dg_quantizer.rhs):
      assert isinstance(q.numerics.noise_fn, stochastic_rounding.JaxUniform)
  assert cfg.apply_custom_vjp_on_jax is True


def test_config_v4_defaults_and_fp8():
  cfg = config.config_v4()
  assert isinstance(cfg.drhs.dg_quantizer.lhs.numerics, no_numerics.NoNumerics)
  assert cfg.drhs.dg_accumulator_dtype is None
  assert cfg.dlhs.rhs.use_fwd_quant is False and cfg.drhs.rhs.use_fwd_quant is False
  assert isinstance(cfg.dlhs.dg_quantizer.lhs.numerics.noise_fn, stochastic_rounding.JaxUniform)
  assert cfg.dlhs.dg_quantizer.rhs.numerics.noise_fn is None
  f8 = config.config_v4(fwd_bits='e4m3', dlhs_bits='e5m2', drhs_bits='e5m2')
  n = f8.fwd.dg_quantizer.lhs.numerics
  assert isinstance(n, fp8_numerics.Fp8Numerics) and n.dtype == utils.float8_e4m3fn
  assert n.get_quant_bound() == 448.0 and f8.fwd.dg_accumulator_dtype == utils.float32
  g = f8.dlhs.dg_quantizer.lhs.numerics
  assert g.dtype == utils.float8_e5m2 and g.stochastic_rounding is True and g.get_quant_bound() == 57344.0
  assert f8.dlhs.dg_quantizer.rhs.numerics.stochastic_rounding is False
  fwd8 = config.config_fwd_fp8('e5m2')
  assert isinstance(fwd8.dlhs.dg_quantizer.lhs.numerics, no_numerics.NoNumerics)


def test_fully_quantized_sr_argument_checks():
  with pytest.raises(AssertionError):
    config.fully_quantized(use_stochastic_rounding=None, vjp_lhs_stochastic_rounding=True)
  with pytest.raises(AssertionError):
    config.fully_quantized(use_stochastic_rounding=True, vjp_lhs_stochastic_rounding=True,
                           vjp_rhs_stochastic_rounding=False)
  cfg = config.fully_quantized(use_stochastic_rounding=None, vjp_lhs_stochastic_rounding=True,
                               vjp_rhs_stochastic_rounding=False)
  assert cfg.dlhs.dg_quantizer.rhs.numerics.noise_fn is None


def test_int_numerics_bounds_table():
  for pz, pmv, b8 in ((False, False, 128.0), (False, True, 127.5), (True, False, 127.5), (True, True, 127.0)):
    n = int_numerics.IntSymmetric(bits=8, preserve_zero=pz, preserve_max_val=pmv, clip=True,
                                  clip_gradient=False, round=True, noise_fn=None, dtype=utils.int8)
    assert n.get_quant_bound() == b8
  n4 = config.fully_quantized(fwd_bits=4).fwd.dg_quantizer.lhs.numerics
  assert n4.dtype is utils.int4 and n4.get_quant_bound() == 7.5 and n4._get_fwd_clip_bound() == 7.0


@pytest.mark.parametrize('partitionable', [False, True])
def test_set_context_key_fanout_matches_oracle(partitionable, monkeypatch):
  monkeypatch.setattr(utils, 'threefry_partitionable', partitionable)
  monkeypatch.setattr(R, 'PARTITIONABLE', partitionable)
  key = prng.prng_key(42)
  cfg = config.set_context(config.fully_quantized(), key, None)
  ocfg = R.set_context(R.fully_quantized(), key)
  for name in ('fwd', 'dlhs', 'drhs'):
    raw, oraw = getattr(cfg, name), getattr(ocfg, name)
    np.testing.assert_array_equal(raw.dg_quantizer.lhs.context.key, oraw.lhs.key)
    np.testing.assert_array_equal(raw.dg_quantizer.rhs.context.key, oraw.rhs.key)
  # set_context copies: the input config keeps its empty contexts
  base = config.fully_quantized()
  config.set_context(base, key, None)
  assert base.fwd.dg_quantizer.lhs.context.key is None


@pytest.mark.parametrize('dn,ls,rs', [
    ((((1,), (0,)), ((), ())), (5, 7), (7, 3)),
    ((((2,), (1,)), ((0,), (0,))), (2, 5, 7), (2, 7, 3)),
    ((((2,), (0,)), ((), ())), (2, 3, 8), (8, 4, 5)),
    ((((3, 1), (0, 2)), ((0,), (1,))), (2, 4, 5, 6), (6, 2, 4, 3)),
])
def test_backward_dimension_numbers_match_oracle(dn, ls, rs):
  out_rank = len(ls) + len(rs) - 2 * len(dn[0][0]) - len(dn[1][0])
  for y_is_lhs, y_rank in ((False, len(rs)), (True, len(ls))):
    got = aqt._update_dimension_numbers_for_backward(dn, y_is_lhs, out_rank, y_rank)
    want = R.bwd_dimension_numbers(dn, y_is_lhs, out_rank, y_rank)
    assert got == want


@pytest.mark.parametrize('dn,ls,rs', [
    ((((1,), (0,)), ((), ())), (5, 7), (7, 3)),
    ((((2,), (1,)), ((0,), (0,))), (2, 5, 7), (2, 7, 3)),
    ((((2,), (0,)), ((), ())), (2, 3, 8), (8, 4, 5)),                     # 'bsd,dhk->bshk'
    ((((3, 1), (0, 2)), ((0,), (1,))), (2, 4, 5, 6), (6, 2, 4, 3)),
    ((((0, 2), (2, 0)), ((1,), (1,))), (4, 3, 5, 2), (5, 3, 4, 6, 7)),    # contraction pairs out of order
    ((((), ()), ((), ())), (3, 2), (4,)),                                 # outer product
])
def test_backward_dimension_numbers_give_the_autograd_gradients(dn, ls, rs):
  """Independent of the restated formula: the float contraction run with the derived dimension
  numbers and output permutation must equal what torch's autograd returns for the forward
  contraction."""
  g_ = torch.Generator().manual_seed(0)
  lhs = torch.randn(ls, generator=g_, dtype=torch.float64, requires_grad=True)
  rhs = torch.randn(rs, generator=g_, dtype=torch.float64, requires_grad=True)
  out = aqt.lax_dot_general(lhs, rhs, dn)
  g = torch.randn(out.shape, generator=g_, dtype=torch.float64)
  dl_want, dr_want = torch.autograd.grad(out, (lhs, rhs), g)
  for y, y_is_lhs, want in ((rhs, False, dl_want), (lhs, True, dr_want)):
    dims, perm = aqt._update_dimension_numbers_for_backward(dn, y_is_lhs, g.dim(), y.dim())
    got = aqt.lax_dot_general(g, y.detach(), dims).permute(perm)
    assert got.shape == want.shape
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)


def test_matmul_backward_dimension_numbers():
  dn = (((1,), (0,)), ((), ()))
  dims, perm = aqt._update_dimension_numbers_for_backward(dn, False, 2, 2)
  assert dims == (((1,), (1,)), ((), ())) and perm == (0, 1)
  dims, perm = aqt._update_dimension_numbers_for_backward(dn, True, 2, 2)
  assert dims == (((0,), (0,)), ((), ())) and perm == (1, 0)


def test_view_operand_layouts():
  x = torch.zeros((6, 10))
  v = lowering.view_operand(x, [], [0], [1])
  assert v.k_last and not v.copied and tuple(v.mem.shape) == (1, 6, 10) and v.noise_strides == (0, 10, 1)
  v = lowering.view_operand(x, [], [1], [0])  # contraction axis strided
  assert not v.k_last and not v.copied and tuple(v.mem.shape) == (1, 6, 10)
  assert v.noise_strides == (0, 1, 10)
  # a [k, n]-shaped view of an [n, k] buffer: memory order decides, noise counters follow the logical shape
  xt = torch.zeros((10, 6)).t()
  v = lowering.view_operand(xt, [], [0], [1])
  assert not v.k_last and not v.copied and tuple(v.mem.shape) == (1, 10, 6)
  assert v.noise_strides == (0, 10, 1)
  # batched, and 'bsd,dhk' style merged axes
  b = torch.zeros((3, 4, 5))
  v = lowering.view_operand(b, [0], [1], [2])
  assert v.k_last and tuple(v.mem.shape) == (3, 4, 5) and v.noise_strides == (20, 5, 1)
  w = torch.zeros((8, 4, 5))
  v = lowering.view_operand(w, [], [1, 2], [0])
  assert not v.k_last and not v.copied and tuple(v.mem.shape) == (1, 8, 20)
  # batch axis in the middle: needs the canonical copy
  t = torch.zeros((4, 3, 5))
  v = lowering.view_operand(t, [1], [0], [2])
  assert v.copied and v.k_last and tuple(v.mem.shape) == (3, 4, 5)
  assert v.noise_strides == (5, 15, 1)


def test_scale_transposes():
  dn = (((2,), (1,)), ((0,), (0,)))
  ls, rs = (3, 4, 5), (3, 5, 6)
  sl, sr = torch.zeros((3, 4, 1)), torch.zeros((3, 1, 6))
  tl = transpose.lhs_scale_transpose_to_output(sl, dn, ls, rs)
  tr = transpose.rhs_scale_transpose_to_output(sr, dn, ls, rs)
  assert tuple(tl.shape) == (3, 4, 1) and tuple(tr.shape) == (3, 1, 6)
  assert tuple(transpose.lhs_recover_scale_from_scale_t(tl, dn, ls, rs).shape) == (3, 4, 1)
  assert tuple(transpose.rhs_recover_scale_from_scale_t(tr, dn, ls, rs).shape) == (3, 1, 6)
  mm = (((1,), (0,)), ((), ()))
  s = torch.arange(7.0).reshape(1, 7)
  t = transpose.rhs_scale_transpose_for_lhs_input(s, (((1,), (1,)), ((), ())), (5, 7))
  assert tuple(t.shape) == (1, 7)
  t = transpose.rhs_scale_transpose_for_lhs_input(torch.zeros((5, 1)), (((0,), (0,)), ((), ())), (5, 9))
  assert tuple(t.shape) == (5, 1)
  assert transpose.lhs_scale_transpose_to_output(None, mm, (2, 3), (3, 4)) is None


def test_reference_assertions_fire_before_any_kernel():
  cfg = config.fully_quantized()
  mm = (((1,), (0,)), ((), ()))
  a8 = torch.zeros((4, 8), dtype=torch.int8)
  with pytest.raises(AssertionError, match='not yet optimized to accept quantized types'):
    cfg(a8, a8.t(), mm)
  a = torch.zeros((4, 8), dtype=torch.bfloat16)
  b = torch.zeros((8, 4), dtype=torch.float32)
  with pytest.raises(AssertionError, match='Unmatched lhs and rhs dtype'):
    cfg(a, b, mm)
  with pytest.raises(AssertionError, match='Precision'):
    cfg(a, a.t(), mm, precision='highest')
  bad = config.fully_quantized()
  bad.fwd.rhs.calibration_mode = aqt.CalibrationMode.REMAINING_AXIS
  with pytest.raises(AssertionError):
    bad(a, a.t().contiguous(), mm)
  q = aqt_quantizer.quantizer_make(8)
  with pytest.raises(AssertionError, match='second call'):
    q.init_calibration()


def test_no_cpu_fallback():
  cfg = config.fully_quantized()
  a = torch.zeros((4, 64), dtype=torch.bfloat16)
  with pytest.raises(RuntimeError, match='no CPU fallback'):
    cfg(a, torch.zeros((64, 8), dtype=torch.bfloat16), (((1,), (0,)), ((), ())))


def test_einsum_dimension_numbers():
  seen = {}

  def spy(lhs, rhs, dn, precision=None, preferred_element_type=None):
    seen['dn'] = dn
    return aqt.lax_dot_general(lhs, rhs, dn)

  x, w = torch.randn(2, 3, 8), torch.randn(8, 4, 5)
  out = aqt.einsum('bsd,dhk->bshk', x, w, spy)
  assert seen['dn'] == (((2,), (0,)), ((), ()))
  torch.testing.assert_close(out, torch.einsum('bsd,dhk->bshk', x, w))
  out = aqt.einsum('bqd,bkd->bkq', torch.randn(2, 3, 4), torch.randn(2, 5, 4), spy)
  assert seen['dn'] == (((2,), (2,)), ((0,), (0,))) and tuple(out.shape) == (2, 5, 3)


def test_ceil_to_po2_matches_oracle_op_by_op():
  """calibration.py:25-30 in float32 (random scales over 2^-29..2^29) and bfloat16 (every
  positive normal value away from the exponent limits)."""
  import numpy as np
  import torch
  from aqt_amd.v2 import calibration
  from oracle import aqt_ref as R
  v = np.exp(np.random.default_rng(0).uniform(-20, 20, 100000)).astype(np.float32)
  v = np.concatenate([v, np.exp2(np.arange(-29, 30)).astype(np.float32)])
  got = calibration.ceil_to_po2(torch.from_numpy(v)).numpy()
  np.testing.assert_array_equal(got, R.ceil_to_po2(v, 'f32'))
  assert (got >= v).all() and (got < 2 * v).all()
  allb = torch.arange(0x0100, 0x7E80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
  got = calibration.ceil_to_po2(allb)
  assert got.dtype == torch.bfloat16
  np.testing.assert_array_equal(got.float().numpy(), R.ceil_to_po2(allb.float().numpy(), 'bf16'))


def test_standalone_entry_points_and_graph_wrapper_without_a_gpu():
  """The reference's `aqt.jax.v2.pallas` names exist under the same path; nothing computes on the
  CPU: tensors off the GPU are refused, recording a graph needs a GPU."""
  import aqt_amd.v2.pallas as aqt_pl
  from aqt_amd.v2 import aqt_tensor, hip_graph
  for name in ('quant', 'dot_general', 'load_qtensor', 'pallas_call', 'DequantMode'):
    assert hasattr(aqt_pl, name), name
  assert aqt_pl.DequantMode is aqt.DequantMode
  with pytest.raises(NotImplementedError, match='no Pallas'):
    aqt_pl.pallas_call(lambda: None)
  qt = aqt_tensor.QTensor(qvalue=torch.zeros(4, 4, dtype=torch.int8), scale=[torch.ones(4, 1)], scale_t=None,
                          bias=[], dequant_dtype=torch.float32)
  assert aqt_pl.load_qtensor(qt) is qt
  with pytest.raises(Exception):  # no CPU path: the quantize kernel refuses a CPU tensor
    aqt_pl.quant(torch.randn(8, 16), 8, (1,))
  if not torch.cuda.is_available():
    with pytest.raises(RuntimeError, match='needs a GPU'):
      hip_graph.GraphedCall(lambda a: a, torch.zeros(4))


def test_deep_copy_of_a_configuration_is_independent_and_equal():
  """config.set_context copies the configuration on every call (config.py:66-90): the field-wise
  copies of the quantizer, numerics and context classes must behave like copy.deepcopy."""
  import copy
  from aqt_amd.v2 import utils
  cfg = config.fully_quantized(use_stochastic_rounding=True)
  assert copy.deepcopy(cfg) == cfg  # (keys are numpy arrays, which dataclass equality cannot compare: none set yet)
  cfg = config.set_context(cfg, utils.prng_key(3), train_step=7)
  dup = copy.deepcopy(cfg)
  for a, b in ((cfg.fwd, dup.fwd), (cfg.dlhs, dup.dlhs), (cfg.drhs, dup.drhs)):
    for side in ('lhs', 'rhs'):
      qa, qb = getattr(a.dg_quantizer, side), getattr(b.dg_quantizer, side)
      assert qa is not qb and qa.numerics is not qb.numerics and qa.context is not qb.context
      assert qa.calibration is qb.calibration  # the factory is shared, never changed in place
      if qa.context.key is not None:
        assert qa.context.key is not qb.context.key and (qa.context.key == qb.context.key).all()
  dup.fwd.dg_quantizer.lhs.numerics.bits = 4
  dup.fwd.dg_quantizer.lhs.context.train_step = 99
  assert cfg.fwd.dg_quantizer.lhs.numerics.bits == 8 and cfg.fwd.dg_quantizer.lhs.context.train_step == 7
  # the containers above the quantizers are copied too (their own field-wise deep copies)
  assert dup.fwd is not cfg.fwd and dup.fwd.lhs is not cfg.fwd.lhs
  assert cfg.fwd.local_aqt is None or dup.fwd.local_aqt is not cfg.fwd.local_aqt
  assert dup.fwd.dg_quantizer is not cfg.fwd.dg_quantizer and dup.fwd.dot_general is cfg.fwd.dot_general
  dup.fwd.lhs.dequant_mode = aqt.DequantMode.THIS_INPUT
  assert cfg.fwd.lhs.dequant_mode == aqt.DequantMode.OUTPUT

  @dataclasses.dataclass(kw_only=True)
  class WithTable(aqt.Tensor):  # a field a subclass adds is deep-copied, whatever it holds
    table: list = dataclasses.field(default_factory=list)

  t = WithTable(table=[[1, 2]])
  t2 = copy.deepcopy(t)
  assert t2 == t and t2.table is not t.table and t2.table[0] is not t.table[0]


def test_set_context_without_copying_the_settings():
  """copy_settings=False (what the layer modules pass on every call): the same contexts as the deep copy,
  written to quantizers of its own, around the settings objects of the configuration it was given."""
  base = config.fully_quantized(use_stochastic_rounding=True)
  deep = config.set_context(base, utils.prng_key(3), train_step=7, rhs_quant_mode=utils.QuantMode.SERVE)
  lean = config.set_context(base, utils.prng_key(3), train_step=7, rhs_quant_mode=utils.QuantMode.SERVE,
                            copy_settings=False)
  for name in ('fwd', 'dlhs', 'drhs'):
    b, d, l = getattr(base, name), getattr(deep, name), getattr(lean, name)
    assert l is not b and l.dg_quantizer is not b.dg_quantizer
    assert l.lhs is b.lhs and l.local_aqt is b.local_aqt
    for side in ('lhs', 'rhs'):
      qb, qd, ql = (getattr(x.dg_quantizer, side) for x in (b, d, l))
      assert ql is not qb and ql.numerics is qb.numerics
      assert qb.context is None or qb.context.key is None  # the configuration handed in is left as it was
      assert ql.context.quant_mode == qd.context.quant_mode and ql.context.train_step == 7
      assert (ql.context.key is None) == (qd.context.key is None)
      if ql.context.key is not None:
        assert (np.asarray(ql.context.key) == np.asarray(qd.context.key)).all()

  # a dot-general quantizer of another class is deep-copied as before
  class Mine(aqt.DefaultDotGeneralQuantizer):
    pass

  other = config.fully_quantized()
  other.fwd.dg_quantizer = Mine(**{f.name: getattr(other.fwd.dg_quantizer, f.name)
                                   for f in dataclasses.fields(other.fwd.dg_quantizer)})
  got = config.set_context(other, None, train_step=None, copy_settings=False)
  assert got.fwd.lhs is not other.fwd.lhs and got.fwd.dg_quantizer.lhs.numerics is not other.fwd.dg_quantizer.lhs.numerics

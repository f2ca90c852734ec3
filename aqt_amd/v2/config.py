"""Configuration factories and setters (mirrors aqt/jax/v2/config.py:55-818)."""
from __future__ import annotations

import copy
import functools
from typing import Any, Optional, Sequence

from aqt_amd import ops
from aqt_amd.v2 import aqt_dot_general
from aqt_amd.v2 import aqt_quantizer
from aqt_amd.v2 import calibration
from aqt_amd.v2 import stochastic_rounding
from aqt_amd.v2 import utils
from aqt_amd.v2.numerics import fp8_numerics
from aqt_amd.v2.numerics import int_numerics
from aqt_amd.v2.numerics import no_numerics
from aqt_amd.v2.numerics import numerics
from aqt_amd.v2.numerics import utils as numerics_utils
from aqt_amd.v2.aqt_conv_general import conv_general_dilated_make  # re-exported as in config.py:31

# Re-exports, as in the reference (config.py:33-52).
CalibrationMode = aqt_dot_general.CalibrationMode
DequantMode = aqt_dot_general.DequantMode
DotGeneral = aqt_dot_general.DotGeneral
DotGeneralRaw = aqt_dot_general.DotGeneralRaw
LocalAqt = aqt_dot_general.LocalAqt
Tensor = aqt_dot_general.Tensor
dot_general_make = aqt_dot_general.dot_general_make
dot_general_raw_make = aqt_dot_general.dot_general_raw_make
dtypes_allowed_for_int32_accum = aqt_dot_general.dtypes_allowed_for_int32_accum

SKIP = 'skip'


def _split_key(key, num_splits: int):
  """jax.random.split on raw key data (config.py:61-63)."""
  default = (None,) * num_splits
  if key is None:
    return default
  return tuple(ops.prng_split(key, num_splits, utils.threefry_partitionable))


def set_context(cfg: DotGeneral, key, train_step: Optional[int],
                lhs_quant_mode: utils.QuantMode = utils.QuantMode.TRAIN,
                rhs_quant_mode: utils.QuantMode = utils.QuantMode.TRAIN, *, copy_settings: bool = True):
  """Fans the PRNG key out to fwd/dlhs/drhs and lhs/rhs (config.py:66-90).

  Returns a deep copy of `cfg` with the contexts set, as the reference does.  With
  copy_settings=False the copy stops at the quantizers (the objects the contexts are written to)
  and shares the settings objects below them with `cfg`: for a caller that hands the result to
  one dot_general call and drops it (the layer modules, on every call), at a fifth of the cost.
  """

  def set_dg_raw_context(cfg_raw: DotGeneralRaw, key):
    key1, key2 = _split_key(key, num_splits=2)
    lhs_context = utils.Context(key=key1, train_step=train_step, quant_mode=lhs_quant_mode)
    rhs_context = utils.Context(key=key2, train_step=train_step, quant_mode=rhs_quant_mode)
    cfg_raw.dg_quantizer.set_context(lhs_context, rhs_context)

  key_fwd, key_dlhs, key_drhs = _split_key(key, num_splits=3)
  plain = type(cfg) is DotGeneral and all(
      type(raw) is DotGeneralRaw and type(raw.dg_quantizer) is aqt_dot_general.DefaultDotGeneralQuantizer
      for raw in (cfg.fwd, cfg.dlhs, cfg.drhs))
  if copy_settings or not plain:
    ret_cfg = copy.deepcopy(cfg)
  else:
    ret_cfg = aqt_dot_general.clone_down_to_quantizers(cfg)
  set_dg_raw_context(ret_cfg.fwd, key_fwd)
  set_dg_raw_context(ret_cfg.dlhs, key_dlhs)
  set_dg_raw_context(ret_cfg.drhs, key_drhs)
  return ret_cfg


def set_fwd_dequant_mode(cfg: DotGeneral, *, lhs_dequant_mode=None, rhs_dequant_mode=None):
  if lhs_dequant_mode is not None:
    cfg.fwd.lhs.dequant_mode = lhs_dequant_mode
  if rhs_dequant_mode is not None:
    cfg.fwd.rhs.dequant_mode = rhs_dequant_mode


def set_fwd_calibration_mode(cfg: DotGeneral, *, lhs_calibration_mode=SKIP, rhs_calibration_mode=SKIP):
  if lhs_calibration_mode != SKIP:
    cfg.fwd.lhs.calibration_mode = lhs_calibration_mode
  if rhs_calibration_mode != SKIP:
    cfg.fwd.rhs.calibration_mode = rhs_calibration_mode


def set_numerics(cfg: DotGeneralRaw, lhs_numerics: numerics.AqtNumerics,
                 rhs_numerics: numerics.AqtNumerics):
  """config.py:117-137."""
  assert isinstance(cfg.dg_quantizer, aqt_dot_general.DefaultDotGeneralQuantizer)
  cfg.dg_quantizer.lhs.numerics = lhs_numerics
  cfg.dg_quantizer.rhs.numerics = rhs_numerics
  if (lhs_numerics.get_dtype() in dtypes_allowed_for_int32_accum
      and rhs_numerics.get_dtype() in dtypes_allowed_for_int32_accum):
    cfg.dg_accumulator_dtype = utils.int32
  elif (lhs_numerics.get_dtype() in fp8_numerics.fp8_map.values()
        or rhs_numerics.get_dtype() in fp8_numerics.fp8_map.values()):
    cfg.dg_accumulator_dtype = utils.float32
  else:
    cfg.dg_accumulator_dtype = None


def set_fwd_rhs_dtype_int2(cfg: DotGeneral):
  """A special setter for int2 weights (config.py:142-154).  The reference switches the storage
  dtype of the 2-bit weight from int8 to jnp.int2 (an XLA casting limitation keeps it out of
  infer_dtype_from_bits).  torch has no 2-bit dtype: the values stay one per byte in the int8
  container, which holds the same numbers, so this only checks what the reference checks."""
  assert isinstance(cfg.fwd.dg_quantizer.rhs.numerics, int_numerics.IntSymmetric)
  assert cfg.fwd.dg_quantizer.rhs.numerics.bits == 2


def set_accumulator_dtype(cfg: DotGeneral, fwd_dtype, dlhs_dtype, drhs_dtype):
  if fwd_dtype != SKIP:
    cfg.fwd.dg_accumulator_dtype = fwd_dtype
  if dlhs_dtype != SKIP:
    cfg.dlhs.dg_accumulator_dtype = dlhs_dtype
  if drhs_dtype != SKIP:
    cfg.drhs.dg_accumulator_dtype = drhs_dtype


def set_stochastic_rounding(cfg: DotGeneral, vjp_lhs_stochastic_rounding: bool,
                            vjp_rhs_stochastic_rounding: bool, implementation: str,
                            noise_sharing_axes: Sequence[int] = ()):
  """config.py:171-225."""
  noise_implementations = {
      'jax.uniform': stochastic_rounding.JaxUniform(),
      'custom-1': stochastic_rounding.RandomCenteredUniform(),
  }
  assert implementation in noise_implementations, f'{implementation} not supported.'
  if noise_sharing_axes:
    noise_fn = functools.partial(noise_implementations[implementation],
                                 noise_sharing_axes=noise_sharing_axes)
  else:
    noise_fn = noise_implementations[implementation]
  assert isinstance(cfg.dlhs.dg_quantizer, aqt_dot_general.DefaultDotGeneralQuantizer)
  assert isinstance(cfg.drhs.dg_quantizer, aqt_dot_general.DefaultDotGeneralQuantizer)

  def _set(quantizer: aqt_quantizer.Quantizer, is_sr: bool):
    if isinstance(quantizer.numerics, fp8_numerics.Fp8Numerics):
      quantizer.numerics.stochastic_rounding = is_sr
    else:
      quantizer.numerics.noise_fn = noise_fn if is_sr else None

  for dg_quantizer in (cfg.dlhs.dg_quantizer, cfg.drhs.dg_quantizer):
    _set(dg_quantizer.lhs, vjp_lhs_stochastic_rounding)
    _set(dg_quantizer.rhs, vjp_rhs_stochastic_rounding)


def _all_quantizers(cfg: DotGeneral):
  for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
    assert isinstance(raw.dg_quantizer, aqt_dot_general.DefaultDotGeneralQuantizer)
    yield raw.dg_quantizer.lhs
    yield raw.dg_quantizer.rhs


def set_constant_calibration(cfg: DotGeneral, bound: float = 1.0, bias: Optional[float] = None):
  """config.py:228-251."""
  calibration_cls = functools.partial(calibration.ConstantCalibration, bound=bound, bias=bias)
  for q in _all_quantizers(cfg):
    q.calibration = calibration_cls


def set_local_aqt(cfg: DotGeneral, fwd_local_aqt, dlhs_local_aqt, drhs_local_aqt):
  if fwd_local_aqt != SKIP:
    cfg.fwd.local_aqt = fwd_local_aqt
  if dlhs_local_aqt != SKIP:
    cfg.dlhs.local_aqt = dlhs_local_aqt
  if drhs_local_aqt != SKIP:
    cfg.drhs.local_aqt = drhs_local_aqt


def set_use_fwd_quant(cfg: DotGeneral, dlhs_use_fwd_quant, drhs_use_fwd_quant):
  """config.py:268-284."""
  msg = 'use_fwd_quant is incompatible with use_mid_quant right now.'
  for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
    assert raw.dg_quantizer.lhs_mid_alpha is None, msg
    assert raw.dg_quantizer.rhs_mid_alpha is None, msg
  if dlhs_use_fwd_quant != SKIP:
    cfg.dlhs.rhs.use_fwd_quant = dlhs_use_fwd_quant
  if drhs_use_fwd_quant != SKIP:
    cfg.drhs.rhs.use_fwd_quant = drhs_use_fwd_quant


class _MidNumerics(numerics.AqtNumerics):
  """Numerics of the mid-scale quantizers: a bound of 1, values untouched (config.py:308-323)."""

  def get_quant_bound(self):
    return 1.0

  def get_dtype(self):
    assert False, 'Should not request dtype for mid-quantization.'

  def vjp_fwd(self, x, context):
    return x, ()

  def vjp_bwd(self, res, grad):
    assert res == ()
    return grad


def set_use_mid_quant(cfg: DotGeneral, fwd_mid_alpha_both, dlhs_mid_alpha_both, drhs_mid_alpha_both):
  """Enable middle quantization, a variant of SmoothQuant / AWQ (config.py:287-352)."""
  for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
    assert isinstance(raw.dg_quantizer, aqt_dot_general.DefaultDotGeneralQuantizer)
  msg = 'use_fwd_quant is incompatible with use_mid_quant right now.'
  assert not cfg.dlhs.rhs.use_fwd_quant, msg
  assert not cfg.drhs.rhs.use_fwd_quant, msg
  for raw, alpha in ((cfg.fwd, fwd_mid_alpha_both), (cfg.dlhs, dlhs_mid_alpha_both),
                     (cfg.drhs, drhs_mid_alpha_both)):
    if alpha != SKIP:
      raw.dg_quantizer.lhs_mid.numerics = _MidNumerics()
      raw.dg_quantizer.rhs_mid.numerics = _MidNumerics()
      raw.dg_quantizer.lhs_mid.calibration = calibration.AbsMaxCalibration
      raw.dg_quantizer.rhs_mid.calibration = calibration.AbsMaxCalibration
      raw.dg_quantizer.lhs_mid_alpha = alpha
      raw.dg_quantizer.rhs_mid_alpha = alpha


def set_int_numerics_preserve_zero(cfg: DotGeneral, preserve_zero: bool):
  """config.py:355-380."""
  for q in _all_quantizers(cfg):
    if isinstance(q.numerics, int_numerics.IntSymmetric):
      q.numerics.preserve_zero = preserve_zero
      q.numerics.dtype = utils.infer_dtype_from_bits(q.numerics.bits) if preserve_zero else None


def _update_calibration_keywords(quantizer: aqt_quantizer.Quantizer, only_cls=None, **updates):
  calibration_cls = quantizer.calibration
  if calibration_cls is None:
    return False
  keywords = {}
  if isinstance(calibration_cls, functools.partial):
    keywords = dict(calibration_cls.keywords)
    calibration_cls = calibration_cls.func
  if only_cls is not None:
    assert calibration_cls == only_cls, (
        f'clipping_scale is only available in {only_cls.__name__}, while {quantizer.calibration} '
        'is used in current config.')
  keywords.update(updates)
  quantizer.calibration = functools.partial(calibration_cls, **keywords)
  return True


def set_auto_calib_scale(cfg: DotGeneral, auto_clip_search_config: Sequence[float]) -> None:
  """The weight-side (rhs) quantizers search their clipping scale by SNR (config.py:375-410)."""
  for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
    assert isinstance(raw.dg_quantizer, aqt_dot_general.DefaultDotGeneralQuantizer)
    quantizer = raw.dg_quantizer.rhs
    keywords = {}
    if isinstance(quantizer.calibration, functools.partial):
      keywords = dict(quantizer.calibration.keywords)
    keywords.update(auto_clip_search_config=auto_clip_search_config)
    quantizer.calibration = functools.partial(calibration.SnrBasedAutoCalibration, **keywords)


def set_absmax_calib_scale(cfg: DotGeneral, scale: float):
  """config.py:418-460."""
  for q in _all_quantizers(cfg):
    if _update_calibration_keywords(q, calibration.AbsMaxCalibration, clipping_scale=scale):
      if scale < 1.0 and isinstance(q.numerics, int_numerics.IntSymmetric):
        q.numerics.clip_gradient = True


def set_bits(cfg: DotGeneral, fwd_lhs_bit, fwd_rhs_bit, dlhs_lhs_bit, dlhs_rhs_bit, drhs_lhs_bit,
             drhs_rhs_bit) -> DotGeneral:
  """Set quant bits for dot_general; overwrites with AbsMaxCalibration (config.py:463-512)."""
  calibration_cls = calibration.AbsMaxCalibration
  for raw, lb, rb in ((cfg.fwd, fwd_lhs_bit, fwd_rhs_bit), (cfg.dlhs, dlhs_lhs_bit, dlhs_rhs_bit),
                      (cfg.drhs, drhs_lhs_bit, drhs_rhs_bit)):
    set_numerics(raw, numerics_utils.get_numerics(lb), numerics_utils.get_numerics(rb))
    if lb is not None:
      raw.dg_quantizer.lhs.calibration = calibration_cls
    if rb is not None:
      raw.dg_quantizer.rhs.calibration = calibration_cls
  dlhs_use_fwd_quant = False if fwd_rhs_bit is not None else SKIP
  drhs_use_fwd_quant = False if fwd_lhs_bit is not None else SKIP
  set_use_fwd_quant(cfg, dlhs_use_fwd_quant, drhs_use_fwd_quant)
  return cfg


def set_scale_and_bias_dtype(cfg: DotGeneral, dtype):
  """config.py:515-548."""
  for q in _all_quantizers(cfg):
    _update_calibration_keywords(q, dtype=dtype)


def default_unquantized_config() -> DotGeneral:
  """config.py:555-595."""
  def tensor_cfg() -> Tensor:
    return Tensor(use_fwd_quant=False, dequant_mode=DequantMode.OUTPUT,
                  calibration_mode=CalibrationMode.CONTRACTING_AXIS)

  def quantizer() -> aqt_quantizer.Quantizer:
    return aqt_quantizer.Quantizer(numerics=no_numerics.NoNumerics(), calib_shared_axes=None,
                                   scale_stop_grad=True, calibration=None,
                                   context=utils.Context(key=None, train_step=None))

  def dg_raw_cfg(jax_scope_name: str) -> DotGeneralRaw:
    return DotGeneralRaw(
        lhs=tensor_cfg(), rhs=tensor_cfg(),
        dg_quantizer=aqt_dot_general.DefaultDotGeneralQuantizer(
            lhs=quantizer(), rhs=quantizer(), lhs_mid=quantizer(), rhs_mid=quantizer()),
        dg_accumulator_dtype=None, local_aqt=None, jax_scope_name=jax_scope_name)

  return DotGeneral(fwd=dg_raw_cfg('aqt_fwd'), dlhs=dg_raw_cfg('aqt_dlhs'), drhs=dg_raw_cfg('aqt_drhs'))


def fully_quantized(*, fwd_bits=8, bwd_bits=8, use_fwd_quant: bool = True,
                    use_stochastic_rounding: Optional[bool] = True,
                    vjp_lhs_stochastic_rounding: Optional[bool] = None,
                    vjp_rhs_stochastic_rounding: Optional[bool] = None,
                    use_dummy_static_bound: bool = False, dlhs_local_aqt=None,
                    drhs_local_aqt=None) -> DotGeneral:
  """Fully quantized training (config.py:598-658)."""
  cfg = dot_general_make(lhs_bits=fwd_bits, rhs_bits=fwd_bits, bwd_bits=bwd_bits,
                         use_fwd_quant=use_fwd_quant, dlhs_local_aqt=dlhs_local_aqt,
                         drhs_local_aqt=drhs_local_aqt)
  old_style_sr_config = use_stochastic_rounding is not None
  new_style_sr_config_lhs = vjp_lhs_stochastic_rounding is not None
  new_style_sr_config_rhs = vjp_rhs_stochastic_rounding is not None
  assert new_style_sr_config_lhs == new_style_sr_config_rhs, (
      'if you use new style SR config (vjp_xhs_stochastic_rounding), do pass both lhs and rhs '
      'explicitely.')
  assert new_style_sr_config_lhs != old_style_sr_config
  assert not (vjp_lhs_stochastic_rounding and vjp_rhs_stochastic_rounding), (
      'This config is buggy when you set both to True. Contact lew@ or use config_v3')
  if use_stochastic_rounding is True:
    set_stochastic_rounding(cfg, True, True, 'jax.uniform')
  if vjp_lhs_stochastic_rounding is True:
    set_stochastic_rounding(cfg, True, False, 'jax.uniform')
  if vjp_rhs_stochastic_rounding is True:
    set_stochastic_rounding(cfg, False, True, 'jax.uniform')
  if use_dummy_static_bound:
    set_constant_calibration(cfg, 1.0)
  assert cfg.fwd.local_aqt is None, 'local_aqt is not yet supported in fwd.'
  return cfg


def config_v3(*, fwd_bits=8, dlhs_bits=8, drhs_bits=None, use_dummy_static_bound: bool = False,
              rng_type: str = 'jax.uniform', dlhs_local_aqt=None, drhs_local_aqt=None,
              fwd_accumulator_dtype=utils.int32, dlhs_accumulator_dtype=utils.int32,
              drhs_accumulator_dtype=None) -> DotGeneral:
  """config.py:661-721."""
  fwd = dot_general_raw_make(fwd_bits, fwd_bits, jax_scope_name='aqt_fwd', initialize_calibration=False)
  dlhs = dot_general_raw_make(dlhs_bits, dlhs_bits, local_aqt=dlhs_local_aqt,
                              jax_scope_name='aqt_dlhs', initialize_calibration=False)
  drhs = dot_general_raw_make(drhs_bits, drhs_bits, local_aqt=drhs_local_aqt,
                              jax_scope_name='aqt_drhs', initialize_calibration=False)
  cfg = DotGeneral(fwd=fwd, dlhs=dlhs, drhs=drhs)
  cfg.dlhs.rhs.use_fwd_quant = False
  cfg.drhs.rhs.use_fwd_quant = False
  set_stochastic_rounding(cfg, vjp_lhs_stochastic_rounding=True, vjp_rhs_stochastic_rounding=False,
                          implementation=rng_type)
  if use_dummy_static_bound:
    set_constant_calibration(cfg, 1.0)
  set_accumulator_dtype(cfg, fwd_dtype=fwd_accumulator_dtype, dlhs_dtype=dlhs_accumulator_dtype,
                        drhs_dtype=drhs_accumulator_dtype)
  assert cfg.fwd.local_aqt is None, 'local_aqt is not yet supported in fwd.'
  return cfg


def config_v4(*, fwd_bits=8, dlhs_bits=8, drhs_bits=None, use_dummy_static_bound: bool = False,
              rng_type: str = 'jax.uniform', dlhs_local_aqt=None, drhs_local_aqt=None,
              fwd_accumulator_dtype=SKIP, dlhs_accumulator_dtype=SKIP, drhs_accumulator_dtype=SKIP,
              dlhs_use_fwd_quant=SKIP, drhs_use_fwd_quant=SKIP, fwd_mid_alpha_both=SKIP,
              dlhs_mid_alpha_both=SKIP, drhs_mid_alpha_both=SKIP) -> DotGeneral:
  """Version 4 of the user-visible config (config.py:724-788)."""
  cfg = default_unquantized_config()
  set_bits(cfg, fwd_lhs_bit=fwd_bits, fwd_rhs_bit=fwd_bits, dlhs_lhs_bit=dlhs_bits,
           dlhs_rhs_bit=dlhs_bits, drhs_lhs_bit=drhs_bits, drhs_rhs_bit=drhs_bits)
  set_accumulator_dtype(cfg, fwd_dtype=fwd_accumulator_dtype, dlhs_dtype=dlhs_accumulator_dtype,
                        drhs_dtype=drhs_accumulator_dtype)
  set_stochastic_rounding(cfg, vjp_lhs_stochastic_rounding=True, vjp_rhs_stochastic_rounding=False,
                          implementation=rng_type)
  if use_dummy_static_bound:
    set_constant_calibration(cfg, 1.0)
  set_local_aqt(cfg, fwd_local_aqt=SKIP, dlhs_local_aqt=dlhs_local_aqt, drhs_local_aqt=drhs_local_aqt)
  set_use_fwd_quant(cfg, dlhs_use_fwd_quant=dlhs_use_fwd_quant, drhs_use_fwd_quant=drhs_use_fwd_quant)
  set_use_mid_quant(cfg, fwd_mid_alpha_both=fwd_mid_alpha_both,
                    dlhs_mid_alpha_both=dlhs_mid_alpha_both, drhs_mid_alpha_both=drhs_mid_alpha_both)
  assert cfg.fwd.local_aqt is None, 'local_aqt is not yet supported in fwd.'
  return cfg


def config_fwd_fp8(fwd_bits='e4m3') -> DotGeneral:
  """config.py:791-808."""
  assert fwd_bits in fp8_numerics.fp8_map, 'FP8 only supports 4 or 5 exponent bits'
  cfg = config_v4(fwd_bits=8, dlhs_bits=None, drhs_bits=None)
  set_bits(cfg, fwd_lhs_bit=fwd_bits, fwd_rhs_bit=fwd_bits, dlhs_lhs_bit=None, dlhs_rhs_bit=None,
           drhs_lhs_bit=None, drhs_rhs_bit=None)
  set_stochastic_rounding(cfg, False, False, 'jax.uniform')
  assert cfg.fwd.local_aqt is None, 'local_aqt is not yet supported in fwd.'
  return cfg


def set_fwd_calibration(cfg: DotGeneral, calibration_factory) -> DotGeneral:
  """config.py:811-818."""
  assert isinstance(cfg.fwd.dg_quantizer, aqt_dot_general.DefaultDotGeneralQuantizer)
  cfg.fwd.dg_quantizer.lhs.calibration = calibration_factory
  cfg.fwd.dg_quantizer.rhs.calibration = calibration_factory
  return cfg
